"""GPU parity of the decode-step kernels (called through the C ABI) and of the whole decoder step against the
CPU oracle on the same seeded inputs.  Tolerances: fp32 pieces rel-L2 <= 1e-3 (1e-5-ish in practice), bf16
outputs <= 1e-2, logits of a whole step <= 1e-2 with the same greedy token.
"""
import numpy as np
import pytest
import torch

from oracle import chadq_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


@pytest.fixture(scope="module")
def lib():
    from chadslab_amd import _lib

    assert torch.cuda.is_available(), "these tests need the GPU"
    return _lib.load()


def chk(rc, what):
    from chadslab_amd import _lib

    _lib.check(rc, what)


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def bf16_tensor(b):
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16).to(DEV)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def stream():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("d", [32, 96, 2048, 3000])
def test_add_rmsnorm(lib, d):
    r = rng(d)
    res = r.standard_normal(d).astype(np.float32) * 2
    delta = r.standard_normal(d).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(d)).astype(np.float32)
    tr, td, tw = dev(res), dev(delta), dev(w)
    y = torch.zeros(d, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_add_rmsnorm_bf16(tr.data_ptr(), td.data_ptr(), 1, tw.data_ptr(), y.data_ptr(), d, 1e-6, stream()), "norm")
    want_res = res + delta
    assert np.array_equal(tr.cpu().numpy(), want_res)
    want = O.rmsnorm(want_res, w, 1e-6)
    assert O.rel_l2(O.bf16_to_f32(bits(y)), want) < 5e-3  # bf16 rounding of the output
    # delta = NULL leaves the residual alone
    tr2 = dev(res)
    chk(lib.chadq_add_rmsnorm_bf16(tr2.data_ptr(), None, 0, tw.data_ptr(), y.data_ptr(), d, 1e-6, stream()), "norm")
    assert np.array_equal(tr2.cpu().numpy(), res)
    assert O.rel_l2(O.bf16_to_f32(bits(y)), O.rmsnorm(res, w, 1e-6)) < 5e-3


@pytest.mark.parametrize("d,nd", [(2048, 2), (2048, 4), (4096, 4), (3072, 3), (100, 5)])
def test_add_rmsnorm_sums_partial_vectors_in_order(lib, d, nd):
    r = rng(d + nd)
    res = r.standard_normal(d).astype(np.float32)
    delta = r.standard_normal((nd, d)).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(d)).astype(np.float32)
    tr, td, tw = dev(res), dev(delta), dev(w)
    y = torch.zeros(d, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_add_rmsnorm_bf16(tr.data_ptr(), td.data_ptr(), nd, tw.data_ptr(), y.data_ptr(), d, 1e-6, stream()), "norm")
    want = res.copy()
    for j in range(nd):
        want = want + delta[j]  # fp32, in order: the residual must match bit for bit
    assert np.array_equal(tr.cpu().numpy(), want)
    assert O.rel_l2(O.bf16_to_f32(bits(y)), O.rmsnorm(want, w, 1e-6)) < 5e-3


@pytest.mark.parametrize("n,k,ksplit", [(2048, 16384, 4), (2048, 16384, 2), (100, 8192, 2), (33, 4096, 1)])
def test_gemv_splitk_parts(lib, n, k, ksplit):
    r = rng(n + k + ksplit)
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    xb = O.f32_to_bf16(r.standard_normal((1, k)).astype(np.float32))
    tp_, ts, tx = dev(packed), dev(s), bf16_tensor(xb.reshape(-1))
    parts = torch.zeros(ksplit * n, dtype=torch.float32, device=DEV)
    chk(lib.chadq_gemv_i4g32_splitk(tx.data_ptr(), tp_.data_ptr(), ts.data_ptr(), parts.data_ptr(), n, k, ksplit, stream()),
        "splitk")
    got = parts.cpu().numpy().reshape(ksplit, n)
    kp = k // ksplit
    for j in range(ksplit):
        want = O.qgemm_int4g32_f64(xb[:, j * kp:(j + 1) * kp], packed[:, j * kp // 2:(j + 1) * kp // 2], s[:, j * kp // 32:(j + 1) * kp // 32])[0]
        assert O.rel_l2(got[j], want) < 1e-3
    with pytest.raises(ValueError):
        chk(lib.chadq_gemv_i4g32_splitk(tx.data_ptr(), tp_.data_ptr(), ts.data_ptr(), parts.data_ptr(), n, k, 3, stream()), "splitk")


@pytest.mark.parametrize("n,k,nd", [(2560, 2048, 4), (2560, 2048, 0), (100, 512, 1), (9000, 1024, 2), (32768, 2048, 1)])
def test_gemv_addnorm_equals_norm_then_gemv(lib, n, k, nd):
    r = rng(5 * n + k + nd)
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    res = (r.standard_normal(k) * 2).astype(np.float32)
    delta = r.standard_normal((max(nd, 1), k)).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(k)).astype(np.float32)
    tp_, ts, tr, td, tw = dev(packed), dev(s), dev(res), dev(delta), dev(w)
    tro = torch.zeros(k, dtype=torch.float32, device=DEV)
    y = torch.zeros(n, dtype=torch.float32, device=DEV)
    chk(lib.chadq_gemv_i4g32_addnorm(tr.data_ptr(), td.data_ptr() if nd else None, nd, tw.data_ptr(), 1e-6, tro.data_ptr(),
                                     tp_.data_ptr(), ts.data_ptr(), y.data_ptr(), n, k, stream()), "addnorm")
    want_res = res.copy()
    for j in range(nd):
        want_res = want_res + delta[j]
    assert np.array_equal(tro.cpu().numpy(), want_res)      # the residual sum, bit for bit
    assert np.array_equal(tr.cpu().numpy(), res)            # the input residual is left alone
    xb = O.f32_to_bf16(O.rmsnorm(want_res, w, 1e-6))[None, :]
    assert O.rel_l2(y.cpu().numpy(), O.qgemm_int4g32_f64(xb, packed, s)[0]) < 3e-3  # bf16 ties may round the other way
    with pytest.raises(ValueError):
        chk(lib.chadq_gemv_i4g32_addnorm(tr.data_ptr(), None, 0, tw.data_ptr(), 1e-6, tr.data_ptr(), tp_.data_ptr(), ts.data_ptr(),
                                         y.data_ptr(), n, k, stream()), "addnorm")


@pytest.mark.parametrize("f,k,nd", [(16384, 2048, 1), (16384, 2048, 4), (300, 1024, 0), (4096, 256, 2), (4500, 2048, 1), (1, 256, 1)])
def test_gemv_addnorm_geglu_equals_addnorm_then_geglu(lib, f, k, nd):
    # gate+up projection with the GeGLU in its epilogue: rows (2i, 2i+1) = (gate, up) of feature i.  The unfused pair on the
    # GPU - the same projection on the gate-rows-then-up-rows matrix, then chadq_geglu_bf16 - must give the same bits.
    r = rng(11 * f + k + nd)
    u = r.integers(0, 16, (2 * f, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)   # rows 0..f-1 gate, f..2f-1 up
    s = r.lognormal(-5, 0.5, (2 * f, k // 32)).astype(np.float16)
    il = np.arange(2 * f).reshape(2, f).T.reshape(-1)             # interleaved order: g0, u0, g1, u1, ...
    res = (r.standard_normal(k) * 2).astype(np.float32)
    delta = r.standard_normal((max(nd, 1), k)).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(k)).astype(np.float32)
    tp_, ts, tpi, tsi = dev(packed), dev(s), dev(np.ascontiguousarray(packed[il])), dev(np.ascontiguousarray(s[il]))
    tr, td, tw = dev(res), dev(delta), dev(w)
    tro, tro2 = torch.zeros(k, dtype=torch.float32, device=DEV), torch.zeros(k, dtype=torch.float32, device=DEV)
    h = torch.zeros(f, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_gemv_i4g32_addnorm_geglu(tr.data_ptr(), td.data_ptr() if nd else None, nd, tw.data_ptr(), 1e-6, tro.data_ptr(),
                                           tpi.data_ptr(), tsi.data_ptr(), h.data_ptr(), 2 * f, k, stream()), "addnorm geglu")
    gu = torch.zeros(2 * f, dtype=torch.float32, device=DEV)
    h2 = torch.zeros(f, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_gemv_i4g32_addnorm(tr.data_ptr(), td.data_ptr() if nd else None, nd, tw.data_ptr(), 1e-6, tro2.data_ptr(),
                                     tp_.data_ptr(), ts.data_ptr(), gu.data_ptr(), 2 * f, k, stream()), "addnorm")
    chk(lib.chadq_geglu_bf16(gu.data_ptr(), h2.data_ptr(), f, stream()), "geglu")
    assert np.array_equal(tro.cpu().numpy(), tro2.cpu().numpy())
    assert np.array_equal(bits(h), bits(h2))
    # and against the CPU restatement
    want_res = res.copy()
    for j in range(nd):
        want_res = want_res + delta[j]
    xb = O.f32_to_bf16(O.rmsnorm(want_res, w, 1e-6))[None, :]
    y = O.qgemm_int4g32_f64(xb, packed, s)[0]
    want = O.gelu_tanh(y[:f]) * y[f:]
    assert O.rel_l2(O.bf16_to_f32(bits(h)), want) < 6e-3
    with pytest.raises(ValueError):  # an odd number of rows has no pairs
        chk(lib.chadq_gemv_i4g32_addnorm_geglu(tr.data_ptr(), None, 0, tw.data_ptr(), 1e-6, tro.data_ptr(), tpi.data_ptr(),
                                               tsi.data_ptr(), h.data_ptr(), 2 * f - 1, k, stream()), "addnorm geglu")


@pytest.mark.parametrize("n,k,ksplit", [(2048, 16384, 4), (100, 8192, 1)])
def test_gemv_splitk_geglu_equals_geglu_then_gemv(lib, n, k, ksplit):
    r = rng(3 * n + k + ksplit)
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    gu = (r.standard_normal(2 * k) * 2).astype(np.float32)
    tp_, ts, tg = dev(packed), dev(s), dev(gu)
    parts = torch.zeros(ksplit * n, dtype=torch.float32, device=DEV)
    chk(lib.chadq_gemv_i4g32_splitk_geglu(tg.data_ptr(), tp_.data_ptr(), ts.data_ptr(), parts.data_ptr(), n, k, ksplit, stream()),
        "splitk geglu")
    # the unfused pair on the GPU must give the same bits: same GeGLU formula, same GEMV kernel
    h = torch.zeros(k, dtype=torch.bfloat16, device=DEV)
    parts2 = torch.zeros(ksplit * n, dtype=torch.float32, device=DEV)
    chk(lib.chadq_geglu_bf16(tg.data_ptr(), h.data_ptr(), k, stream()), "geglu")
    chk(lib.chadq_gemv_i4g32_splitk(h.data_ptr(), tp_.data_ptr(), ts.data_ptr(), parts2.data_ptr(), n, k, ksplit, stream()), "splitk")
    assert torch.equal(parts, parts2)
    # and the oracle
    hb = O.f32_to_bf16(O.gelu_tanh(gu[:k]) * gu[k:])[None, :]
    want = O.qgemm_int4g32_f64(hb, packed, s)[0]
    assert O.rel_l2(parts.cpu().numpy().reshape(ksplit, n).sum(0), want) < 2e-3


@pytest.mark.parametrize("hq,dh,pos", [(8, 256, 0), (8, 256, 2047), (4, 64, 100), (1, 8, 3)])
def test_rope_kv_write(lib, hq, dh, pos):
    r = rng(hq * 1000 + dh + pos)
    ctx = pos + 5
    qkv = r.standard_normal((hq + 2) * dh).astype(np.float32)
    tq = dev(qkv)
    tp = torch.tensor([pos], dtype=torch.int32, device=DEV)
    q = torch.zeros(hq * dh, dtype=torch.float32, device=DEV)
    kc = torch.zeros(ctx * dh, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(ctx * dh, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_rope_kv_write(tq.data_ptr(), tp.data_ptr(), q.data_ptr(), kc.data_ptr(), vc.data_ptr(), hq, dh, ctx, 10000.0,
                                stream()), "rope")
    want_q = O.rope_rotate_half(qkv[: hq * dh].reshape(hq, dh), pos).reshape(-1)
    want_k = O.rope_rotate_half(qkv[hq * dh: (hq + 1) * dh], pos)
    # fp32 sin/cos of angles up to ~2000 rad: argument rounding alone gives ~1e-4 absolute
    assert np.abs(q.cpu().numpy() - want_q).max() < 2e-3
    kb, vb = bits(kc).reshape(ctx, dh), bits(vc).reshape(ctx, dh)
    assert np.abs(O.bf16_to_f32(kb[pos]) - want_k).max() < 4e-2
    assert np.array_equal(vb[pos], O.f32_to_bf16(qkv[(hq + 1) * dh:]))
    untouched = np.ones(ctx, bool)
    untouched[pos] = False
    assert not kb[untouched].any() and not vb[untouched].any()


def test_rope_position_is_clamped_to_the_cache(lib):
    hq, dh, ctx = 2, 16, 4
    tq = dev(rng(1).standard_normal((hq + 2) * dh).astype(np.float32))
    tp = torch.tensor([1000], dtype=torch.int32, device=DEV)
    q = torch.zeros(hq * dh, dtype=torch.float32, device=DEV)
    guard = torch.zeros((ctx + 4) * dh, dtype=torch.bfloat16, device=DEV)  # 4 rows of canary behind the cache
    vc = torch.zeros((ctx + 4) * dh, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_rope_kv_write(tq.data_ptr(), tp.data_ptr(), q.data_ptr(), guard.data_ptr(), vc.data_ptr(), hq, dh, ctx,
                                10000.0, stream()), "rope")
    torch.cuda.synchronize()
    assert not bits(guard)[ctx * dh:].any() and not bits(vc)[ctx * dh:].any()
    assert bits(vc)[(ctx - 1) * dh: ctx * dh].any()  # landed in the last row


@pytest.mark.parametrize("hq,dh,pos,max_ctx", [(8, 256, 0, 64), (8, 256, 63, 64), (8, 256, 64, 4096), (8, 256, 2047, 4096),
                                               (8, 256, 4095, 4096), (3, 64, 200, 300), (1, 8, 70, 128)])
def test_attn_decode_mqa(lib, hq, dh, pos, max_ctx):
    r = rng(hq + dh + pos)
    q = r.standard_normal(hq * dh).astype(np.float32)
    kc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    vc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    tq, tk, tv = dev(q), bf16_tensor(kc.reshape(-1)), bf16_tensor(vc.reshape(-1))
    tp = torch.tensor([pos], dtype=torch.int32, device=DEV)
    ws = torch.zeros(lib.chadq_attn_decode_mqa_workspace_floats(hq, dh, max_ctx), dtype=torch.float32, device=DEV)
    out = torch.zeros(hq * dh, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_attn_decode_mqa(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), tp.data_ptr(), ws.data_ptr(), out.data_ptr(),
                                  hq, dh, max_ctx, stream()), "attn")
    kk = O.bf16_to_f32(kc[: pos + 1]).astype(np.float64)
    vv = O.bf16_to_f32(vc[: pos + 1]).astype(np.float64)
    s = q.reshape(hq, dh).astype(np.float64) @ kk.T / np.sqrt(dh)
    p = np.exp(s - s.max(-1, keepdims=True))
    want = (p / p.sum(-1, keepdims=True)) @ vv
    assert O.rel_l2(O.bf16_to_f32(bits(out)).reshape(hq, dh), want) < 1e-2


@pytest.mark.parametrize("hq,dh,pos,max_ctx", [(8, 256, 0, 64), (8, 256, 31, 64), (8, 256, 32, 4096), (8, 256, 2047, 4096),
                                               (8, 256, 4095, 4096), (8, 256, 8191, 8192), (3, 64, 200, 300), (1, 16, 70, 128),
                                               (8, 256, 4099, 4100), (8, 256, 77, 4100), (8, 256, 9000, 9001), (2, 256, 100, 130)])
def test_attn_decode_mqa_fused_equals_rope_write_attend(lib, hq, dh, pos, max_ctx):
    r = rng(7 * hq + dh + pos)
    qkv = r.standard_normal((hq + 2) * dh).astype(np.float32)
    kc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    vc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    tq, tk, tv = dev(qkv), bf16_tensor(kc.reshape(-1)), bf16_tensor(vc.reshape(-1))
    tp = torch.tensor([pos], dtype=torch.int32, device=DEV)
    table = torch.zeros(max_ctx * dh, dtype=torch.float32, device=DEV)
    chk(lib.chadq_rope_table(table.data_ptr(), dh, max_ctx, 10000.0, stream()), "table")
    ws = torch.zeros(lib.chadq_attn_decode_mqa_fused_workspace_floats(hq, dh, max_ctx), dtype=torch.float32, device=DEV)
    out = torch.zeros(hq * dh, dtype=torch.bfloat16, device=DEV)
    # oracle: rotate, write the cache row, attend
    q = O.rope_rotate_half(qkv[: hq * dh].reshape(hq, dh), pos)
    kc[pos] = O.f32_to_bf16(O.rope_rotate_half(qkv[hq * dh: (hq + 1) * dh], pos))
    vc[pos] = O.f32_to_bf16(qkv[(hq + 1) * dh:])
    kk = O.bf16_to_f32(kc[: pos + 1]).astype(np.float64)
    vv = O.bf16_to_f32(vc[: pos + 1]).astype(np.float64)
    s = q.astype(np.float64) @ kk.T / np.sqrt(dh)
    pr = np.exp(s - s.max(-1, keepdims=True))
    want = (pr / pr.sum(-1, keepdims=True)) @ vv
    for call in range(2):  # the second call finds the new row already in the cache
        chk(lib.chadq_attn_decode_mqa_fused(tq.data_ptr(), tp.data_ptr(), table.data_ptr(), tk.data_ptr(), tv.data_ptr(),
                                            ws.data_ptr(), out.data_ptr(), hq, dh, max_ctx, stream()), "attn fused")
        torch.cuda.synchronize()
        assert O.rel_l2(O.bf16_to_f32(bits(out)).reshape(hq, dh), want) < 1e-2, "call %d" % call
    kb, vb = bits(tk).reshape(max_ctx, dh), bits(tv).reshape(max_ctx, dh)
    assert np.array_equal(vb, vc)  # V row written exactly, every other row untouched
    assert np.abs(O.bf16_to_f32(kb[pos]) - O.bf16_to_f32(kc[pos])).max() < 4e-2  # fp32 sin/cos of large angles
    rest = np.ones(max_ctx, bool)
    rest[pos] = False
    assert np.array_equal(kb[rest], kc[rest])


@pytest.mark.parametrize("hq,pos,max_ctx,n", [(8, 0, 64, 2048), (8, 31, 64, 2048), (8, 32, 4096, 2048), (8, 2047, 4096, 2048),
                                              (8, 2048, 4096, 2048), (8, 2111, 4096, 2048), (8, 4095, 4096, 2048),
                                              (8, 8191, 8192, 2048), (2, 70, 128, 100), (4, 300, 512, 4100), (6, 129, 256, 65),
                                              (8, 9000, 9001, 2048), (8, 100, 4100, 300)])
def test_attn_fused_oproj_equals_attention_then_projection(lib, hq, pos, max_ctx, n):
    """The output projection with the combination of the attention partials folded in, against (a) the separate calls on the
    GPU - the same bf16 attention vector through the oracle's f64 GEMV, and identical caches - and (b) the oracle end to end."""
    dh, k = 256, hq * 256
    r = rng(11 * hq + pos + n)
    qkv = r.standard_normal((hq + 2) * dh).astype(np.float32)
    kc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    vc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    sc = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    tq, tp = dev(qkv), torch.tensor([pos], dtype=torch.int32, device=DEV)
    tw, ts = dev(packed), dev(sc)
    table = torch.zeros(max_ctx * dh, dtype=torch.float32, device=DEV)
    chk(lib.chadq_rope_table(table.data_ptr(), dh, max_ctx, 10000.0, stream()), "table")
    nws = lib.chadq_attn_decode_mqa_fused_workspace_floats(hq, dh, max_ctx)
    # separate calls
    tk1, tv1 = bf16_tensor(kc.reshape(-1)), bf16_tensor(vc.reshape(-1))
    ws1 = torch.zeros(nws, dtype=torch.float32, device=DEV)
    att = torch.zeros(k, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_attn_decode_mqa_fused(tq.data_ptr(), tp.data_ptr(), table.data_ptr(), tk1.data_ptr(), tv1.data_ptr(),
                                        ws1.data_ptr(), att.data_ptr(), hq, dh, max_ctx, stream()), "attn fused")
    # one call; the workspace starts out full of NaN: slices past the context must never reach a sum
    tk2, tv2 = bf16_tensor(kc.reshape(-1)), bf16_tensor(vc.reshape(-1))
    ws2 = torch.full((nws,), float("nan"), dtype=torch.float32, device=DEV)
    parts = torch.full((hq // 2, n), float("nan"), dtype=torch.float32, device=DEV)
    prev = None
    for call in range(3):  # the later calls find the new row already in the cache
        chk(lib.chadq_attn_decode_mqa_fused_oproj_i4g32(tq.data_ptr(), tp.data_ptr(), table.data_ptr(), tk2.data_ptr(),
                                                        tv2.data_ptr(), ws2.data_ptr(), tw.data_ptr(), ts.data_ptr(),
                                                        parts.data_ptr(), hq, dh, max_ctx, n, stream()), "attn fused oproj")
        torch.cuda.synchronize()
        got = parts.cpu().numpy()
        assert np.isfinite(got).all(), "call %d" % call
        assert np.array_equal(bits(tk2), bits(tk1)) and np.array_equal(bits(tv2), bits(tv1))
        # the two heads of a pair add into one accumulator in whatever order they arrive: the same bits every time
        assert prev is None or np.array_equal(got.view(np.uint32), prev.view(np.uint32)), "call %d" % call
        prev = got.copy()
        # (a) per pair of heads, on the attention vector the separate kernel rounded to bf16: the two combinations may
        # round a value to neighbouring bf16 numbers, nothing more
        ab = bits(att)
        for hp in range(hq // 2):
            xb = np.zeros((1, k), dtype=np.uint16)
            xb[0, hp * 512:(hp + 1) * 512] = ab[hp * 512:(hp + 1) * 512]
            assert O.rel_l2(got[hp], O.qgemm_int4g32_f64(xb, packed, sc)[0]) < 3e-3, "call %d pair %d" % (call, hp)
    # (b) the oracle: rotate, write the cache row, attend, round, project
    q = O.rope_rotate_half(qkv[: hq * dh].reshape(hq, dh), pos)
    kc[pos] = O.f32_to_bf16(O.rope_rotate_half(qkv[hq * dh: (hq + 1) * dh], pos))
    vc[pos] = O.f32_to_bf16(qkv[(hq + 1) * dh:])
    kk = O.bf16_to_f32(kc[: pos + 1]).astype(np.float64)
    vv = O.bf16_to_f32(vc[: pos + 1]).astype(np.float64)
    sco = q.astype(np.float64) @ kk.T / np.sqrt(dh)
    pr = np.exp(sco - sco.max(-1, keepdims=True))
    want_att = ((pr / pr.sum(-1, keepdims=True)) @ vv).astype(np.float32).reshape(1, k)
    want = O.qgemm_int4g32_f64(O.f32_to_bf16(want_att), packed, sc)[0]
    assert O.rel_l2(got.sum(0), want) < 1e-2


def test_attn_fused_oproj_refuses_shapes_it_does_not_cover(lib):
    z = torch.zeros(4096, dtype=torch.float32, device=DEV)
    for hq, dh in ((3, 256), (8, 128), (10, 256), (0, 256)):
        with pytest.raises(ValueError):
            chk(lib.chadq_attn_decode_mqa_fused_oproj_i4g32(z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(),
                                                            z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), hq, dh, 64,
                                                            16, stream()), "attn fused oproj")


@pytest.mark.parametrize("hq,dh,pos,max_ctx", [(8, 256, 40, 4096), (8, 256, 2047, 4096), (8, 256, 0, 64), (4, 64, 40, 200), (8, 256, 40, 16384)])
def test_attn_fused_never_lets_rows_past_the_context_in(lib, hq, dh, pos, max_ctx):
    """Cache rows behind the current position hold NaN: the result must be what it is with zeros there (the kernel for
    8 heads of 256 reads such rows before it knows the position and has to mask them; the general one never reads them)."""
    r = rng(5 * hq + dh + pos)
    qkv = r.standard_normal((hq + 2) * dh).astype(np.float32)
    kc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    vc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    tq, tp = dev(qkv), torch.tensor([pos], dtype=torch.int32, device=DEV)
    table = torch.zeros(max_ctx * dh, dtype=torch.float32, device=DEV)
    chk(lib.chadq_rope_table(table.data_ptr(), dh, max_ctx, 10000.0, stream()), "table")
    outs = []
    for fill in (0x0000, 0x7FC0, 0x7F80):  # zeros, NaN, +inf behind the context
        k2, v2 = kc.copy(), vc.copy()
        k2[pos + 1:] = fill
        v2[pos + 1:] = fill
        tk, tv = bf16_tensor(k2.reshape(-1)), bf16_tensor(v2.reshape(-1))
        ws = torch.zeros(lib.chadq_attn_decode_mqa_fused_workspace_floats(hq, dh, max_ctx), dtype=torch.float32, device=DEV)
        out = torch.zeros(hq * dh, dtype=torch.bfloat16, device=DEV)
        chk(lib.chadq_attn_decode_mqa_fused(tq.data_ptr(), tp.data_ptr(), table.data_ptr(), tk.data_ptr(), tv.data_ptr(),
                                            ws.data_ptr(), out.data_ptr(), hq, dh, max_ctx, stream()), "attn fused")
        torch.cuda.synchronize()
        outs.append(bits(out).copy())
        assert np.array_equal(bits(tk).reshape(max_ctx, dh)[pos + 1:], k2[pos + 1:])  # and never written
    assert np.isfinite(O.bf16_to_f32(outs[0])).all()
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])


def test_rope_table_matches_the_rotation(lib):
    dh, ctx = 64, 300
    table = torch.zeros(ctx * dh, dtype=torch.float32, device=DEV)
    chk(lib.chadq_rope_table(table.data_ptr(), dh, ctx, 10000.0, stream()), "table")
    t = table.cpu().numpy().reshape(ctx, dh // 2, 2)
    ang = np.arange(ctx)[:, None] * (10000.0 ** (-2.0 * np.arange(dh // 2) / dh))[None, :]
    assert np.abs(t[..., 0] - np.cos(ang)).max() < 2e-4 and np.abs(t[..., 1] - np.sin(ang)).max() < 2e-4


def test_attention_random_shapes(lib):
    r = rng(777)
    for _ in range(14):
        hq = int(r.integers(1, 9))
        dh = int(r.choice([16, 32, 48, 64, 96, 128, 160, 256]))
        max_ctx = int(r.integers(40, 3000))
        pos = int(r.integers(0, max_ctx))
        test_attn_decode_mqa_fused_equals_rope_write_attend(lib, hq, dh, pos, max_ctx)
        test_attn_decode_mqa(lib, hq, dh, pos, max_ctx)


def test_gemv_addnorm_and_geglu_random_shapes(lib):
    r = rng(778)
    for _ in range(10):
        k = 256 * int(r.integers(1, 9))
        n = int(r.integers(1, 3000)) if r.random() < 0.7 else int(r.integers(8192, 9000))
        test_gemv_addnorm_equals_norm_then_gemv(lib, n, k, int(r.integers(0, 5)))
    for _ in range(6):
        ksplit = int(r.choice([1, 2, 4]))
        k = 4096 * ksplit * int(r.integers(1, 3))
        test_gemv_splitk_geglu_equals_geglu_then_gemv(lib, int(r.integers(1, 1200)), k, ksplit)


@pytest.mark.parametrize("F", [1, 255, 16384])
def test_geglu(lib, F):
    gu = (rng(F).standard_normal(2 * F) * 3).astype(np.float32)
    t = dev(gu)
    h = torch.zeros(F, dtype=torch.bfloat16, device=DEV)
    chk(lib.chadq_geglu_bf16(t.data_ptr(), h.data_ptr(), F, stream()), "geglu")
    want = O.gelu_tanh(gu[:F]) * gu[F:]
    assert O.rel_l2(O.bf16_to_f32(bits(h)), want) < 5e-3


@pytest.mark.parametrize("n", [1, 7, 256, 70000, 256000])
def test_argmax_and_advance(lib, n):
    v = rng(n).standard_normal(n).astype(np.float32)
    if n > 10:
        v[[3, n - 2]] = v.max() + 1  # a tie: the lower index must win
    t = dev(v)
    scratch = torch.zeros(512, dtype=torch.float32, device=DEV)
    tok = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    pos = torch.tensor([41], dtype=torch.int32, device=DEV)
    chk(lib.chadq_argmax_f32(t.data_ptr(), n, scratch.data_ptr(), tok.data_ptr(), pos.data_ptr(), 1, stream()), "argmax")
    assert int(tok.item()) == int(np.argmax(v)) and int(pos.item()) == 42
    chk(lib.chadq_argmax_f32(t.data_ptr(), n, scratch.data_ptr(), tok.data_ptr(), None, 0, stream()), "argmax")
    assert int(tok.item()) == int(np.argmax(v)) and int(pos.item()) == 42


@pytest.mark.parametrize("n,k", [(256000, 2048), (8192, 256), (9001, 1024), (20000, 2048), (1000, 512), (8192, 4096), (300, 64)])
def test_gemv_argmax_equals_gemv_then_argmax_then_embed(lib, n, k):
    """The output table's GEMV with the argmax candidates in its epilogue and the winner's table row written by the kernel
    that picks it, against the three separate calls: the same logits, token and row, bit for bit - with equal largest
    logits in three different workgroups (the lowest row must win), with NaN activations (token 0) and without the row."""
    r = rng(3 * n + k)
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    sc = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    xb = O.f32_to_bf16(r.standard_normal((1, k)).astype(np.float32))
    tx = bf16_tensor(xb.reshape(-1))
    nscr = lib.chadq_gemv_i4g32_argmax_scratch_bytes(n, k)
    assert nscr >= 2048

    def separate(tp_, ts, txx):
        y = torch.zeros(n, dtype=torch.float32, device=DEV)
        tok = torch.full((1,), -1, dtype=torch.int32, device=DEV)
        scratch = torch.zeros(512, dtype=torch.float32, device=DEV)
        row = torch.zeros(k, dtype=torch.float32, device=DEV)
        chk(lib.chadq_gemv_i4g32(txx.data_ptr(), tp_.data_ptr(), ts.data_ptr(), y.data_ptr(), 1, n, k, stream()), "gemv")
        chk(lib.chadq_argmax_f32(y.data_ptr(), n, scratch.data_ptr(), tok.data_ptr(), None, 0, stream()), "argmax")
        chk(lib.chadq_embed_i4g32(tok.data_ptr(), tp_.data_ptr(), ts.data_ptr(), row.data_ptr(), k, n, stream()), "embed")
        return y.cpu().numpy(), int(tok.item()), row.cpu().numpy()

    def fused(tp_, ts, txx, with_row=True, advance=1):
        y = torch.full((n,), float("nan"), dtype=torch.float32, device=DEV)
        tok = torch.full((1,), -1, dtype=torch.int32, device=DEV)
        pos = torch.tensor([41], dtype=torch.int32, device=DEV)
        scratch = torch.full((nscr // 4,), float("nan"), dtype=torch.float32, device=DEV)
        row = torch.full((k,), float("nan"), dtype=torch.float32, device=DEV)
        chk(lib.chadq_gemv_i4g32_argmax(txx.data_ptr(), tp_.data_ptr(), ts.data_ptr(), y.data_ptr(), n, k, scratch.data_ptr(),
                                        tok.data_ptr(), pos.data_ptr() if advance else None, advance,
                                        row.data_ptr() if with_row else None, stream()), "gemv argmax")
        assert int(pos.item()) == 41 + advance
        return y.cpu().numpy(), int(tok.item()), row.cpu().numpy()

    def same(a, b):
        return np.array_equal(a.view(np.uint32), b.view(np.uint32))

    tp_, ts = dev(packed), dev(sc)
    y0, t0, row0 = separate(tp_, ts, tx)
    y1, t1, row1 = fused(tp_, ts, tx)
    assert O.rel_l2(y0, O.qgemm_int4g32_f64(xb, packed, sc)[0]) < 1e-3
    assert same(y1, y0) and t1 == t0 == int(np.argmax(y0)) and same(row1, row0)
    assert same(row1, ((packed_u(packed[t1]).astype(np.float32) - 8) * np.repeat(sc[t1].astype(np.float32), 32)))
    y2, t2, row2 = fused(tp_, ts, tx, with_row=False, advance=0)
    assert same(y2, y0) and t2 == t0 and np.isnan(row2).all()
    # the winning row copied to an earlier and a later row, far enough apart to sit in other workgroups
    if n >= 300:
        lo, hi = (t0 + n // 3) % n, (t0 + 2 * n // 3) % n
        first = min(lo, hi, t0)
        p2, s2 = packed.copy(), sc.copy()
        p2[[lo, hi]], s2[[lo, hi]] = packed[t0], sc[t0]
        tp2, ts2 = dev(p2), dev(s2)
        ya, ta, rowa = separate(tp2, ts2, tx)
        yb, tb, rowb = fused(tp2, ts2, tx)
        assert ya[lo] == ya[hi] == ya[t0] == ya.max()
        assert same(yb, ya) and ta == tb == first and same(rowb, rowa)
    # NaN activations: every logit NaN, token 0 and its row
    xn = xb.copy()
    xn[0, 5] = 0x7FC0
    yn, tn, rown = fused(tp_, ts, bf16_tensor(xn.reshape(-1)))
    assert np.isnan(yn).all() and tn == 0
    assert same(rown, ((packed_u(packed[0]).astype(np.float32) - 8) * np.repeat(sc[0].astype(np.float32), 32)))


def packed_u(row):
    """The 4-bit values of a packed row, low nibble first."""
    return np.stack([row & 15, row >> 4], axis=-1).reshape(-1)


def _sample_margin(v, k, temperature, u):
    """Distance of u from the nearest interval boundary of the truncated softmax (float64), as a fraction of 1."""
    idx = np.arange(v.size)[~np.isnan(v)]
    order = idx[np.lexsort((idx, -v[idx].astype(np.float64)))][:k]
    c = np.cumsum(np.exp((v[order].astype(np.float64) - float(v[order[0]])) / temperature))
    return float(np.abs(c / c[-1] - u).min())


@pytest.mark.parametrize("n", [5, 300, 256000, 1500000])
def test_argmax_special_values(lib, n):
    # NaN never wins; among equal values (-inf, -0/+0, runs of the maximum) the lowest index; all NaN gives token 0
    r = rng(50 + n)
    scratch = torch.zeros(512, dtype=torch.float32, device=DEV)
    tok = torch.full((1,), -1, dtype=torch.int32, device=DEV)

    def run(v):
        chk(lib.chadq_argmax_f32(dev(v).data_ptr(), n, scratch.data_ptr(), tok.data_ptr(), None, 0, stream()), "argmax")
        return int(tok.item())

    v = r.standard_normal(n).astype(np.float32)
    v[r.integers(0, n, max(1, n // 7))] = np.nan
    assert run(v) == int(np.nanargmax(v))
    v = np.full(n, -np.inf, np.float32)
    v[0] = np.nan
    assert run(v) == (1 if n > 1 else 0)
    v = np.full(n, np.nan, np.float32)
    assert run(v) == 0
    v = np.zeros(n, np.float32)
    v[n // 2:] = -0.0
    v[0] = -1.0
    assert run(v) == 1
    v = (r.integers(0, 3, n)).astype(np.float32)  # long runs of the maximum
    assert run(v) == int(np.argmax(v))


@pytest.mark.parametrize("n,k,temperature", [(256000, 1, 1.0), (256000, 8, 0.7), (256000, 50, 1.0), (256000, 64, 1.3),
                                             (1000, 64, 1.0), (97, 5, 0.5), (5, 5, 1.0), (1, 1, 1.0), (786432, 40, 1.0)])
def test_sample_topk_matches_the_oracle(lib, n, k, temperature):
    r = rng(1000 + n + k)
    v = (r.standard_normal(n) * 3).astype(np.float32)
    if n > 10:
        v[[3, n - 2]] = v.max() + 0.5   # two equal best logits: index 3 comes first
        v[5] = np.nan                   # never a candidate
    t = dev(v)
    ws = torch.zeros(49152 // 4, dtype=torch.float32, device=DEV)
    tok = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    pos = torch.tensor([7], dtype=torch.int32, device=DEV)
    checked = 0
    for u in np.concatenate([[0.0, 0.999999], r.random(30)]).astype(np.float32):
        ud = torch.tensor([u], dtype=torch.float32, device=DEV)
        chk(lib.chadq_sample_topk_f32(t.data_ptr(), n, k, temperature, ud.data_ptr(), ws.data_ptr(), tok.data_ptr(),
                                      pos.data_ptr(), 1, stream()), "sample_topk")
        got = int(tok.item())
        if _sample_margin(v, k, temperature, float(u)) > 1e-5:  # fp32 sums may land on the other side of a boundary
            assert got == O.sample_topk(v, k, temperature, float(u)), (n, k, u)
            checked += 1
        assert 0 <= got < n
    assert checked >= 25 and int(pos.item()) == 7 + 32


@pytest.mark.parametrize("n,k,levels", [(256000, 50, 6), (256000, 64, 3), (5000, 20, 2), (700, 64, 40), (256000, 7, 5), (300, 64, 1)])
def test_sample_topk_with_many_equal_logits(lib, n, k, levels):
    # few distinct values: the k-th best lies inside a run of equal logits, of which the lowest indices are candidates
    r = rng(2000 + n + k)
    v = (r.integers(0, levels, n) * 0.25).astype(np.float32)
    v[r.integers(0, n, 5)] = np.nan
    v[r.integers(0, n, 3)] = -np.inf
    v[n // 2] = -0.0 if levels == 1 else v[n // 2]
    t = dev(v)
    ws = torch.zeros(49152 // 4, dtype=torch.float32, device=DEV)
    tok = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    checked = 0
    for u in np.concatenate([[0.0, 0.999999], r.random(40)]).astype(np.float32):
        ud = torch.tensor([u], dtype=torch.float32, device=DEV)
        chk(lib.chadq_sample_topk_f32(t.data_ptr(), n, k, 1.0, ud.data_ptr(), ws.data_ptr(), tok.data_ptr(), None, 0, stream()),
            "sample_topk")
        if _sample_margin(v, k, 1.0, float(u)) > 1e-5:
            assert int(tok.item()) == O.sample_topk(v, k, 1.0, float(u)), (n, k, levels, u)
            checked += 1
    assert checked >= 30


def test_sample_topk_rejects_bad_arguments(lib):
    t = dev(np.zeros(100, np.float32))
    ws = torch.zeros(49152 // 4, dtype=torch.float32, device=DEV)
    tok = torch.zeros(1, dtype=torch.int32, device=DEV)
    u = torch.zeros(1, dtype=torch.float32, device=DEV)
    for n, k, temp in [(100, 0, 1.0), (100, 65, 1.0), (10, 11, 1.0), (100, 5, 0.0), (786433, 5, 1.0)]:
        assert lib.chadq_sample_topk_f32(t.data_ptr(), n, k, temp, u.data_ptr(), ws.data_ptr(), tok.data_ptr(), None, 0, stream()) != 0
    assert lib.chadq_sample_topk_f32(t.data_ptr(), 100, 5, 1.0, None, ws.data_ptr(), tok.data_ptr(), None, 0, stream()) != 0


def test_embed_row(lib):
    V, d = 50, 96
    p, s = O.quantize_int4_g32(rng(9).standard_normal((V, d)).astype(np.float32))
    tp_, ts = dev(p), dev(s)
    x = torch.zeros(d, dtype=torch.float32, device=DEV)
    for token in (0, 17, 49, 10 ** 6, -3):  # the last two are clamped into the table
        tt = torch.tensor([token], dtype=torch.int32, device=DEV)
        chk(lib.chadq_embed_i4g32(tt.data_ptr(), tp_.data_ptr(), ts.data_ptr(), x.data_ptr(), d, V, stream()), "embed")
        row = min(max(token, 0), V - 1)
        assert np.array_equal(x.cpu().numpy(), O.dequant_int4g32(p[row: row + 1], s[row: row + 1])[0])


# ---------------------------------------------------------------------------------------------- whole step
def _model(seed, cfg):
    r = rng(seed)

    def q(n, k):
        return O.quantize_int4_g32((r.standard_normal((n, k)) * 0.05).astype(np.float32))

    def norm():
        return (1 + 0.1 * r.standard_normal(cfg.d)).astype(np.float32)

    layers = [{"ln1": norm(), "wqkv": q((cfg.hq + 2) * cfg.dh, cfg.d), "wo": q(cfg.d, cfg.hq * cfg.dh), "ln2": norm(),
               "wgu": q(2 * cfg.ffn, cfg.d), "wd": q(cfg.d, cfg.ffn)} for _ in range(cfg.n_layers)]
    return {"layers": layers, "lnf": norm(), "emb": q(cfg.vocab, cfg.d)}


def _upload(m):
    from chadslab_amd import QWeightInt4G32

    def qw(ps):
        return QWeightInt4G32(dev(ps[0]), dev(ps[1]))

    return {"layers": [{k: (qw(v) if isinstance(v, tuple) else dev(v)) for k, v in L.items()} for L in m["layers"]],
            "lnf": dev(m["lnf"]), "emb": qw(m["emb"])}


def _run_steps(cfg, seed, pos0, nsteps, use_graph):
    from chadslab_amd.decoder import QuantDecoder

    m = _model(seed, cfg)
    dec = QuantDecoder(cfg, _upload(m), DEV)
    r = rng(seed + 1)
    kc = [O.f32_to_bf16(r.standard_normal((cfg.max_ctx, cfg.dh)).astype(np.float32)) for _ in range(cfg.n_layers)]
    vc = [O.f32_to_bf16(r.standard_normal((cfg.max_ctx, cfg.dh)).astype(np.float32)) for _ in range(cfg.n_layers)]
    for li in range(cfg.n_layers):
        dec.kcache[li].copy_(bf16_tensor(kc[li].reshape(-1)))
        dec.vcache[li].copy_(bf16_tensor(vc[li].reshape(-1)))
    tok = 5
    dec.token.fill_(tok)
    dec.pos.fill_(pos0)
    if use_graph:
        dec.capture()
    for step in range(nsteps):
        want = O.decode_step(m, tok, pos0 + step, kc, vc, cfg.hq, cfg.dh, cfg.eps, cfg.rope_base)
        if use_graph:
            dec.graph.replay()
        else:
            dec.step()
        torch.cuda.synchronize()
        got = dec.logits.cpu().numpy()
        assert O.rel_l2(got, want) < 1e-2, "step %d" % step
        assert int(dec.pos.item()) == pos0 + step + 1
        gtok = int(dec.token.item())
        assert gtok == int(np.argmax(got))
        # the greedy token must agree unless the oracle's top two logits are closer than the tolerance allows
        top2 = np.sort(want)[-2:]
        if top2[1] - top2[0] > 2e-2 * np.abs(want).max():
            assert gtok == int(np.argmax(want)), "step %d" % step
        # the caches must have received this step's row in every layer
        for li in (0, cfg.n_layers - 1):
            row = bits(dec.kcache[li]).reshape(cfg.max_ctx, cfg.dh)[pos0 + step]
            assert O.rel_l2(O.bf16_to_f32(row), O.bf16_to_f32(kc[li][pos0 + step])) < 2e-2
        tok = gtok
        if gtok != int(np.argmax(want)):
            break  # sequences diverge legitimately after a near-tie


def test_decoder_step_small_eager():
    from chadslab_amd.decoder import DecoderConfig

    _run_steps(DecoderConfig(n_layers=2, d=512, hq=4, dh=64, ffn=1024, vocab=1000, max_ctx=256), 40, 100, 4, False)


def test_decoder_step_small_graph_replay():
    from chadslab_amd.decoder import DecoderConfig

    _run_steps(DecoderConfig(n_layers=2, d=512, hq=4, dh=64, ffn=1024, vocab=1000, max_ctx=256), 41, 60, 5, True)


def test_decoder_sampling_eager_and_graph_draw_the_same_tokens():
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder

    cfg = DecoderConfig(n_layers=2, d=512, hq=4, dh=64, ffn=1024, vocab=1000, max_ctx=256)
    m = _upload(_model(46, cfg))
    runs = []
    for use_graph, top_k in ((False, 20), (True, 20), (False, 0), (False, 1)):
        dec = QuantDecoder(cfg, m, DEV)
        dec.set_sampling(top_k=top_k, temperature=1.5, seed=1234)
        if use_graph:
            dec.capture()
            with pytest.raises(RuntimeError):
                dec.set_sampling(top_k=0)
        runs.append(dec.generate(5, 0, 24))
    sampled, replayed, greedy, top1 = runs
    assert sampled == replayed  # same seed, same draws, whether the step is launched or replayed
    assert top1 == greedy       # k = 1 is argmax
    assert all(0 <= t < cfg.vocab for t in sampled) and sampled != greedy


def test_decoder_feed_then_generate_continues_the_same_sequence():
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder

    cfg = DecoderConfig(n_layers=2, d=512, hq=4, dh=64, ffn=1024, vocab=1000, max_ctx=256)
    m = _upload(_model(47, cfg))
    a = QuantDecoder(cfg, m, DEV)
    seq = a.generate(5, 0, 12)           # 5 -> seq[0] -> seq[1] ...
    b = QuantDecoder(cfg, m, DEV)
    b.capture()
    nxt = b.feed([5] + seq[:6], 0)       # teacher-forced over the first seven tokens
    assert nxt == seq[6] and int(b.pos.item()) == 7
    assert b.generate(nxt, 7, 5) == seq[7:12]


@pytest.mark.parametrize("layers,steps", [(2, 4), (3, 3), (2, 1)])
def test_decoder_graph_of_several_steps_produces_the_same_tokens(layers, steps):
    """A graph that holds several consecutive steps (tokens handed on through a ring in device memory) against the same
    steps launched one by one; also a token count that is not a multiple of the graph's, and feed() beside such a graph."""
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder

    cfg = DecoderConfig(n_layers=layers, d=512, hq=4, dh=64, ffn=1024, vocab=1000, max_ctx=256)
    m = _upload(_model(48, cfg))
    a = QuantDecoder(cfg, m, DEV)
    seq = a.generate(5, 0, 20)
    b = QuantDecoder(cfg, m, DEV)
    b.capture(steps)
    assert b.generate(5, 0, 14) == seq[:14]     # 14 = full replays plus a remainder of single steps
    assert int(b.pos.item()) == 14
    nxt = b.feed([5] + seq[:6], 0)               # feed sets the token before every step: one step at a time
    assert nxt == seq[6] and int(b.pos.item()) == 7
    assert b.generate(nxt, 7, 2 * steps) == seq[7:7 + 2 * steps]
    with pytest.raises(ValueError):
        b.capture(0)


@pytest.mark.parametrize("layers", [2, 3])
def test_decoder_greedy_step_hands_the_next_row_on(layers):
    """A greedy step's last kernel writes the table row of the token it chose where the next step starts from: a step
    without its own embedding launch must then give the same bits as one with it, eagerly and from a graph (which holds
    no embedding launch), also after the token was set by hand (set_state / embed_token)."""
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder

    cfg = DecoderConfig(n_layers=layers, d=512, hq=4, dh=64, ffn=1024, vocab=1000, max_ctx=64)
    m = _upload(_model(49, cfg))
    a, b, c = QuantDecoder(cfg, m, DEV), QuantDecoder(cfg, m, DEV), QuantDecoder(cfg, m, DEV)
    for d in (a, b, c):
        d.set_state(9, 3)
    c.capture()  # (its warm-up run writes cache row 3 as the first replay will)
    logits = []
    for d, run in ((a, lambda: a.step()), (b, lambda: b.step(embed=False)), (c, lambda: c.graph.replay())):
        seq = []
        for _ in range(3):
            run()
            seq.append((d.logits.cpu().numpy().copy(), int(d.token.item()), int(d.pos.item())))
        logits.append(seq)
    for other in logits[1:]:
        for (la, ta, pa), (lo, to, po) in zip(logits[0], other):
            assert np.array_equal(la, lo) and ta == to and pa == po
    # a token written by hand needs its row fetched before a step that does not fetch it
    for d in (a, c):
        d.token.fill_(77)
        d.pos.fill_(10)
    a.step()
    c.embed_token()
    c.graph.replay()
    assert np.array_equal(a.logits.cpu().numpy(), c.logits.cpu().numpy()) and int(a.token.item()) == int(c.token.item())
    with pytest.raises(ValueError):
        a.set_state(cfg.vocab, 0)


def test_decoder_step_odd_layer_count_graph_replay():
    from chadslab_amd.decoder import DecoderConfig

    # three layers: the residual stream's two buffers end a step swapped; the captured graph must not care
    _run_steps(DecoderConfig(n_layers=3, d=256, hq=2, dh=64, ffn=512, vocab=500, max_ctx=128), 44, 50, 4, True)


def test_decoder_step_odd_sizes_generic_gemv():
    from chadslab_amd.decoder import DecoderConfig

    # d and ffn that are not multiples of 256 send every GEMV down the generic kernel
    _run_steps(DecoderConfig(n_layers=1, d=96, hq=2, dh=32, ffn=160, vocab=77, max_ctx=80), 42, 70, 3, False)


def test_decoder_step_gemma_shapes_two_layers():
    from chadslab_amd.decoder import DecoderConfig

    # the benchmark's layer shapes (d 2048, 8 query heads x 256, 1 KV head, FFN 16384) at context 2048
    _run_steps(DecoderConfig(n_layers=2, d=2048, hq=8, dh=256, ffn=16384, vocab=8192, max_ctx=2304), 43, 2047, 2, True)


def test_decoder_step_config4_full_size_graph_replay():
    """The benchmark's whole decode step at its full shape: 18 layers, d 2048, 8 x 256 query heads on one KV head,
    FFN 16384, vocabulary 256000, caches filled to context 2048, weights quantised on the device from N(0, 0.02)
    (what bench.py times).

    An 18-layer random-weight network amplifies rounding differences: two CPU restatements that differ only in the
    precision of the GEMV sums (fp32 against float64, same bf16 rounding points) end 8.8e-3 apart in the logits
    (2.0e-3 after two layers; tests/test_decode_rounding_growth.py reproduces both figures on the CPU), so an end-to-end
    bound of 1e-2 separates nothing at this depth.  The check is
    therefore made where it is sharp: every layer of the GPU step is compared with the oracle's layer applied to the
    same input (the residual vector the GPU step itself had there), the logits with the oracle's output projection of
    the GPU's final residual vector; the graph-replayed step must then reproduce the eager one bit for bit; the
    end-to-end figure is held to a loose bound and the greedy token to the oracle's unless its top two are close."""
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder, random_weights

    cfg = DecoderConfig(max_ctx=2304)
    assert (cfg.n_layers, cfg.d, cfg.hq, cfg.dh, cfg.ffn, cfg.vocab) == (18, 2048, 8, 256, 16384, 256000)
    w = random_weights(cfg, 4004, DEV)
    dec = QuantDecoder(cfg, w, DEV)

    def host(qw):
        return (qw.packed.cpu().numpy(), qw.scale.cpu().numpy())

    m = {"layers": [{k: (host(v) if hasattr(v, "packed") else v.cpu().numpy()) for k, v in L.items()} for L in w["layers"]],
         "lnf": w["lnf"].cpu().numpy(), "emb": host(w["emb"])}
    r = rng(4005)
    pos0, tok = 2047, 123456
    kc = [O.f32_to_bf16(r.standard_normal((cfg.max_ctx, cfg.dh)).astype(np.float32)) for _ in range(cfg.n_layers)]
    vc = [O.f32_to_bf16(r.standard_normal((cfg.max_ctx, cfg.dh)).astype(np.float32)) for _ in range(cfg.n_layers)]

    def fill():
        for li in range(cfg.n_layers):
            dec.kcache[li].copy_(bf16_tensor(kc[li].reshape(-1)))
            dec.vcache[li].copy_(bf16_tensor(vc[li].reshape(-1)))
        dec.token.fill_(tok)
        dec.pos.fill_(pos0)

    # ---- eager step with the residual vector recorded at every layer boundary
    fill()
    trace = []
    print("config 4 full size: eager traced step, token %d, position %d" % (tok, pos0), flush=True)
    dec.step(trace)
    torch.cuda.synchronize()
    assert len(trace) == cfg.n_layers + 1
    xs = [t.cpu().numpy() for t in trace]
    eager_logits, eager_tok = dec.logits.cpu().numpy().copy(), int(dec.token.item())
    ep, es = m["emb"]
    assert np.array_equal(xs[0], O.dequant_int4g32(ep[tok: tok + 1], es[tok: tok + 1])[0])  # the embedding row, exact
    worst = 0.0
    for li, L in enumerate(m["layers"]):
        kl, vl = kc[li].copy(), vc[li].copy()
        want_x = O.decode_layer(L, xs[li], pos0, kl, vl, cfg.hq, cfg.dh, cfg.eps, cfg.rope_base)
        err = O.rel_l2(xs[li + 1] - xs[li], want_x - xs[li])  # what the layer added to the residual stream
        worst = max(worst, err)
        assert err < 5e-3, "layer %d: rel-L2 %.3e of the layer's contribution" % (li, err)
        assert O.rel_l2(xs[li + 1], want_x) < 3e-3, "layer %d residual" % li
        krow = bits(dec.kcache[li]).reshape(cfg.max_ctx, cfg.dh)[pos0]
        vrow = bits(dec.vcache[li]).reshape(cfg.max_ctx, cfg.dh)[pos0]
        assert O.rel_l2(O.bf16_to_f32(krow), O.bf16_to_f32(kl[pos0])) < 1e-2, "layer %d K row" % li
        assert O.rel_l2(O.bf16_to_f32(vrow), O.bf16_to_f32(vl[pos0])) < 1e-2, "layer %d V row" % li
    print("worst per-layer rel-L2 of a layer's contribution: %.3e" % worst, flush=True)
    want_logits = O.decode_logits(m, xs[-1], cfg.eps)
    assert eager_logits.shape == (256000,) and np.isfinite(eager_logits).all()
    assert O.rel_l2(eager_logits, want_logits) < 2e-3, "output projection: %.3e" % O.rel_l2(eager_logits, want_logits)
    assert eager_tok == int(np.argmax(eager_logits))

    # ---- the same step replayed from a captured graph: same kernels, same inputs, same bits
    fill()
    dec.capture()
    dec.graph.replay()
    torch.cuda.synchronize()
    assert np.array_equal(dec.logits.cpu().numpy(), eager_logits)
    assert int(dec.token.item()) == eager_tok and int(dec.pos.item()) == pos0 + 1

    # ---- end to end against the oracle's own step (loose for the reason given above), then a second replayed step
    kc2, vc2 = [a.copy() for a in kc], [a.copy() for a in vc]
    want = O.decode_step(m, tok, pos0, kc2, vc2, cfg.hq, cfg.dh, cfg.eps, cfg.rope_base)
    e2e = O.rel_l2(eager_logits, want)
    print("end-to-end rel-L2 of the logits against the oracle's own 18-layer step: %.3e" % e2e, flush=True)
    assert e2e < 2e-2   # measured 1.4e-2; two CPU restatements differ by 8.8e-3 here (tests/test_decode_rounding_growth.py)
    top2 = np.sort(want)[-2:]
    if top2[1] - top2[0] > 2.0 * np.abs(eager_logits - want).max():  # the oracle's winner leads by more than the logits differ
        assert eager_tok == int(np.argmax(want))
    dec.graph.replay()  # position 2048 with the token the first step chose
    torch.cuda.synchronize()
    want2 = O.decode_step(m, eager_tok, pos0 + 1, kc2, vc2, cfg.hq, cfg.dh, cfg.eps, cfg.rope_base)
    got2 = dec.logits.cpu().numpy()
    assert int(dec.pos.item()) == pos0 + 2 and np.isfinite(got2).all()
    assert O.rel_l2(got2, want2) < 2.5e-2, "second step: %.3e" % O.rel_l2(got2, want2)


def test_decoder_refuses_positions_past_the_cache_and_tokens_outside_the_table():
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder

    cfg = DecoderConfig(n_layers=1, d=256, hq=2, dh=64, ffn=512, vocab=300, max_ctx=16)
    dec = QuantDecoder(cfg, _upload(_model(48, cfg)), DEV)
    assert len(dec.generate(5, 10, 6)) == 6          # positions 10..15: the last rows of the cache
    with pytest.raises(ValueError):
        dec.generate(5, 10, 7)                        # would need row 16
    with pytest.raises(ValueError):
        dec.feed([1, 2, 3], 14)
    with pytest.raises(ValueError):
        dec.feed([1, 300], 0)                         # token outside [0, vocab)
    with pytest.raises(ValueError):
        dec.generate(-1, 0, 1)

"""Pins the CPU oracle (oracle/chadq_oracle.py and its scalar C twin) WITHOUT a GPU.

The reference snapshot holds no golden vector, known-answer test or fixture for this path, so each oracle
function is pinned by what the mathematics fixes: exhaustive enumeration, brute force on tiny inputs, special
cases with exact answers, library routines (torch bf16 rounding, torch matmul, scipy softmax, torch silu),
int64 arithmetic, and the independent C twin.  Every check is chosen so that a plausible slip (swapped nibble,
wrong zero point, scale indexed by the wrong group, transposed operand) fails it.
"""
import os

import numpy as np
import pytest
import scipy.special
import torch

from oracle import build_oracle as B
from oracle import chadq_oracle as O
from ctypes import c_double, c_float, c_int8, c_int32, c_uint8, c_uint16

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


# ------------------------------------------------------------------ pack / unpack
def test_unpack_every_byte_value():
    wp = np.arange(256, dtype=np.uint8)[None, :]
    q = O.unpack_int4(wp)[0]
    for b in range(256):
        assert q[2 * b] == (b & 15) - 8       # low nibble first
        assert q[2 * b + 1] == (b >> 4) - 8   # high nibble second


def test_pack_every_nibble_pair():
    lo, hi = np.meshgrid(np.arange(-8, 8), np.arange(-8, 8), indexing="ij")
    q = np.stack([lo.ravel(), hi.ravel()], axis=1).astype(np.int8)  # 256 rows of (k=0, k=1)
    wp = O.pack_int4(q)
    assert wp.shape == (256, 1)
    for (a, b), byte in zip(q, wp[:, 0]):
        assert int(byte) == ((int(a) + 8) | ((int(b) + 8) << 4))
    assert np.array_equal(O.unpack_int4(wp), q)
    assert len(set(wp[:, 0].tolist())) == 256  # a bijection onto bytes


def test_pack_hand_written_fixture():
    q = np.array([[-8, 7, 0, -1, 1, -2, 3, 4, -3, 5, -4, 6, 2, -5, -6, -7]], dtype=np.int8)
    expect = np.array([[0xF0, 0x78, 0x69, 0xCB, 0xD5, 0xE4, 0x3A, 0x12]], dtype=np.uint8)
    assert np.array_equal(O.pack_int4(q), expect)
    assert np.array_equal(O.unpack_int4(expect), q)


def test_pack_roundtrip_random_and_range_check():
    q = rng(1).integers(-8, 8, (37, 96), dtype=np.int8)
    assert np.array_equal(O.unpack_int4(O.pack_int4(q)), q)
    with pytest.raises(ValueError):
        O.pack_int4(np.array([[8, 0]], dtype=np.int8))
    with pytest.raises(ValueError):
        O.pack_int4(np.zeros((2, 3), dtype=np.int8))


def test_c_twin_pack_unpack(oracle_c):
    wp = rng(2).integers(0, 256, 1000, dtype=np.uint8)
    q = np.empty(2000, dtype=np.int8)
    oracle_c.oracle_unpack_i4(B.ptr(wp, c_uint8), B.ptr(q, c_int8), wp.size)
    assert np.array_equal(q, O.unpack_int4(wp[None])[0])
    back = np.empty_like(wp)
    oracle_c.oracle_pack_i4(B.ptr(q, c_int8), B.ptr(back, c_uint8), wp.size)
    assert np.array_equal(back, wp)


# ------------------------------------------------------------------ bf16 / fp16
def test_bf16_rounding_matches_torch():
    r = rng(3)
    vals = np.concatenate([
        r.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** r.integers(-30, 30, 20000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, np.inf, -np.inf, 3.4e38, 1e-45, 1e-40, 65504.0], dtype=np.float32),
        # exact ties: bf16 value + half an ulp, for even and odd last bits
        (np.arange(0x3F80, 0x3FA0, dtype=np.uint32) << 16 | 0x8000).astype(np.uint32).view(np.float32),
        (np.arange(0x0001, 0x0020, dtype=np.uint32) << 16 | 0x8000).astype(np.uint32).view(np.float32),  # denormals
    ]).astype(np.float32)
    ours = O.f32_to_bf16(vals)
    theirs = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, theirs)
    assert np.array_equal(O.bf16_to_f32(ours), torch.from_numpy(theirs.view(np.int16)).view(torch.bfloat16).float().numpy())
    nan = O.f32_to_bf16(np.array([np.nan], dtype=np.float32))
    assert np.isnan(O.bf16_to_f32(nan))[0]


def test_c_twin_bf16_and_f16(oracle_c):
    vals = (rng(4).standard_normal(5000) * 100).astype(np.float32)
    out = np.empty(vals.size, dtype=np.uint16)
    oracle_c.oracle_f32_to_bf16(B.ptr(vals, c_float), B.ptr(out, c_uint16), vals.size)
    assert np.array_equal(out, O.f32_to_bf16(vals))
    allh = np.arange(65536, dtype=np.uint16)
    f = np.empty(65536, dtype=np.float32)
    oracle_c.oracle_f16_to_f32(B.ptr(allh, c_uint16), B.ptr(f, c_float), 65536)
    ref = allh.view(np.float16).astype(np.float32)
    both_nan = np.isnan(f) & np.isnan(ref)
    assert np.array_equal(f[~both_nan], ref[~both_nan]) and (np.isnan(f) == np.isnan(ref)).all()


# ------------------------------------------------------------------ dequant
def test_dequant_int4_triple_loop():
    r = rng(5)
    n, k = 4, 64
    q = r.integers(-8, 8, (n, k), dtype=np.int8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    d = O.dequant_int4g32(O.pack_int4(q), s)
    for i in range(n):
        for g in range(k // 32):
            for j in range(32):
                assert d[i, g * 32 + j] == np.float32(int(q[i, g * 32 + j])) * np.float32(s[i, g])


def test_dequant_int4_special_cases():
    n, k = 3, 96
    s = rng(6).lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    zeros = np.full((n, k // 2), 0x88, dtype=np.uint8)  # every nibble = zero point
    assert np.array_equal(O.dequant_int4g32(zeros, s), np.zeros((n, k), np.float32))
    ones = np.ones((n, k // 32), dtype=np.float16)
    q = rng(7).integers(-8, 8, (n, k), dtype=np.int8)
    assert np.array_equal(O.dequant_int4g32(O.pack_int4(q), ones), q.astype(np.float32))
    # a one-hot activation picks out one dequantised column
    d = O.dequant_int4g32(O.pack_int4(q), s)
    for kk in (0, 31, 32, 95):
        x = np.zeros((1, k), dtype=np.float32)
        x[0, kk] = 1.0
        assert np.array_equal(O.qgemv_int4g32(O.f32_to_bf16(x), O.pack_int4(q), s)[0], d[:, kk])
    with pytest.raises(ValueError):
        O.dequant_int4g32(O.pack_int4(q), s[:, :2])


def test_dequant_int8():
    r = rng(8)
    w = r.integers(-127, 128, (5, 17), dtype=np.int8)
    s = r.uniform(0.001, 0.02, 5).astype(np.float32)
    d = O.dequant_int8(w, s)
    for i in range(5):
        for j in range(17):
            assert d[i, j] == np.float32(int(w[i, j])) * s[i]


# ------------------------------------------------------------------ integer accumulation is exact
def test_integer_accumulation_exact(oracle_c):
    r = rng(9)
    m, n, k = 3, 24, 4096
    q = r.integers(-8, 8, (n, k), dtype=np.int8)
    packed = O.pack_int4(q)
    ones = np.ones((n, k // 32), dtype=np.float16)
    xi = r.integers(-8, 9, (m, k))
    xb = O.f32_to_bf16(xi.astype(np.float32))
    brute = xi.astype(np.int64) @ q.astype(np.int64).T
    assert np.abs(brute).max() < 2 ** 24
    assert np.array_equal(O.qgemv_int4g32(xb, packed, ones).astype(np.int64), brute)
    assert np.array_equal(O.qgemm_int4g32_f64(xb, packed, ones).astype(np.int64), brute)
    yc = np.empty((m, n), dtype=np.float32)
    oracle_c.oracle_gemm_i4g32_f32(B.ptr(xb, c_uint16), B.ptr(packed, c_uint8), B.ptr(ones.view(np.uint16), c_uint16),
                                   B.ptr(yc, c_float), m, n, k)
    assert np.array_equal(yc.astype(np.int64), brute)


# ------------------------------------------------------------------ float products
def _i4_case(seed, m, n, k):
    r = rng(seed)
    q = r.integers(-8, 8, (n, k), dtype=np.int8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    x = O.f32_to_bf16(r.standard_normal((m, k)).astype(np.float32))
    return q, O.pack_int4(q), s, x


def test_qgemv_int4_against_brute_force_and_torch(oracle_c):
    m, n, k = 4, 48, 256
    q, packed, s, x = _i4_case(10, m, n, k)
    xf = O.bf16_to_f32(x).astype(np.float64)
    sf = s.astype(np.float64)
    brute = np.einsum("mgk,ngk,ng->mn", xf.reshape(m, k // 32, 32), q.astype(np.float64).reshape(n, k // 32, 32), sf)
    y64 = O.qgemm_int4g32_f64(x, packed, s)
    assert O.rel_l2(y64, brute) < 1e-14
    assert O.rel_l2(O.qgemv_int4g32(x, packed, s), brute) < 1e-6
    t = torch.matmul(torch.from_numpy(O.bf16_to_f32(x)), torch.from_numpy(O.dequant_int4g32(packed, s)).T).numpy()
    assert O.rel_l2(t, brute) < 1e-6
    yc = np.empty((m, n), dtype=np.float64)
    oracle_c.oracle_gemm_i4g32_f64(B.ptr(x, c_uint16), B.ptr(packed, c_uint8), B.ptr(s.view(np.uint16), c_uint16),
                                   B.ptr(yc, c_double), m, n, k)
    assert O.rel_l2(yc, brute) < 1e-14
    # bf16 output is the RNE rounding of the fp32 result
    yb = O.qgemm_int4g32_bf16(x, packed, s)
    assert O.rel_l2(O.bf16_to_f32(yb), brute) < 4e-3


def test_qgemv_int4_linearity_and_row_independence():
    m, n, k = 2, 32, 128
    q, packed, s, _ = _i4_case(11, m, n, k)
    r = rng(12)
    a = r.integers(-64, 64, (1, k)).astype(np.float32)  # integers: a+b exact in bf16 range
    b = r.integers(-64, 64, (1, k)).astype(np.float32)
    ya = O.qgemm_int4g32_f64(O.f32_to_bf16(a), packed, s)
    yb = O.qgemm_int4g32_f64(O.f32_to_bf16(b), packed, s)
    yab = O.qgemm_int4g32_f64(O.f32_to_bf16(a + b), packed, s)
    assert O.rel_l2(yab, ya + yb) < 1e-13
    both = O.qgemm_int4g32_f64(O.f32_to_bf16(np.concatenate([a, b])), packed, s)
    assert np.array_equal(both[0:1], ya) and np.array_equal(both[1:2], yb)


def test_qgemv_int8_against_brute_force(oracle_c):
    r = rng(13)
    m, n, k = 2, 40, 160
    w = r.integers(-127, 128, (n, k), dtype=np.int8)
    s = r.uniform(0.001, 0.02, n).astype(np.float32)
    x = r.standard_normal((m, k)).astype(np.float32)
    brute = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            brute[i, j] = float(s[j]) * sum(float(x[i, t]) * int(w[j, t]) for t in range(k))
    assert O.rel_l2(O.qgemv_int8_f64(x, w, s), brute) < 1e-13
    assert O.rel_l2(O.qgemv_int8(x, w, s), brute) < 1e-6
    yc = np.empty((m, n), dtype=np.float64)
    oracle_c.oracle_gemm_i8row_f64(B.ptr(x, c_float), B.ptr(w, c_int8), B.ptr(s, c_float), B.ptr(yc, c_double), m, n, k)
    assert O.rel_l2(yc, brute) < 1e-13
    xb = O.f32_to_bf16(x)
    assert O.rel_l2(O.bf16_to_f32(O.qgemm_int8_bf16(xb, w, s)), O.qgemm_int8_f64(xb, w, s)) < 4e-3


# ------------------------------------------------------------------ router / silu / MoE
def test_softmax_and_route(oracle_c):
    r = rng(14)
    logits = r.standard_normal((64, 8)).astype(np.float32)
    assert np.allclose(O.softmax(logits), scipy.special.softmax(logits.astype(np.float64), axis=-1), rtol=1e-6, atol=1e-7)
    idx, w = O.moe_route(logits, 2, True)
    order = np.argsort(-scipy.special.softmax(logits.astype(np.float64), axis=-1), axis=-1, kind="stable")[:, :2]
    assert np.array_equal(idx, order)
    assert np.allclose(w.sum(-1), 1.0, atol=1e-6) and (w[:, 0] >= w[:, 1]).all()
    _, w_raw = O.moe_route(logits, 2, False)
    assert np.allclose(w_raw, np.take_along_axis(O.softmax(logits), idx, -1)) and (w_raw.sum(-1) < 1).all()
    ic = np.empty((64, 2), dtype=np.int32)
    wc = np.empty((64, 2), dtype=np.float32)
    oracle_c.oracle_moe_route(B.ptr(logits, c_float), B.ptr(ic, c_int32), B.ptr(wc, c_float), 64, 8, 2, 1)
    assert np.array_equal(ic, idx) and np.allclose(wc, w, rtol=1e-5)


def test_route_ties_go_to_lower_index(oracle_c):
    logits = np.array([[1.0, 3.0, 3.0, 0.0], [2.0, 2.0, 2.0, 2.0], [0.0, 1.0, 5.0, 5.0]], dtype=np.float32)
    idx, _ = O.moe_route(logits, 2, True)
    assert idx.tolist() == [[1, 2], [0, 1], [2, 3]]
    ic = np.empty((3, 2), dtype=np.int32)
    wc = np.empty((3, 2), dtype=np.float32)
    oracle_c.oracle_moe_route(B.ptr(logits, c_float), B.ptr(ic, c_int32), B.ptr(wc, c_float), 3, 4, 2, 1)
    assert ic.tolist() == idx.tolist()


def test_silu_matches_torch(oracle_c):
    x = np.linspace(-20, 20, 4001, dtype=np.float32)
    assert np.allclose(O.silu(x), torch.nn.functional.silu(torch.from_numpy(x)).numpy(), rtol=2e-6, atol=1e-7)
    out = np.empty_like(x)
    oracle_c.oracle_silu(B.ptr(x, c_float), B.ptr(out, c_float), x.size)
    assert np.allclose(out, O.silu(x), rtol=2e-6, atol=1e-7)


def _experts(seed, e, h, f):
    r = rng(seed)
    out = []
    for _ in range(e):
        ws = []
        for shape in ((f, h), (f, h), (h, f)):
            ws += list(O.quantize_int4_g32((r.standard_normal(shape) * 0.05).astype(np.float32)))
        out.append(tuple(ws))
    return out


def test_moe_equals_masked_dense_sum():
    t, h, f, e = 12, 64, 96, 4
    experts = _experts(15, e, h, f)
    r = rng(16)
    x = O.f32_to_bf16(r.standard_normal((t, h)).astype(np.float32))
    logits = r.standard_normal((t, e)).astype(np.float32)
    idx, w = O.moe_route(logits, 2, True)
    dense = np.zeros((t, h), dtype=np.float64)
    for ei, (gp, gs, up, us, dp, ds) in enumerate(experts):
        g = O.qgemv_int4g32(x, gp, gs)
        u = O.qgemv_int4g32(x, up, us)
        hm = O.f32_to_bf16(O.silu(g) * u)
        d = O.qgemv_int4g32(hm, dp, ds)
        gate = np.where(idx == ei, w, 0).sum(-1)  # routing weight of this expert per token (0 if not selected)
        dense += gate[:, None].astype(np.float64) * d
    y = O.bf16_to_f32(O.moe_qffn(x, logits, experts, 2, True))
    assert O.rel_l2(y, dense) < 4e-3  # one bf16 rounding of the result
    # permutation of the tokens permutes the output
    perm = r.permutation(t)
    yp = O.moe_qffn(x[perm], logits[perm], experts, 2, True)
    assert np.array_equal(yp, O.moe_qffn(x, logits, experts, 2, True)[perm])


def test_moe_single_expert_is_a_plain_gated_ffn():
    t, h, f = 5, 64, 64
    experts = _experts(17, 1, h, f)
    x = O.f32_to_bf16(rng(18).standard_normal((t, h)).astype(np.float32))
    logits = np.zeros((t, 1), dtype=np.float32)
    gp, gs, up, us, dp, ds = experts[0]
    hm = O.f32_to_bf16(O.silu(O.qgemv_int4g32(x, gp, gs)) * O.qgemv_int4g32(x, up, us))
    plain = O.f32_to_bf16(O.qgemv_int4g32(hm, dp, ds))
    assert np.array_equal(O.moe_qffn(x, logits, experts, 1, True), plain)


# ------------------------------------------------------------------ quantisers
def test_quantizers_invert_within_half_a_step():
    w = (rng(19).standard_normal((16, 128)) * 0.1).astype(np.float32)
    p, s = O.quantize_int4_g32(w)
    assert np.allclose(s.astype(np.float32), np.abs(w.reshape(16, 4, 32)).max(-1) / 7, rtol=1e-3)
    err = np.abs(O.dequant_int4g32(p, s) - w)
    assert (err <= 0.5 * np.repeat(s.astype(np.float32), 32, 1) * 1.01 + 1e-9).all()
    q8, s8 = O.quantize_int8_row(w)
    assert (np.abs(O.dequant_int8(q8, s8) - w) <= 0.5 * s8[:, None] * 1.0001 + 1e-9).all()
    assert np.abs(q8).max() == 127


# ------------------------------------------------------------------ frozen fixtures
def test_golden_fixtures_reproduce():
    g = np.load(os.path.join(GOLD, "i4g32_n64_k128.npz"))
    assert np.array_equal(O.pack_int4(g["q"]), g["packed"])
    assert np.array_equal(O.dequant_int4g32(g["packed"], g["scale"]), g["dequant"])
    assert np.array_equal(O.qgemm_int4g32_f64(g["x_bf16"], g["packed"], g["scale"]), g["y_f64"])
    assert np.array_equal(O.qgemm_int4g32_bf16(g["x_bf16"], g["packed"], g["scale"]), g["y_bf16"])
    g8 = np.load(os.path.join(GOLD, "i8row_n64_k128.npz"))
    assert np.array_equal(O.qgemv_int8_f64(g8["x_f32"], g8["w"], g8["scale"]), g8["y_f64"])
    assert np.array_equal(O.qgemm_int8_bf16(g8["x_bf16"], g8["w"], g8["scale"]), g8["yb_bf16"])
    gm = np.load(os.path.join(GOLD, "moe_t16_h64_f96_e4.npz"))
    idx, w = O.moe_route(gm["logits"], 2, True)
    assert np.array_equal(idx, gm["idx"]) and np.array_equal(w, gm["w"])
    experts = [tuple(gm["e%d_%s_%s" % (i, n, t)] for n in "gud" for t in "ps") for i in range(4)]
    assert np.array_equal(O.moe_qffn(gm["x_bf16"], gm["logits"], experts, 2, True), gm["y_bf16"])


# ------------------------------------------------------------------ decode step
def _tiny_model(seed, n_layers, d, hq, dh, ffn, vocab):
    r = rng(seed)

    def q(n, k):
        return O.quantize_int4_g32((r.standard_normal((n, k)) * 0.05).astype(np.float32))

    layers = [{"ln1": (1 + 0.1 * r.standard_normal(d)).astype(np.float32), "wqkv": q((hq + 2) * dh, d), "wo": q(d, hq * dh),
               "ln2": (1 + 0.1 * r.standard_normal(d)).astype(np.float32), "wgu": q(2 * ffn, d), "wd": q(d, ffn)}
              for _ in range(n_layers)]
    return {"layers": layers, "lnf": (1 + 0.1 * r.standard_normal(d)).astype(np.float32), "emb": q(vocab, d)}


def test_decode_pieces_against_torch():
    r = rng(30)
    x = r.standard_normal(96).astype(np.float32) * 3
    w = r.standard_normal(96).astype(np.float32)
    t = torch.from_numpy(x)
    ref = t * torch.rsqrt(t.pow(2).mean() + 1e-6) * torch.from_numpy(w)
    assert np.allclose(O.rmsnorm(x, w, 1e-6), ref.numpy(), rtol=1e-5, atol=1e-6)
    g = r.standard_normal(1000).astype(np.float32) * 3
    assert np.allclose(O.gelu_tanh(g), torch.nn.functional.gelu(torch.from_numpy(g), approximate="tanh").numpy(), rtol=1e-5, atol=1e-6)
    # rotate-half RoPE as a complex rotation of (v[j], v[j+half])
    v = r.standard_normal((3, 64)).astype(np.float32)
    pos, half = 77, 32
    ang = pos * (10000.0 ** (-2.0 * np.arange(half) / 64))
    z = (v[:, :half] + 1j * v[:, half:]) * np.exp(1j * ang)
    assert np.allclose(O.rope_rotate_half(v, pos), np.concatenate([z.real, z.imag], -1), rtol=1e-4, atol=1e-4)
    assert np.allclose(O.rope_rotate_half(v, 0), v)  # position 0 is the identity
    assert np.allclose(np.linalg.norm(O.rope_rotate_half(v, 1234), axis=-1), np.linalg.norm(v, axis=-1), rtol=1e-5)


def test_decode_step_against_independent_torch_model():
    n_layers, d, hq, dh, ffn, vocab, ctx = 2, 128, 2, 32, 256, 300, 40
    m = _tiny_model(31, n_layers, d, hq, dh, ffn, vocab)
    r = rng(32)
    pos0 = 17
    kc = [O.f32_to_bf16(r.standard_normal((ctx, dh)).astype(np.float32)) for _ in range(n_layers)]
    vc = [O.f32_to_bf16(r.standard_normal((ctx, dh)).astype(np.float32)) for _ in range(n_layers)]
    kc_t = [torch.from_numpy(O.bf16_to_f32(a).copy()) for a in kc]
    vc_t = [torch.from_numpy(O.bf16_to_f32(a).copy()) for a in vc]

    def bf(t):  # round a torch fp32 tensor to bf16 and back
        return t.to(torch.bfloat16).to(torch.float32)

    def deq(pw):
        return torch.from_numpy(O.dequant_int4g32(*pw))

    def torch_step(token, pos):
        x = deq(m["emb"])[token].clone()
        for li, L in enumerate(m["layers"]):
            xn = bf(x * torch.rsqrt(x.pow(2).mean() + 1e-6) * torch.from_numpy(L["ln1"]))
            qkv = deq(L["wqkv"]) @ xn
            inv = 10000.0 ** (-2.0 * torch.arange(dh // 2, dtype=torch.float64) / dh)
            rot = torch.polar(torch.ones(dh // 2, dtype=torch.float64), pos * inv)

            def rope(vv):
                zc = torch.complex(vv[..., : dh // 2].double(), vv[..., dh // 2:].double()) * rot
                return torch.cat([zc.real, zc.imag], -1).float()

            q = rope(qkv[: hq * dh].reshape(hq, dh))
            kc_t[li][pos] = bf(rope(qkv[hq * dh: (hq + 1) * dh]))
            vc_t[li][pos] = bf(qkv[(hq + 1) * dh:])
            p = torch.softmax(q @ kc_t[li][: pos + 1].T / dh ** 0.5, dim=-1)
            att = bf((p @ vc_t[li][: pos + 1]).reshape(-1))
            x = x + deq(L["wo"]) @ att
            xn = bf(x * torch.rsqrt(x.pow(2).mean() + 1e-6) * torch.from_numpy(L["ln2"]))
            gu = deq(L["wgu"]) @ xn
            h = bf(torch.nn.functional.gelu(gu[:ffn], approximate="tanh") * gu[ffn:])
            x = x + deq(L["wd"]) @ h
        xn = bf(x * torch.rsqrt(x.pow(2).mean() + 1e-6) * torch.from_numpy(m["lnf"]))
        return (deq(m["emb"]) @ xn).numpy()

    tok = 5
    for step in range(3):
        lo = O.decode_step(m, tok, pos0 + step, kc, vc, hq, dh)
        lt = torch_step(tok, pos0 + step)
        assert O.rel_l2(lo, lt) < 2e-3  # both round through bf16 at the same places; fp32 summation orders differ
        assert int(lo.argmax()) == int(lt.argmax())
        tok = int(lo.argmax())


def test_sample_topk_special_cases():
    r = np.random.Generator(np.random.PCG64(77))
    for _ in range(20):  # k = 1 is argmax with the lowest index among equals, whatever u and temperature are
        v = r.integers(-3, 4, 50).astype(np.float32)
        assert O.sample_topk(v, 1, 0.3, r.random()) == int(np.argmax(v))
    v = np.array([1.0, 3.0, 3.0, 2.0], np.float32)  # equal logits: the lower index comes first and has the same weight
    assert O.sample_topk(v, 2, 1.0, 0.0) == 1 and O.sample_topk(v, 2, 1.0, 0.49) == 1
    assert O.sample_topk(v, 2, 1.0, 0.51) == 2 and O.sample_topk(v, 2, 1.0, 0.999) == 2
    assert O.sample_topk(np.array([np.nan, 1.0, np.nan, 5.0]), 3, 1.0, 0.0) == 3  # NaN is never a candidate
    assert O.sample_topk(np.array([np.nan, np.nan]), 2, 1.0, 0.5) == 0
    assert O.sample_topk(np.array([-np.inf, -np.inf, -np.inf]), 2, 1.0, 0.9) == 0
    assert O.sample_topk(np.array([0.0, 100.0, 0.0]), 3, 0.01, 0.999999) == 1  # a cold temperature is greedy


def test_sample_topk_draws_the_truncated_softmax():
    from scipy.special import softmax

    r = np.random.Generator(np.random.PCG64(78))
    v = r.standard_normal(12).astype(np.float32) * 2
    k, temperature, draws = 5, 0.7, 20000
    top = torch.topk(torch.from_numpy(v), k).indices.numpy()  # independent selection of the candidates
    want = softmax(v[top].astype(np.float64) / temperature)
    counts = np.zeros(12)
    for j in range(draws):
        counts[O.sample_topk(v, k, temperature, (j + 0.5) / draws)] += 1
    assert counts.sum() == draws and set(np.nonzero(counts)[0]) <= set(top.tolist())
    assert np.abs(counts[top] / draws - want).max() <= 1.5 / draws  # a uniform grid of u hits each interval to +-1



# ------------------------------------------------------------------ tile order (a layout of this build)
def _tile_loops(wp, sc_u16):
    """The layout written out address by address, without numpy reshapes: unit (band, 256 k) of 4096 bytes, a group's
    32 rows next to each other; scale block of 512 bytes, per row the even groups' scales, 256 bytes on the odd ones'."""
    n, kh = wp.shape
    k = kh * 2
    wt = np.zeros(n * kh, np.uint8)
    st = np.zeros(n * (k // 32), np.uint16)
    for row in range(n):
        b, r = divmod(row, 32)
        for g in range(k // 32):                      # 16 packed bytes = one scale group
            c, g8 = divmod(g, 8)
            dst = (b * (k // 256) + c) * 4096 + (g8 * 32 + r) * 16
            wt[dst:dst + 16] = wp[row, g * 16:(g + 1) * 16]
            dsts = ((b * (k // 256) + c) * 512 + ((g8 % 2) * 32 + r) * 8 + (g8 // 2) * 2) // 2
            st[dsts] = sc_u16[row, g]
    return wt.reshape(n, kh), st.reshape(n, k // 32)


@pytest.mark.parametrize("n,k", [(32, 256), (64, 512), (96, 768)])
def test_tile_order_against_address_loops_and_round_trip(n, k):
    r = np.random.default_rng(600 + n + k)
    wp = r.integers(0, 256, (n, k // 2), dtype=np.uint8)
    sc = r.integers(0, 65536, (n, k // 32), dtype=np.uint16)
    wt, st = O.tile_int4g32(wp, sc.view(np.float16))
    wl, sl = _tile_loops(wp, sc)
    assert np.array_equal(wt, wl) and np.array_equal(st.view(np.uint16), sl)
    a, b = O.untile_int4g32(wt, st)
    assert np.array_equal(a, wp) and np.array_equal(b.view(np.uint16), sc)


def test_tile_order_hand_placed_bytes_and_bijection():
    n, k = 64, 512
    # every byte carries its own address, so the tiled array is the permutation itself
    wp = np.arange(n * k // 2, dtype=np.uint32)
    tag = (wp % 251).astype(np.uint8).reshape(n, k // 2)
    wt, _ = O.tile_int4g32(tag, np.zeros((n, k // 32), np.float16))
    # row 37 (band 1, r = 5), scale group 14 (unit 1, group 6 of it), byte 3 of the group
    src = 37 * (k // 2) + 14 * 16 + 3
    dst = (1 * (k // 256) + 1) * 4096 + (6 * 32 + 5) * 16 + 3
    assert wt.reshape(-1)[dst] == src % 251
    # row 0, group 0 stays at the very start; row 31, group 0 ends the first 512 bytes; row 0, group 1 follows it
    assert wt.reshape(-1)[0] == tag[0, 0] and wt.reshape(-1)[31 * 16 + 5] == tag[31, 5] and wt.reshape(-1)[512 + 2] == tag[0, 16 + 2]
    idx = np.arange(n * k // 2, dtype=np.int64)
    lo, hi = (idx & 0xFF).astype(np.uint8).reshape(n, -1), (idx >> 8).astype(np.uint8).reshape(n, -1)
    perm = O.tile_int4g32(lo, np.zeros((n, k // 32), np.float16))[0].astype(np.int64) + \
        (O.tile_int4g32(hi, np.zeros((n, k // 32), np.float16))[0].astype(np.int64) << 8)
    assert np.array_equal(np.sort(perm.reshape(-1)), idx)  # a bijection: every byte appears exactly once
    s = np.arange(n * k // 32, dtype=np.uint16).reshape(n, k // 32)
    st = O.tile_int4g32(np.zeros((n, k // 2), np.uint8), s.view(np.float16))[1].view(np.uint16).reshape(-1)
    assert np.array_equal(np.sort(st), s.reshape(-1))
    # row 40 (band 1, r = 8), unit 1: its even groups' scales at (3 * 512 + 8 * 8) / 2, the odd ones' 128 entries on
    at = (3 * 512 + 8 * 8) // 2
    assert np.array_equal(st[at:at + 4], s[40, 8:16:2]) and np.array_equal(st[at + 128:at + 132], s[40, 9:16:2])


def test_tile_order_refuses_shapes_it_cannot_tile():
    for n, k in ((48, 256), (32, 128), (32, 288)):
        with pytest.raises(ValueError):
            O.tile_int4g32(np.zeros((n, k // 2), np.uint8), np.zeros((n, k // 32), np.float16))

"""The decode attention entry point that allocates nothing (chadq_attn_decode_mqa_fused_static: the split-context
partials live in a device array inside the library) against chadq_attn_decode_mqa_fused with a caller's workspace:
same kernels, so the outputs and the cache rows written must agree bit for bit.  Two calls in a row, the second on a
smaller problem (fewer heads, narrower heads, a shorter context), so that what the first call left in the shared
array lies beyond what the second one writes and must not leak into its result.
"""
import numpy as np
import pytest
import torch

from oracle import chadq_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(lib, seed, hq, dh, pos, max_ctx):
    from chadslab_amd import _lib

    r = np.random.Generator(np.random.PCG64(seed))
    s = torch.cuda.current_stream().cuda_stream
    qkv = torch.from_numpy(r.standard_normal((hq + 2) * dh).astype(np.float32)).to(DEV)
    kc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))
    vc = O.f32_to_bf16(r.standard_normal((max_ctx, dh)).astype(np.float32))

    def cache(b):
        return torch.from_numpy(b.reshape(-1).view(np.int16)).view(torch.bfloat16).to(DEV)

    tp = torch.tensor([pos], dtype=torch.int32, device=DEV)
    table = torch.zeros(max_ctx * dh, dtype=torch.float32, device=DEV)
    _lib.check(lib.chadq_rope_table(table.data_ptr(), dh, max_ctx, 10000.0, s), "table")
    # existing entry point, caller's workspace
    k1, v1 = cache(kc), cache(vc)
    ws = torch.zeros(lib.chadq_attn_decode_mqa_fused_workspace_floats(hq, dh, max_ctx), dtype=torch.float32, device=DEV)
    want = torch.zeros(hq * dh, dtype=torch.bfloat16, device=DEV)
    _lib.check(lib.chadq_attn_decode_mqa_fused(qkv.data_ptr(), tp.data_ptr(), table.data_ptr(), k1.data_ptr(), v1.data_ptr(),
                                               ws.data_ptr(), want.data_ptr(), hq, dh, max_ctx, s), "fused")
    # the one that allocates nothing; torch's allocator must not be asked for anything during the call
    k2, v2 = cache(kc), cache(vc)
    got = torch.zeros(hq * dh, dtype=torch.bfloat16, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    _lib.check(lib.chadq_attn_decode_mqa_fused_static(qkv.data_ptr(), tp.data_ptr(), table.data_ptr(), k2.data_ptr(),
                                                      v2.data_ptr(), got.data_ptr(), hq, dh, max_ctx, s), "fused static")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before

    def bits(t):
        return t.view(torch.int16).cpu().numpy()

    assert np.array_equal(bits(got), bits(want)), "hq=%d dh=%d pos=%d max_ctx=%d" % (hq, dh, pos, max_ctx)
    assert np.array_equal(bits(k2), bits(k1)) and np.array_equal(bits(v2), bits(v1))
    # and the result is the attention it claims to be (f64 softmax attention over the updated cache)
    q = O.rope_rotate_half(qkv.cpu().numpy()[: hq * dh].reshape(hq, dh), pos)
    kk = O.bf16_to_f32(k2.view(torch.int16).cpu().numpy().view(np.uint16).reshape(max_ctx, dh)[: pos + 1]).astype(np.float64)
    vv = O.bf16_to_f32(v2.view(torch.int16).cpu().numpy().view(np.uint16).reshape(max_ctx, dh)[: pos + 1]).astype(np.float64)
    sc = q.astype(np.float64) @ kk.T / np.sqrt(dh)
    p = np.exp(sc - sc.max(-1, keepdims=True))
    ref = (p / p.sum(-1, keepdims=True)) @ vv
    assert O.rel_l2(O.bf16_to_f32(got.view(torch.int16).cpu().numpy().view(np.uint16)).reshape(hq, dh), ref) < 1e-2


def test_static_scratch_attention_equals_workspace_attention_twice():
    from chadslab_amd import _lib

    lib = _lib.load()
    assert torch.cuda.is_available()
    print("case 1: hq=8 dh=256 pos=8191 max_ctx=8192 (the scratch's full size)", flush=True)
    _case(lib, 11, 8, 256, 8191, 8192)
    print("case 2: hq=3 dh=64 pos=200 max_ctx=300 (smaller, right after)", flush=True)
    _case(lib, 12, 3, 64, 200, 300)
    print("case 3: hq=8 dh=256 pos=2047 max_ctx=4096 (the decode step's shape)", flush=True)
    _case(lib, 13, 8, 256, 2047, 4096)


def test_static_scratch_attention_rejects_a_cache_beyond_its_scratch():
    from chadslab_amd import _lib

    lib = _lib.load()
    z = torch.zeros(64, dtype=torch.float32, device=DEV)
    rc = lib.chadq_attn_decode_mqa_fused_static(z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(),
                                                8, 256, 8193, None)
    assert rc == -4 and b"8192" in lib.chadq_last_error()

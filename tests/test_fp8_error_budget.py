"""Why the prefill GEMM keeps bf16 operands: the error budget of an fp8 (e4m3) dequantisation target, measured on
the CPU so that the decision can be re-derived from the tree.

gfx950's fp8 matrix instruction takes both operands in 8 bits or fewer.  Emulated here, at the benchmark's own
distributions (x ~ N(0,1) rounded to bf16; 4-bit weights with fp16 group scales ~ LogNormal(-5, 0.5)) against the
float64 product:
  * activations rounded to e4m3 (per-row scale into its range)          -> rel-L2 about 2.7e-2
  * weights (u-8)*scale rounded to e4m3 (what an fp8 B operand holds)   -> rel-L2 about 2.7e-2
both above the 1e-2 the benchmark allows a bf16 output, while
  * the shipped form (bf16 activations, weights rounded to bf16)        -> about 1.7e-3
  * activations split into two e4m3 terms (two MFMAs instead of one)    -> about 7e-4, which meets the bound but
    spends the factor of two the fp8 instruction gains, and still needs the group scale outside the operand:
    the integers u-8 are exact in e4m3, the fp16 scales are not powers of two (the hardware's block scales are).
The e4m3 rounding is written out in numpy and pinned against torch's float8_e4m3fn cast.
"""
import numpy as np
import torch

from oracle import chadq_oracle as O


def e4m3_round(v):
    """float32 -> nearest e4m3fn value (4 exponent bits, bias 7, 3 mantissa bits, max 448, subnormal step 2^-9), ties to
    even, saturating; returned as float32."""
    v = np.asarray(v, dtype=np.float32)
    a = np.minimum(np.abs(v).astype(np.float64), 448.0)
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -20)))
    e = np.clip(e, -6, 8)                      # exponent of the binade; below 2^-6 the subnormal step applies
    step = 2.0 ** (e - 3)
    q = np.rint(a / step) * step               # np.rint: ties to even
    return (np.sign(v) * np.minimum(q, 448.0)).astype(np.float32)


def test_e4m3_rounding_matches_torch():
    r = np.random.Generator(np.random.PCG64(5))
    v = np.concatenate([r.standard_normal(20000).astype(np.float32) * s for s in (1e-3, 0.05, 1.0, 30.0, 200.0)])
    v = np.concatenate([v, np.array([0.0, 448.0, -448.0, 2.0 ** -9, 2.0 ** -10, 0.4375, 0.46875, 17.0, 18.0, 19.0], np.float32)])
    v = v[np.abs(v) <= 448.0]  # torch's cast turns what lies beyond the range into NaN; the study never leaves it
    want = torch.from_numpy(v).to(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(e4m3_round(v), want)


def test_fp8_operands_miss_the_tolerance_that_bf16_operands_meet():
    r = np.random.Generator(np.random.PCG64(1002))
    m, n, k = 64, 1024, 4096
    x = O.bf16_to_f32(O.f32_to_bf16(r.standard_normal((m, k)).astype(np.float32)))
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    w = O.dequant_int4g32(packed, s)
    truth = x.astype(np.float64) @ w.astype(np.float64).T

    def err(xa, wa):
        return O.rel_l2(xa.astype(np.float64) @ wa.astype(np.float64).T, truth)

    # shipped: weights rounded to bf16 for the matrix core
    wb = O.bf16_to_f32(O.f32_to_bf16(w))
    shipped = err(x, wb)
    # e4m3 activations, scaled per row so that the row's largest value sits at the top of the range
    sc = np.abs(x).max(1, keepdims=True) / 448.0
    x8 = e4m3_round(x / sc) * sc
    act8 = err(x8, w)
    # e4m3 weights with the group scale folded in (scaled by 64 into the normal range; exact power of two)
    w8 = e4m3_round(w * 64.0) / 64.0
    wt8 = err(x, w8)
    # two e4m3 terms for the activations
    rem = x - x8
    sc2 = np.maximum(np.abs(rem).max(1, keepdims=True), 1e-30) / 448.0
    two = err(x8 + e4m3_round(rem / sc2) * sc2, w)
    print("shipped bf16 %.2e | x e4m3 %.2e | w e4m3 %.2e | x as two e4m3 terms %.2e" % (shipped, act8, wt8, two))
    assert shipped < 4e-3                      # measured 1.7e-3
    assert 2.0e-2 < act8 < 3.5e-2              # measured 2.7e-2: fails the 1e-2 bound
    assert 2.0e-2 < wt8 < 3.5e-2               # measured 2.7e-2: fails the 1e-2 bound
    assert two < 4e-3                          # measured 6.7e-4: meets it, at the price of the second MFMA
    # the integer part of a weight is exact in e4m3; it is the fp16 scale that does not fit an fp8 operand
    ints = np.arange(-8, 8, dtype=np.float32)
    assert np.array_equal(e4m3_round(ints), ints)
    sf = s.astype(np.float32)
    assert np.mean(e4m3_round(sf * 4096.0) / 4096.0 != sf) > 0.8

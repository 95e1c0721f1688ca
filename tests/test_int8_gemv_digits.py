"""The fixed-point digit arithmetic of the int8 matrix-core GEMV (chadslab_amd/csrc/gemv_i8row_mfma.hip, stage_x),
restated in numpy and checked exhaustively on the CPU: the kernel's parity tests show that its results are right, these
show why - every integer the kernel can form is split into three int8 digits that put it back together exactly."""
import numpy as np

MAGIC = np.float32(12582912.0)  # 1.5 * 2^23: x + MAGIC holds rint(x) in its mantissa as 0x400000 + rint(x)


def digits_of(t):
    """t: float32 values already multiplied by the block's power-of-two scale, |t| <= 2^21.  The kernel's three
    instructions: one FMA onto MAGIC, an add of 0x408080 and an XOR with 0x808080; the low three bytes are a2, a1, a0."""
    bits = (t.astype(np.float32) + MAGIC).view(np.uint32)
    z = ((bits + np.uint32(0x408080)) ^ np.uint32(0x808080)).astype(np.uint32)
    a2 = (z & 0xFF).astype(np.uint8).view(np.int8).astype(np.int64)
    a1 = ((z >> 8) & 0xFF).astype(np.uint8).view(np.int8).astype(np.int64)
    a0 = ((z >> 16) & 0xFF).astype(np.uint8).view(np.int8).astype(np.int64)
    return a0, a1, a2


def test_every_integer_in_range_splits_into_three_int8_digits_exactly():
    x = np.arange(-(1 << 21), (1 << 21) + 1, dtype=np.int64)
    a0, a1, a2 = digits_of(x.astype(np.float32))
    assert np.array_equal(a0 * 65536 + a1 * 256 + a2, x)
    assert a0.min() >= -33 and a0.max() <= 32          # the top digit stays far inside int8
    assert a1.min() >= -128 and a1.max() <= 127 and a2.min() >= -128 and a2.max() <= 127


def test_fractions_round_to_nearest_even_like_rint():
    r = np.random.default_rng(5)
    t = (r.uniform(-1, 1, 200000) * (1 << 21)).astype(np.float32)
    t = np.concatenate([t, np.array([0.5, 1.5, 2.5, -0.5, -1.5, 2097151.5, -2097151.5, 0.0, -0.0], np.float32)])
    a0, a1, a2 = digits_of(t)
    assert np.array_equal(a0 * 65536 + a1 * 256 + a2, np.rint(t.astype(np.float64)).astype(np.int64))


def test_block_scale_keeps_the_fixed_point_value_in_range_and_small_integers_exact():
    # scale = 2^(20 - e) with 2^e <= max|x| < 2^(e+1), built from the exponent field as the kernel does
    r = np.random.default_rng(6)
    for mag in (1e-25, 1e-3, 1.0, 7.99, 8.0, 1e6, 1e37):
        x = (r.standard_normal(2048) * mag).astype(np.float32)
        x[0] = np.float32(mag)
        ef = int((np.abs(x).max().view(np.uint32) >> 23) & 0xFF)
        ec = max(ef, 27)
        up = np.uint32((274 - ec) << 23).view(np.float32)
        down = np.uint32((ec - 20) << 23).view(np.float32)
        t = x * up
        assert np.abs(t).max() < (1 << 21)
        a0, a1, a2 = digits_of(t)
        back = (a0 * 65536 + a1 * 256 + a2).astype(np.float64) * float(down)
        # what is dropped per element is at most half a unit of 2^(e-20): below 2^-21 of the block's largest |x|
        assert np.abs(back - x.astype(np.float64)).max() <= 0.5 * float(down) * (1 + 1e-12)
    xi = r.integers(-1000, 1001, 2048).astype(np.float32)
    ef = int((np.abs(xi).max().view(np.uint32) >> 23) & 0xFF)
    up = np.uint32((274 - ef) << 23).view(np.float32)
    a0, a1, a2 = digits_of(xi * up)
    assert np.array_equal((a0 * 65536 + a1 * 256 + a2) * float(np.uint32((ef - 20) << 23).view(np.float32)), xi.astype(np.float64))

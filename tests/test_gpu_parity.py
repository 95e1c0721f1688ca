"""GPU parity: the HIP path, called through the C ABI (chadslab_amd.ops -> ctypes -> libchadq.so), against the
CPU oracle on the same seeded inputs.  Bit-exact for unpack/pack/dequant and integer accumulation; rel-L2
<= 1e-3 for fp32 outputs and <= 1e-2 for bf16 outputs against the float64 ground truth (tolerances from the
benchmark statement).  Full benchmark shapes are covered too: the numpy oracle finishes them in seconds.
"""
import os

import numpy as np
import pytest
import torch

from oracle import chadq_oracle as O

pytestmark = pytest.mark.gpu

TOL_F32 = 1e-3   # fp32 out
TOL_BF16 = 1e-2  # bf16 out
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from chadslab_amd import _lib, ops as _ops

    assert torch.cuda.is_available(), "these tests need the GPU"
    _lib.load()  # raises if libchadq.so is missing: there is no fallback to hide behind
    return _ops


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def bf16_tensor(b):
    return torch.from_numpy(b.view(np.int16)).view(torch.bfloat16).to(DEV)


def i4_case(seed, m, n, k, integer_x=False):
    from chadslab_amd import QWeightInt4G32

    r = rng(seed)
    u = r.integers(0, 16, (n, k), dtype=np.uint8)
    packed = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
    s = r.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    x = r.integers(-8, 9, (m, k)).astype(np.float32) if integer_x else r.standard_normal((m, k)).astype(np.float32)
    xb = O.f32_to_bf16(x)
    qw = QWeightInt4G32(torch.from_numpy(packed).to(DEV), torch.from_numpy(s).to(DEV))
    return packed, s, xb, qw


def i8_case(seed, m, n, k):
    from chadslab_amd import QWeightInt8

    r = rng(seed)
    x = r.standard_normal((m, k)).astype(np.float32)
    w = r.integers(-127, 128, (n, k), dtype=np.int8)
    s = r.uniform(0.001, 0.02, n).astype(np.float32)
    return x, w, s, QWeightInt8(torch.from_numpy(w).to(DEV), torch.from_numpy(s).to(DEV))


# ------------------------------------------------------------------ unpack / pack / dequant: bit-exact
@pytest.mark.parametrize("nbytes", [0, 1, 15, 16, 17, 255, 256, 4096 + 7, 1 << 20])
def test_unpack_bit_exact(ops, nbytes):
    wp = rng(nbytes).integers(0, 256, nbytes, dtype=np.uint8)
    if nbytes >= 256:
        wp[:256] = np.arange(256)  # every byte value
    out = ops.unpack_int4(torch.from_numpy(wp).to(DEV)).cpu().numpy()
    assert np.array_equal(out, O.unpack_int4(wp[None])[0] if nbytes else np.zeros(0, np.int8))


def test_unpack_unaligned_view(ops):
    wp = rng(3).integers(0, 256, 1001, dtype=np.uint8)
    t = torch.from_numpy(wp).to(DEV)[1:]  # data pointer off 16-byte alignment
    assert np.array_equal(ops.unpack_int4(t).cpu().numpy(), O.unpack_int4(wp[None, 1:])[0])


def test_pack_roundtrip(ops):
    q = rng(4).integers(-8, 8, (33, 130), dtype=np.int8)
    p = ops.pack_int4(torch.from_numpy(q).to(DEV))
    assert np.array_equal(p.cpu().numpy(), O.pack_int4(q))
    assert np.array_equal(ops.unpack_int4(p).cpu().numpy(), q)


def test_dequant_exact(ops):
    packed, s, _, qw = i4_case(5, 1, 96, 256)
    assert np.array_equal(ops.dequantize(qw).cpu().numpy(), O.dequant_int4g32(packed, s))
    _, w, s8, q8 = i8_case(6, 1, 50, 70)
    assert np.array_equal(ops.dequantize(q8).cpu().numpy(), O.dequant_int8(w, s8))


def test_bench_probe_reads_every_byte():
    # the loads-only kernel bench.py times beside the GEMV lives in its own small library next to bench.py
    import ctypes

    path = os.path.join(os.path.dirname(GOLD.rstrip(os.sep)), os.pardir, "bench_probe.so")
    if not os.path.exists(path):
        pytest.skip("bench_probe.so has not been built (__graft_entry__.build() builds it)")
    lib = ctypes.CDLL(os.path.abspath(path))
    lib.bench_probe_read.restype = ctypes.c_int
    lib.bench_probe_read.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    n = 5 * 16384 + 100  # the tail that does not fill 16 KiB is left alone
    data = rng(11).integers(0, 256, n, dtype=np.uint8)
    t = torch.from_numpy(data).to(DEV)
    out = torch.zeros(n // 16384, dtype=torch.int32, device=DEV)
    assert lib.bench_probe_read(t.data_ptr(), n, out.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    want = np.bitwise_xor.reduce(data[:5 * 16384].view(np.uint32).reshape(5, -1), axis=1)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want)


# ------------------------------------------------------------------ golden fixtures
def test_golden_int4(ops):
    from chadslab_amd import QWeightInt4G32

    g = np.load(os.path.join(GOLD, "i4g32_n64_k128.npz"))
    qw = QWeightInt4G32(torch.from_numpy(g["packed"]).to(DEV), torch.from_numpy(g["scale"]).to(DEV))
    x = bf16_tensor(g["x_bf16"])
    assert np.array_equal(ops.unpack_int4(qw.packed).cpu().numpy(), g["q"])
    assert np.array_equal(ops.dequantize(qw).cpu().numpy(), g["dequant"])
    assert O.rel_l2(ops.qgemv(x, qw).cpu().numpy(), g["y_f64"]) <= TOL_F32
    assert O.rel_l2(O.bf16_to_f32(bits(ops.qgemm(x, qw))), g["y_f64"]) <= TOL_BF16


def test_golden_int8(ops):
    from chadslab_amd import QWeightInt8

    g = np.load(os.path.join(GOLD, "i8row_n64_k128.npz"))
    q8 = QWeightInt8(torch.from_numpy(g["w"]).to(DEV), torch.from_numpy(g["scale"]).to(DEV))
    assert O.rel_l2(ops.qgemv(torch.from_numpy(g["x_f32"]).to(DEV), q8).cpu().numpy(), g["y_f64"]) <= TOL_F32
    assert O.rel_l2(O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(g["x_bf16"]), q8))), g["yb_f64"]) <= TOL_BF16


# ------------------------------------------------------------------ GEMV int4 (config 1)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 16])
@pytest.mark.parametrize("n,k", [(64, 128), (33, 32), (100, 4160), (48, 12288), (257, 2048), (1000, 4096), (16, 8192)])
def test_gemv_int4_shapes(ops, m, n, k):
    packed, s, xb, qw = i4_case(100 + m + n + k, m, n, k)
    y = ops.qgemv(bf16_tensor(xb), qw).cpu().numpy()
    assert y.shape == (m, n) and np.isfinite(y).all()
    assert O.rel_l2(y, O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_F32


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8, 9, 13, 16])
def test_gemv_int4_config1_full_size(ops, m):
    packed, s, xb, qw = i4_case(1001, m, 14336, 4096)
    y = ops.qgemv(bf16_tensor(xb), qw).cpu().numpy()
    assert O.rel_l2(y, O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_F32


@pytest.mark.parametrize("m,n,k", [(1, 32768, 2048), (1, 8200, 1024), (2, 8192, 8192), (5, 9001, 4096), (3, 8192, 256),
                                   (1, 11008, 4096), (2, 12345, 512), (4, 20000, 512), (8, 28672, 512), (1, 5000, 2048),
                                   (7, 12345, 768)])
def test_gemv_int4_tall_matrices(ops, m, n, k):
    # 8192 rows and more take the kernels with 32- and 64-row workgroups (a ragged last workgroup included); row
    # counts that would end mid-round on the chip run with tiles of 6, 7, 12, 13 or 14 rows instead of 8 or 16
    packed, s, xb, qw = i4_case(3000 + n + k, m, n, k)
    y = ops.qgemv(bf16_tensor(xb), qw).cpu().numpy()
    assert np.isfinite(y).all() and O.rel_l2(y, O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_F32


@pytest.mark.parametrize("m", [1, 4])
def test_gemv_int4_output_table_256000_rows(ops, m):
    # the decode step's output projection: 256000 rows of K = 2048 (the tallest matrix the benchmark has); the float64
    # truth and the integer brute force are formed 32000 rows at a time to keep the host's copies small
    from chadslab_amd import QWeightInt4G32

    n, k, step = 256000, 2048, 32000
    packed, s, xb, qw = i4_case(4100 + m, m, n, k)
    y = ops.qgemv(bf16_tensor(xb), qw).cpu().numpy()
    assert y.shape == (m, n) and np.isfinite(y).all()
    want = np.concatenate([O.qgemm_int4g32_f64(xb, packed[r: r + step], s[r: r + step]) for r in range(0, n, step)], axis=1)
    assert O.rel_l2(y, want) <= TOL_F32
    xi = O.f32_to_bf16(rng(4102).integers(-8, 9, (m, k)).astype(np.float32))
    yi = ops.qgemv(bf16_tensor(xi), QWeightInt4G32(qw.packed, torch.ones_like(qw.scale))).cpu().numpy()
    xf = O.bf16_to_f32(xi).astype(np.float64)  # small integers: float64 sums of their products are exact
    brute = np.concatenate([xf @ O.unpack_int4(packed[r: r + step]).astype(np.float64).T for r in range(0, n, step)], axis=1)
    assert np.abs(brute).max() < 2 ** 24 and np.array_equal(yi, brute.astype(np.float32))


@pytest.mark.parametrize("m,n,k", [(1, 14336, 4096), (2, 14336, 4096), (8, 512, 4096), (4, 96, 256), (2, 40, 96),
                                   (5, 14336, 4096), (8, 14336, 4096), (6, 300, 512), (7, 8192, 256),
                                   (9, 8192, 2048), (12, 14336, 4096), (16, 512, 4096), (16, 300, 512), (11, 64, 256)])
def test_gemv_int4_integer_accumulation_bit_exact(ops, m, n, k):
    from chadslab_amd import QWeightInt4G32

    packed, _, xb, qw = i4_case(7, m, n, k, integer_x=True)
    ones = QWeightInt4G32(qw.packed, torch.ones_like(qw.scale))
    y = ops.qgemv(bf16_tensor(xb), ones).cpu().numpy()
    brute = O.bf16_to_f32(xb).astype(np.int64) @ O.unpack_int4(packed).astype(np.int64).T
    assert np.abs(brute).max() < 2 ** 24
    assert np.array_equal(y.astype(np.int64), brute) and np.array_equal(y, brute.astype(np.float32))


def test_gemv_int4_row_consistency_and_linearity(ops):
    packed, s, xb, qw = i4_case(8, 8, 512, 4096)
    x = bf16_tensor(xb)
    y8 = ops.qgemv(x, qw).cpu().numpy()
    for r in (0, 3, 7):
        y1 = ops.qgemv(x[r:r + 1].contiguous(), qw).cpu().numpy()
        assert O.rel_l2(y1[0], y8[r]) <= 1e-6  # same products, possibly another summation order
    a = rng(9).integers(-64, 64, (1, 4096)).astype(np.float32)
    b = rng(10).integers(-64, 64, (1, 4096)).astype(np.float32)
    ya, yb, yab = (ops.qgemv(bf16_tensor(O.f32_to_bf16(v)), qw).cpu().numpy() for v in (a, b, a + b))
    assert O.rel_l2(yab, ya + yb) <= 1e-5


def test_gemv_int4_zero_weights_and_special_scales(ops):
    from chadslab_amd import QWeightInt4G32

    n, k = 64, 4096
    x = bf16_tensor(O.f32_to_bf16(rng(11).standard_normal((2, k)).astype(np.float32)))
    zero = QWeightInt4G32(torch.full((n, k // 2), 0x88, dtype=torch.uint8, device=DEV), torch.ones(n, k // 32, dtype=torch.float16, device=DEV))
    y = ops.qgemv(x, zero).cpu().numpy()
    # u = 8 everywhere: the 128+u offset must cancel; what is left is fp32 rounding of sums near 136*sum|x|,
    # about 1e-4 of the size a typical output has for these shapes (~300)
    assert np.abs(y).max() <= 2e-2
    # one-hot activation returns one dequantised column exactly
    packed, s, _, qw = i4_case(12, 1, n, k)
    d = O.dequant_int4g32(packed, s)
    for kk in (0, 31, 32, 2047, 4095):
        e = np.zeros((1, k), np.float32)
        e[0, kk] = 1.0
        assert np.array_equal(ops.qgemv(bf16_tensor(O.f32_to_bf16(e)), qw).cpu().numpy()[0], d[:, kk])


# ------------------------------------------------------------------ GEMV int8 (config 0)
@pytest.mark.parametrize("m,n,k", [(1, 16384, 2048), (1, 64, 16), (3, 100, 1040), (2, 77, 4096), (16, 40, 256),
                                   # rows of 2049..8192 k (4 or 8 chunks per row), and beyond (the general kernel)
                                   (1, 5000, 4096), (2, 300, 3008), (1, 4500, 8192), (3, 33, 6000), (1, 50, 8208),
                                   (1, 9000, 1024), (2, 8200, 528)])
def test_gemv_int8(ops, m, n, k):
    x, w, s, q8 = i8_case(1000 if (n, k) == (16384, 2048) else 20 + n, m, n, k)
    y = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
    assert O.rel_l2(y, O.qgemv_int8_f64(x, w, s)) <= TOL_F32


# K a multiple of 128 runs on the int8 matrix core (activations as three fixed-point digits per 2048 k), one pass over
# the weights for any M <= 16; other K keep the fp32 kernels
@pytest.mark.parametrize("m,n,k", [(1, 16384, 2048), (4, 16384, 2048), (5, 16384, 2048), (8, 16384, 2048), (9, 16384, 2048),
                                   (16, 16384, 2048), (1, 1, 128), (4, 63, 128), (5, 65, 256), (8, 129, 1152), (12, 200, 2176),
                                   (16, 77, 1920), (3, 4100, 4096), (7, 300, 6144), (16, 130, 8192), (2, 50, 10240),
                                   (13, 70, 12416)])
def test_gemv_int8_matrix_core(ops, m, n, k):
    x, w, s, q8 = i8_case(300 + m + n, m, n, k)
    y = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
    assert O.rel_l2(y, O.qgemv_int8_f64(x, w, s)) <= TOL_F32


@pytest.mark.parametrize("m,n,k", [(2, 300, 2048), (2, 300, 2064), (1, 100, 4096), (5, 333, 4096), (8, 64, 2048), (16, 70, 6144),
                                   (11, 90, 128)])
def test_gemv_int8_integer_exact(ops, m, n, k):
    from chadslab_amd import QWeightInt8

    r = rng(21 + m)
    x = r.integers(-8, 9, (m, k)).astype(np.float32)
    w = r.integers(-128, 128, (n, k), dtype=np.int8)
    q8 = QWeightInt8(torch.from_numpy(w).to(DEV), torch.ones(n, device=DEV))
    y = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
    assert np.array_equal(y.astype(np.int64), x.astype(np.int64) @ w.astype(np.int64).T)


def test_gemv_int8_rows_do_not_depend_on_their_neighbours(ops):
    """Row m of an M-row call equals the one-row call on x[m] bit for bit (per-row scales, exact integer sums), for
    every form of the matrix-core kernel (M <= 4, <= 8, <= 16) and across a 2048-k block boundary."""
    x, w, s, q8 = i8_case(77, 16, 333, 4096)
    xt = torch.from_numpy(x).to(DEV)
    one = torch.cat([ops.qgemv(xt[i:i + 1], q8) for i in range(16)]).cpu().numpy()
    for m in (3, 4, 7, 8, 11, 16):
        assert np.array_equal(ops.qgemv(xt[:m], q8).cpu().numpy(), one[:m]), m


def test_gemv_int8_outliers_zero_rows_and_non_finite_values(ops):
    x, w, s, q8 = i8_case(78, 6, 200, 4096)
    x[0, 17] = 3.0e6          # one huge value: the block's fixed-point scale follows it
    x[1, :] = 0.0             # an all-zero row
    x[2, 2048:] *= 1.0e-20    # a block of tiny values next to an ordinary one
    x[3, :] *= 1.0e15
    y = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
    ref = O.qgemv_int8_f64(x, w, s)
    for m in range(6):
        assert O.rel_l2(y[m:m + 1], ref[m:m + 1]) <= TOL_F32 or not ref[m].any(), m
    assert not y[1].any()
    x[4, 3000] = np.inf
    x[5, 5] = np.nan
    y2 = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
    assert np.isnan(y2[4]).all() and np.isnan(y2[5]).all()   # a non-finite activation makes its own row NaN ...
    assert np.array_equal(y2[:4], y[:4])                      # ... and no other


def test_gemv_int8_outlier_column_error_bound_per_element(ops):
    """The matrix-core int8 GEMV holds a block of 2048 activations in fixed point relative to the block's largest |x|:
    the header's bound |err| <= |s[n]| * sum over blocks of 2^-21 * max|x| * sum|W[n,k]| is checked element by element
    with one outlier column, in particular on output rows whose weight at the outlier is ZERO (there the outlier adds
    nothing to the exact result and the whole difference is the other elements' lost low bits).  chadq_gemv_i8row_fp32
    has no such term: the same inputs come out at fp32 accuracy."""
    m_rows, n, k = 5, 512, 4096
    x, w, s, _ = i8_case(781, m_rows, n, k)
    col = 17
    x[:, col] = 3.0e6 * np.array([1, -1, 1, 1, -1], np.float32)
    w[::2, col] = 0                              # every other output row ignores the outlier
    x[3, 2048 + 5] = -7.0e4                      # a second, smaller outlier in row 3's second block
    from chadslab_amd import QWeightInt8

    q8 = QWeightInt8(torch.from_numpy(w).to(DEV), torch.from_numpy(s).to(DEV))
    xt = torch.from_numpy(x).to(DEV)
    ref = O.qgemv_int8_f64(x, w, s)
    y = ops.qgemv(xt, q8).cpu().numpy().astype(np.float64)
    aw = np.abs(w.astype(np.float64))
    bound = np.zeros((m_rows, n))
    for b0 in range(0, k, 2048):
        bmax = np.abs(x[:, b0:b0 + 2048]).max(axis=1).astype(np.float64)            # [M]
        bound += 2.0 ** -21 * bmax[:, None] * aw[:, b0:b0 + 2048].sum(axis=1)[None, :]
    bound = np.abs(s.astype(np.float64))[None, :] * bound
    slack = 4e-7 * np.abs(ref) + 1e-30                                               # the fp32 roundings of the sums
    err = np.abs(y - ref)
    assert (err <= bound + slack).all(), float((err / (bound + slack)).max())
    # the bound is not vacuous: on the rows that ignore the outlier the error is a visible fraction of the result ...
    zero_rows = err[:, ::2] / (np.abs(ref[:, ::2]) + 1e-30)
    assert np.median(zero_rows) > 1e-3
    # ... and the fp32 form has none of it
    yf = ops.qgemv(xt, q8, fp32_elements=True).cpu().numpy().astype(np.float64)
    mag = (np.abs(x.astype(np.float64)) @ (aw * np.abs(s.astype(np.float64))[:, None]).T)  # sum of |terms|
    assert (np.abs(yf - ref) <= 1e-5 * mag).all()
    assert np.median(np.abs(yf[:, ::2] - ref[:, ::2]) / (np.abs(ref[:, ::2]) + 1e-30)) < 1e-5


@pytest.mark.parametrize("m,n,k", [(1, 16384, 2048), (2, 300, 4096), (5, 333, 2048), (16, 70, 6144), (3, 100, 1040)])
def test_gemv_int8_fp32_elements_entry_point(ops, m, n, k):
    x, w, s, q8 = i8_case(790 + m, m, n, k)
    y = ops.qgemv(torch.from_numpy(x).to(DEV), q8, fp32_elements=True).cpu().numpy()
    assert O.rel_l2(y, O.qgemv_int8_f64(x, w, s)) <= TOL_F32
    xi = rng(791 + m).integers(-2000, 2001, (m, k)).astype(np.float32)
    one = type(q8)(q8.w, torch.ones_like(q8.scale))
    yi = ops.qgemv(torch.from_numpy(xi).to(DEV), one, fp32_elements=True).cpu().numpy()
    want = xi.astype(np.int64) @ w.astype(np.int64).T
    ok = np.abs(want) < 2 ** 24
    assert np.array_equal(yi[ok].astype(np.int64), want[ok])
    xinf = x.copy()
    xinf[0, 3] = np.inf
    yinf = ops.qgemv(torch.from_numpy(xinf).to(DEV), q8, fp32_elements=True).cpu().numpy()
    nz = w[:, 3] != 0  # IEEE arithmetic element by element: inf * w is an infinity, inf * 0 a NaN
    assert np.isinf(yinf[0][nz]).all() and np.isnan(yinf[0][~nz]).all()
    assert np.isfinite(yinf[1:]).all()


def test_gemv_int8_integer_digit_sums_that_cancel_stay_exact(ops):
    """The matrix-core kernel sums three base-256 digits of the fixed-point activations separately and recombines
    D0 * 2^16 + D1 * 2^8 + D2.  Here the digit sums are far beyond 2^24 and cancel: x = 32768 (digits 1, -128, 0)
    against weights +64 and x = 32512 (digits 0, 127, 0) against weights -64, so D0 * 2^16 = 2.1e9 and D1 * 2^8 = -2.1e9
    while the result is 8.4e6 + small.  Recombined in float64 the result is the exact integer (fp32 recombination
    was off by up to 128 here)."""
    n, k = 64, 2048
    r = rng(795)
    w = np.zeros((n, k), np.int8)
    x = np.zeros((1, k), np.float32)
    x[0, 0:1024:2], x[0, 1:1024:2] = 32768.0, 32512.0
    w[:, 0:1024:2], w[:, 1:1024:2] = 64, -64
    w[:, 0:1024:2] += r.integers(-1, 2, (n, 512)).astype(np.int8)   # a little variety per output row
    x[0, 1024:1100] = r.integers(-50, 51, 76)                        # the other half of K: small integers
    w[:, 1024:1100] = r.integers(-127, 128, (n, 76))
    from chadslab_amd import QWeightInt8

    q8 = QWeightInt8(torch.from_numpy(w).to(DEV), torch.ones(n, device=DEV))
    want = x.astype(np.int64) @ w.astype(np.int64).T
    assert np.abs(want).max() < 2 ** 24 and np.abs(want).min() > 2 ** 22
    y = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
    assert np.array_equal(y.astype(np.int64), want)


# ------------------------------------------------------------------ seeded random shapes (ragged edges of every kind)
def test_random_shapes_int4_gemv_and_gemm(ops):
    r = rng(4242)
    for case in range(36):
        m = int(r.choice([1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 40, 130]))
        n = int(r.integers(1, 700)) if case % 3 else int(r.integers(8192, 9500))
        k = 32 * int(r.integers(1, 70))
        if n >= 8192:
            k = 32 * int(r.integers(1, 20))  # keep the float64 reference quick
        packed, s, xb, qw = i4_case(5000 + case, m, n, k)
        ref = O.qgemm_int4g32_f64(xb, packed, s)
        if m <= 16:
            y = ops.qgemv(bf16_tensor(xb), qw).cpu().numpy()
            assert y.shape == (m, n) and np.isfinite(y).all() and O.rel_l2(y, ref) <= TOL_F32, ("gemv", m, n, k)
        yb = O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), qw)))
        assert yb.shape == (m, n) and np.isfinite(yb).all() and O.rel_l2(yb, ref) <= TOL_BF16, ("gemm", m, n, k)


def test_random_shapes_int8(ops):
    r = rng(4243)
    for case in range(16):
        m = int(r.choice([1, 3, 8, 33, 129]))
        n = int(r.integers(1, 600))
        k = 16 * int(r.integers(1, 90))
        x, w, s, q8 = i8_case(6000 + case, m, n, k)
        xb = O.f32_to_bf16(x)
        yb = O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), q8)))
        assert O.rel_l2(yb, O.qgemm_int8_f64(xb, w, s)) <= TOL_BF16, ("gemm8", m, n, k)
        y1 = ops.qgemv(torch.from_numpy(x[:1]).to(DEV), q8).cpu().numpy()
        ref1 = (x[:1].astype(np.float64) @ (w.astype(np.float64) * s[:, None].astype(np.float64)).T)
        assert O.rel_l2(y1, ref1) <= TOL_F32, ("gemv8", n, k)
    # the GEMV at every M it takes: K a multiple of 128 (int8 matrix core, all three operand forms, one to six
    # 2048-blocks) and other K (fp32 kernels), ragged N
    for case in range(40):
        m = int(r.integers(1, 17))
        n = int(r.integers(1, 400)) if case % 4 else int(r.integers(8192, 8400))
        k = 128 * int(r.integers(1, 90)) if case % 2 else 16 * int(r.integers(1, 300))
        if n >= 8192:
            k = min(k, 2048)
        x, w, s, q8 = i8_case(7000 + case, m, n, k)
        y = ops.qgemv(torch.from_numpy(x).to(DEV), q8).cpu().numpy()
        assert y.shape == (m, n) and np.isfinite(y).all() and O.rel_l2(y, O.qgemv_int8_f64(x, w, s)) <= TOL_F32, ("gemv8", m, n, k)


# ------------------------------------------------------------------ prefill GEMM (config 2)
@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (1, 64, 128), (37, 100, 96), (130, 70, 288), (5, 33, 32), (128, 64, 256), (200, 192, 1056)])
def test_gemm_int4(ops, m, n, k):
    packed, s, xb, qw = i4_case(1002 if m == 512 else 30 + m, m, n, k)
    y = O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), qw)))
    assert y.shape == (m, n)
    assert O.rel_l2(y, O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_BF16


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (3, 40, 16), (129, 65, 272), (64, 128, 128)])
def test_gemm_int8(ops, m, n, k):
    x, w, s, q8 = i8_case(40 + m, m, n, k)
    xb = O.f32_to_bf16(x)
    y = O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), q8)))
    assert O.rel_l2(y, O.qgemm_int8_f64(xb, w, s)) <= TOL_BF16


@pytest.mark.parametrize("m,n,k", [(4096, 4096, 512), (3300, 3500, 256), (2817, 4099, 768), (8192, 1536, 1024)])
def test_gemm_int4_many_rows_tile(ops, m, n, k):
    # enough 256 x 256 tiles to cover the chip: these shapes run on the large-tile kernel (K a multiple of 256), with
    # ragged last tiles in both directions and, for n = 4099, rows the vector stores cannot take
    packed, s, xb, qw = i4_case(600 + m + n + k, m, n, k)
    y = O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), qw)))
    assert y.shape == (m, n) and np.isfinite(y).all()
    assert O.rel_l2(y, O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_BF16


def test_gemm_int4_many_rows_full_k_and_integer_exact(ops):
    from chadslab_amd import QWeightInt4G32

    # 4096 x 4096 x 4096: the float64 truth is formed for a sample of rows only (the oracle's full product would take
    # minutes); every row of the result is still checked for being finite
    m = n = k = 4096
    packed, s, xb, qw = i4_case(611, m, n, k)
    y = O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), qw)))
    assert np.isfinite(y).all()
    rows = rng(612).choice(m, 96, replace=False)
    rows[:4] = (0, 255, 256, 4095)
    assert O.rel_l2(y[rows], O.qgemm_int4g32_f64(xb[rows], packed, s)) <= TOL_BF16
    # integer activations and unit scales: every sum is an integer below 2^24, so fp32 accumulation is exact and the
    # only rounding is the final one to bf16
    xi = O.f32_to_bf16(rng(613).integers(-4, 5, (m, 1024)).astype(np.float32))
    pk, _, _, q1 = i4_case(614, 1, n, 1024)
    yi = bits(ops.qgemm(bf16_tensor(xi), QWeightInt4G32(q1.packed, torch.ones_like(q1.scale))))
    brute = O.bf16_to_f32(xi[rows]).astype(np.float64) @ O.unpack_int4(pk).astype(np.float64).T
    assert np.abs(brute).max() < 2 ** 24
    assert np.array_equal(yi[rows], O.f32_to_bf16(brute.astype(np.float32)))


def test_gemm_agrees_with_gemv_at_m8(ops):
    packed, s, xb, qw = i4_case(50, 8, 1024, 4096)
    x = bf16_tensor(xb)
    gemv = ops.qgemv(x, qw).cpu().numpy()
    gemm = O.bf16_to_f32(bits(ops.qgemm(x, qw)))
    assert O.rel_l2(gemm, gemv) <= TOL_BF16


def test_gemm_int4_integer_exact_when_scales_are_one(ops):
    from chadslab_amd import QWeightInt4G32

    packed, _, xb, qw = i4_case(51, 64, 128, 512, integer_x=True)
    ones = QWeightInt4G32(qw.packed, torch.ones_like(qw.scale))
    # |sum| <= 512*8*8 = 32768 needs 16 bits: bf16 output cannot hold it, so compare after rounding the
    # exact integer result to bf16 (fp32 accumulation of exact integers is exact)
    brute = (O.bf16_to_f32(xb).astype(np.int64) @ O.unpack_int4(packed).astype(np.int64).T).astype(np.float32)
    assert np.array_equal(bits(ops.qgemm(bf16_tensor(xb), ones)), O.f32_to_bf16(brute))


# ------------------------------------------------------------------ full benchmark sizes: properties that need no CPU reference
def test_full_size_properties_without_a_reference(ops):
    from chadslab_amd import QWeightInt4G32, QWeightInt8

    # config 1: rows of an M=8 product equal the M=1 products; integer inputs make linearity exact
    n, k = 14336, 4096
    packed, s, xb, qw = i4_case(1001, 8, n, k)
    x = bf16_tensor(xb)
    y8 = ops.qgemv(x, qw).cpu().numpy()
    for r in (0, 5):
        assert O.rel_l2(ops.qgemv(x[r:r + 1].contiguous(), qw).cpu().numpy()[0], y8[r]) <= 1e-6
    ones = QWeightInt4G32(qw.packed, torch.ones_like(qw.scale))
    a = rng(2).integers(-4, 5, (1, k)).astype(np.float32)
    b = rng(3).integers(-4, 5, (1, k)).astype(np.float32)
    ya, yb, yab = (ops.qgemv(bf16_tensor(O.f32_to_bf16(v)), ones).cpu().numpy() for v in (a, b, a + b))
    assert np.array_equal(yab, ya + yb)
    # config 2: the prefill kernel and the decode kernel agree on the rows they share
    packed2, s2, xb2, qw2 = i4_case(1002, 512, 4096, 4096)
    x2 = bf16_tensor(xb2)
    gemm = O.bf16_to_f32(bits(ops.qgemm(x2, qw2)))
    gemv = ops.qgemv(x2[100:108].contiguous(), qw2).cpu().numpy()
    assert O.rel_l2(gemm[100:108], gemv) <= TOL_BF16
    # ... and a permutation of the activation rows permutes the output rows, bit for bit
    perm = rng(4).permutation(512)
    gemm_p = bits(ops.qgemm(bf16_tensor(xb2[perm]), qw2))
    assert np.array_equal(gemm_p, bits(ops.qgemm(x2, qw2))[perm])
    # config 0: scaling a row's scale scales that output; integer inputs make linearity exact
    x0, w0, s0, q8 = i8_case(1000, 1, 16384, 2048)
    y0 = ops.qgemv(torch.from_numpy(x0).to(DEV), q8).cpu().numpy()
    q8b = QWeightInt8(q8.w, q8.scale * 2.0)
    assert np.array_equal(ops.qgemv(torch.from_numpy(x0).to(DEV), q8b).cpu().numpy(), 2.0 * y0)
    q1 = QWeightInt8(q8.w, torch.ones_like(q8.scale))
    ia = rng(5).integers(-8, 9, (1, 2048)).astype(np.float32)
    ib = rng(6).integers(-8, 9, (1, 2048)).astype(np.float32)
    za, zb, zab = (ops.qgemv(torch.from_numpy(v).to(DEV), q1).cpu().numpy() for v in (ia, ib, ia + ib))
    assert np.array_equal(zab, za + zb)


# ------------------------------------------------------------------ operator layer and error behaviour
def test_qlinear_dispatch(ops):
    packed, s, xb, qw = i4_case(60, 6, 128, 256)
    x = bf16_tensor(xb).reshape(2, 3, 256)
    y = ops.qlinear(x, qw)
    assert y.shape == (2, 3, 128) and y.dtype == torch.float32  # decode sizes come back in fp32
    assert O.rel_l2(y.reshape(6, 128).cpu().numpy(), O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_F32
    packed, s, xb, qw = i4_case(61, 40, 128, 256)
    y = ops.qlinear(bf16_tensor(xb), qw)
    assert y.dtype == torch.bfloat16 and O.rel_l2(O.bf16_to_f32(bits(y)), O.qgemm_int4g32_f64(xb, packed, s)) <= TOL_BF16
    assert ops.qlinear(bf16_tensor(xb), qw, out_dtype=torch.float32).dtype == torch.float32


def test_errors_surface_as_exceptions(ops):
    from chadslab_amd import QWeightInt4G32, _lib

    _, _, xb, qw = i4_case(62, 1, 64, 128)
    with pytest.raises(ValueError):
        ops.qgemv(bf16_tensor(xb)[:, :96].contiguous(), qw)          # K mismatch
    with pytest.raises(ValueError):
        ops.qgemv(bf16_tensor(xb).float(), qw)                       # wrong dtype
    with pytest.raises(ValueError):
        ops.qgemv(bf16_tensor(np.zeros((17, 128), np.uint16)), qw)   # M beyond the GEMV's range
    lib = _lib.load()
    assert lib.chadq_gemv_i4g32(None, None, None, None, 1, 64, 128, None) == -1
    assert b"null" in lib.chadq_last_error()
    assert lib.chadq_gemv_i4g32(None, None, None, None, 1, 64, 100, None) == -2
    assert b"multiple of 32" in lib.chadq_last_error()
    assert lib.chadq_gemv_i4g32(None, None, None, None, 1, 0, 128, None) == 0  # empty output: nothing to do


# ------------------------------------------------------------------ MoE (config 3)
def _experts(seed, e, h, f):
    """e experts of random int4 group-32 weights: numpy tuples for the oracle and device containers for the ops."""
    from chadslab_amd import QWeightInt4G32

    r = rng(seed)
    host, dev = [], []
    for _ in range(e):
        hw, dw = [], []
        for (n, k) in ((f, h), (f, h), (h, f)):
            u = r.integers(0, 16, (n, k), dtype=np.uint8)
            p = (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)
            s = (r.lognormal(-5, 0.5, (n, k // 32)) * (0.6 if n == h else 1.0)).astype(np.float16)
            hw += [p, s]
            dw.append(QWeightInt4G32(torch.from_numpy(p).to(DEV), torch.from_numpy(s).to(DEV)))
        host.append(tuple(hw))
        dev.append(tuple(dw))
    return host, dev


def test_moe_route_matches_oracle(ops):
    r = rng(70)
    logits = r.standard_normal((300, 8)).astype(np.float32)
    logits[5, 2] = logits[5, 6] = logits[5].max() + 1.0   # tie for first place
    logits[9, :] = 0.25                                    # all equal
    logits[11, 1] = logits[11, 3]                          # tie somewhere
    for top_k, renorm in ((2, True), (2, False), (1, True), (4, True)):
        idx, w = ops.moe_route(torch.from_numpy(logits).to(DEV), top_k, renorm)
        oi, ow = O.moe_route(logits, top_k, renorm)
        assert np.array_equal(idx.cpu().numpy(), oi)       # indices bit-exact
        assert np.allclose(w.cpu().numpy(), ow, rtol=2e-5, atol=1e-7)
    assert idx.cpu().numpy()[9].tolist() == [0, 1, 2, 3]


def test_moe_golden(ops):
    from chadslab_amd import QWeightInt4G32

    g = np.load(os.path.join(GOLD, "moe_t16_h64_f96_e4.npz"))
    experts = [tuple(QWeightInt4G32(torch.from_numpy(g["e%d_%s_p" % (i, n)]).to(DEV), torch.from_numpy(g["e%d_%s_s" % (i, n)]).to(DEV))
                     for n in "gud") for i in range(4)]
    y = ops.moe_ffn(bf16_tensor(g["x_bf16"]), torch.from_numpy(g["logits"]).to(DEV), experts, top_k=2, renorm=True)
    assert O.rel_l2(O.bf16_to_f32(bits(y)), O.bf16_to_f32(g["y_bf16"])) <= TOL_BF16


@pytest.mark.parametrize("t,h,f,e,top_k", [(256, 512, 1024, 8, 2), (37, 128, 160, 3, 1), (64, 256, 256, 1, 1), (130, 256, 512, 16, 4),
                                           (300, 256, 512, 2, 2), (33, 256, 768, 8, 2), (200, 512, 512, 3, 1),
                                           # more than 1024 pairs (the router sorts them in several passes) and more than
                                           # 4096 (its ranks go through memory instead of LDS)
                                           (400, 256, 256, 8, 4), (1200, 256, 256, 4, 4), (1100, 64, 96, 5, 4)])
def test_moe_ffn(ops, t, h, f, e, top_k):
    host, dev = _experts(80 + t, e, h, f)
    r = rng(81 + t)
    xb = O.f32_to_bf16(r.standard_normal((t, h)).astype(np.float32))
    logits = r.standard_normal((t, e)).astype(np.float32)
    y = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), dev, top_k=top_k, renorm=True)))
    ref = O.bf16_to_f32(O.moe_qffn(xb, logits, host, top_k, True))
    assert np.isfinite(y).all() and O.rel_l2(y, ref) <= TOL_BF16
    # token order does not matter
    perm = r.permutation(t)
    yp = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb[perm]), torch.from_numpy(logits[perm]).to(DEV), dev, top_k=top_k, renorm=True)))
    assert np.array_equal(yp, y[perm])


def test_moe_ffn_empty_experts_and_one_crowded_expert(ops):
    # experts 2..7 get nothing, expert 0 gets every token (three token tiles of 96), expert 1 the second choice of most
    t, h, f, e = 250, 256, 512, 8
    host, dev = _experts(90, e, h, f)
    r = rng(91)
    xb = O.f32_to_bf16(r.standard_normal((t, h)).astype(np.float32))
    logits = r.standard_normal((t, e)).astype(np.float32)
    logits[:, 0] += 30.0
    logits[:, 1] += 15.0
    logits[:7, 1] -= 40.0  # a few tokens take some other expert second: tiles of very few rows
    y = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), dev, top_k=2, renorm=True)))
    ref = O.bf16_to_f32(O.moe_qffn(xb, logits, host, 2, True))
    assert np.isfinite(y).all() and O.rel_l2(y, ref) <= TOL_BF16


def test_moe_ffn_random_shapes(ops):
    r = rng(4244)
    for case in range(8):
        e = int(r.integers(1, 9))
        top_k = int(r.integers(1, min(e, 4) + 1))
        t = int(r.integers(1, 300))
        if case % 2:  # shapes the expert kernel takes (multiples of 256) / shapes that go the general way
            h, f = 256 * int(r.integers(1, 4)), 256 * int(r.integers(1, 4))
        else:
            h, f = 32 * int(r.integers(1, 12)), 32 * int(r.integers(1, 12))
        host, dev = _experts(7000 + case, e, h, f)
        xb = O.f32_to_bf16(r.standard_normal((t, h)).astype(np.float32))
        logits = r.standard_normal((t, e)).astype(np.float32)
        y = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), dev, top_k=top_k, renorm=bool(case & 2))))
        ref = O.bf16_to_f32(O.moe_qffn(xb, logits, host, top_k, bool(case & 2)))
        assert np.isfinite(y).all() and O.rel_l2(y, ref) <= TOL_BF16, (t, h, f, e, top_k)


def test_moe_config3_full_size(ops):
    t, h, f, e = 256, 4096, 14336, 8
    host, dev = _experts(1003, e, h, f)
    r = rng(1003)
    logits = r.standard_normal((t, e)).astype(np.float32)
    xb = O.f32_to_bf16(r.standard_normal((t, h)).astype(np.float32))
    y = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), dev, top_k=2, renorm=True)))
    ref = O.bf16_to_f32(O.moe_qffn(xb, logits, host, 2, True))
    assert O.rel_l2(y, ref) <= TOL_BF16
    # the same experts in tile order: the matrix-core kernel for that order holds the dequantised weights in fp16 (the
    # row-major one in bf16), so the two agree within rounding, and each with the oracle
    tiled = [tuple(ops.to_tiles(m) for m in tr) for tr in dev]
    yt = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), tiled, top_k=2, renorm=True)))
    assert np.isfinite(yt).all() and O.rel_l2(yt, ref) <= TOL_BF16
    assert O.rel_l2(yt, ref) <= O.rel_l2(y, ref) * 1.05 + 1e-4  # never less accurate than the bf16 form
    assert O.rel_l2(yt, y) <= 6e-3


# ------------------------------------------------------------------ tile order (load-time repack for the experts)
@pytest.mark.parametrize("n,k", [(32, 256), (64, 512), (96, 1280), (256, 4096), (14336, 4096), (4096, 14336)])
def test_repack_tiles_bit_exact_and_round_trip(ops, n, k):
    from chadslab_amd import QWeightInt4G32

    r = rng(5100 + n + k)
    p = r.integers(0, 256, (n, k // 2), dtype=np.uint8)
    s = r.integers(0, 65536, (n, k // 32), dtype=np.uint16)  # every bit pattern, NaNs included: the repack moves bytes
    qw = QWeightInt4G32(torch.from_numpy(p).to(DEV), torch.from_numpy(s).view(torch.float16).to(DEV))
    tl = ops.to_tiles(qw)
    wp_t, sc_t = O.tile_int4g32(p, s.view(np.float16))
    assert np.array_equal(tl.packed.cpu().numpy(), wp_t)
    assert np.array_equal(tl.scale.view(torch.int16).cpu().numpy().view(np.uint16), sc_t.view(np.uint16))
    back = ops.to_rows(tl)
    assert torch.equal(back.packed, qw.packed) and torch.equal(back.scale.view(torch.int16), qw.scale.view(torch.int16))


def test_repack_tiles_refuses_bad_shapes_and_aliasing(ops):
    from chadslab_amd import QWeightInt4G32, _lib

    for n, k in ((48, 256), (32, 128), (32, 288)):
        qw = QWeightInt4G32(torch.zeros(n, k // 2, dtype=torch.uint8, device=DEV), torch.zeros(n, k // 32, dtype=torch.float16, device=DEV))
        with pytest.raises(ValueError):
            ops.to_tiles(qw)
    lib = _lib.load()
    a = torch.zeros(32, 128, dtype=torch.uint8, device=DEV)
    sc = torch.zeros(32, 8, dtype=torch.float16, device=DEV)
    sc2 = torch.zeros_like(sc)
    assert lib.chadq_repack_i4g32_tiles(a.data_ptr(), sc.data_ptr(), a.data_ptr(), sc2.data_ptr(), 32, 256, None) == -2  # in place
    assert lib.chadq_repack_i4g32_tiles(a.data_ptr(), sc.data_ptr(), None, sc2.data_ptr(), 32, 256, None) == -1


@pytest.mark.parametrize("t,h,f,e,top_k", [(256, 512, 1024, 8, 2), (64, 256, 256, 1, 1), (130, 256, 512, 16, 4), (300, 256, 768, 2, 2),
                                           (1200, 256, 256, 4, 4), (200, 768, 1280, 3, 2), (96, 1024, 2048, 2, 1)])
def test_moe_ffn_tiled_agrees_with_row_major_and_oracle(ops, t, h, f, e, top_k):
    host, dev = _experts(8800 + t, e, h, f)
    r = rng(8801 + t)
    xb = O.f32_to_bf16(r.standard_normal((t, h)).astype(np.float32))
    logits = r.standard_normal((t, e)).astype(np.float32)
    y = bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), dev, top_k=top_k, renorm=True))
    tiled = [tuple(ops.to_tiles(m) for m in tr) for tr in dev]
    yt = bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), tiled, top_k=top_k, renorm=True))
    ref = O.bf16_to_f32(O.moe_qffn(xb, logits, host, top_k, True))
    assert np.isfinite(O.bf16_to_f32(yt)).all() and O.rel_l2(O.bf16_to_f32(yt), ref) <= TOL_BF16
    assert O.rel_l2(O.bf16_to_f32(yt), O.bf16_to_f32(y)) <= 6e-3  # fp16 against bf16 dequantised weights: rounding only
    # token order does not matter
    perm = r.permutation(t)
    yp = bits(ops.moe_ffn(bf16_tensor(xb[perm]), torch.from_numpy(logits[perm]).to(DEV), tiled, top_k=top_k, renorm=True))
    assert np.array_equal(yp, yt[perm])


def test_moe_ffn_tiled_wide_ranges_of_activations_and_scales(ops):
    """The tile-order kernels carry activations and dequantised weights as fp16: rows are scaled by a power of two first,
    so activations far outside fp16's range (and rows of very different magnitude side by side) must come out as the
    oracle has them, row by row; scales from fp16's smallest normal up to 32, negative and zero ones included."""
    t, h, f, e, top_k = 160, 512, 768, 4, 2
    host, dev = _experts(9100, e, h, f)
    r = rng(9101)
    # scales: magnitudes 2^-14 .. 2^5 for the gate/up matrices (|dequantised weight| up to 256), signs mixed, some zero
    host2, dev2 = [], []
    from chadslab_amd import QWeightInt4G32
    for tr in host:
        hw, dw = [], []
        for i in range(3):
            p, s = tr[2 * i], tr[2 * i + 1].astype(np.float32)
            if i < 2:
                mag = np.exp2(r.integers(-14, 6, s.shape)).astype(np.float32) * (1 + r.random(s.shape).astype(np.float32) * 0.99)
                sgn = np.where(r.random(s.shape) < 0.3, -1.0, 1.0).astype(np.float32)
                s = (mag * sgn * (r.random(s.shape) > 0.05)).astype(np.float32)
            s16 = s.astype(np.float16)
            hw += [p, s16]
            dw.append(QWeightInt4G32(torch.from_numpy(p).to(DEV), torch.from_numpy(s16).to(DEV)))
        host2.append(tuple(hw))
        dev2.append(tuple(dw))
    x = r.standard_normal((t, h)).astype(np.float32)
    x *= np.exp2(r.integers(-40, 41, (t, 1))).astype(np.float32)   # rows from 2^-40 to 2^40
    x[3] = 0.0                                                       # an all-zero row
    x[5, ::7] *= 2.0 ** 20                                           # a row with a few huge elements beside tiny ones
    xb = O.f32_to_bf16(x)
    logits = r.standard_normal((t, e)).astype(np.float32)
    tiled = [tuple(ops.to_tiles(m) for m in tr) for tr in dev2]
    with np.errstate(over="ignore", invalid="ignore"):
        ref = O.bf16_to_f32(O.moe_qffn(xb, logits, host2, top_k, True))
    y = O.bf16_to_f32(bits(ops.moe_ffn(bf16_tensor(xb), torch.from_numpy(logits).to(DEV), tiled, top_k=top_k, renorm=True)))
    fin = np.isfinite(ref).all(axis=1)
    assert fin.sum() >= t // 2                      # the case is not degenerate
    assert np.isfinite(y[fin]).all()
    for row in np.nonzero(fin)[0]:                  # row by row: every row has its own magnitude
        n = np.linalg.norm(ref[row].astype(np.float64))
        if n == 0:
            assert not y[row].any()
        else:
            assert np.linalg.norm((y[row] - ref[row]).astype(np.float64)) <= TOL_BF16 * n, row
    assert not np.isfinite(y[~fin]).all(axis=1).any() or not (~fin).any()  # rows the oracle overflows on overflow here too


def test_moe_ffn_tiled_refuses_mixed_and_unaligned_shapes(ops):
    host, dev = _experts(8900, 2, 256, 256)
    tiled = [tuple(ops.to_tiles(m) for m in tr) for tr in dev]
    x = torch.zeros(8, 256, dtype=torch.bfloat16, device=DEV)
    z = torch.zeros(8, 2, device=DEV)
    with pytest.raises(TypeError):
        ops.moe_ffn(x, z, [tiled[0], dev[1]], top_k=1)
    # H = 288 is a multiple of 32 (fine for the row-major entry point) but not of 256: the tiled one refuses it
    from chadslab_amd import _lib
    lib = _lib.load()
    need = lib.chadq_moe_ffn_i4g32_workspace_bytes(8, 288, 256, 1, 1)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    arr = (_lib.MoeExpertI4G32 * 1)(_lib.MoeExpertI4G32(*[ws.data_ptr()] * 6))
    y = torch.empty(8, 288, dtype=torch.bfloat16, device=DEV)
    x2 = torch.zeros(8, 288, dtype=torch.bfloat16, device=DEV)
    z1 = torch.zeros(8, 1, device=DEV)
    assert lib.chadq_moe_ffn_i4g32_tiled(x2.data_ptr(), z1.data_ptr(), arr, y.data_ptr(), 8, 288, 256, 1, 1, 1, ws.data_ptr(), need, None) == -2

"""GPU coverage of what sits upstream of the hot path: the quantisers run on the device and must produce the packed
bytes and scales of the oracle's quantisers bit for bit; a weight container written to disk and loaded straight to the
GPU must feed the HIP GEMV / GEMM within tolerance of the float64 truth; and a decoder saved and loaded again must
take exactly the step it took on the original weights.
"""
import numpy as np
import pytest
import torch

from oracle import chadq_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def bf16_tensor(b):
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16).to(DEV)


@pytest.mark.parametrize("n,k,std", [(64, 128, 1.0), (300, 4096, 0.02), (2048, 2048, 0.05), (17, 32, 3.0)])
def test_device_quantisers_equal_the_oracle_bit_for_bit(n, k, std):
    from chadslab_amd import _lib
    from chadslab_amd.formats import quantize_int4_g32, quantize_int8_row

    _lib.load()
    r = rng(n + k)
    w = (r.standard_normal((n, k)) * std).astype(np.float32)
    w[0, :32] = 0.0                      # an all-zero group: scale 0, every nibble 8
    w[1 % n, 5] = np.float32(3.0e5)      # a group whose absmax / 7 is large but finite in fp16
    w[2 % n, 40 % k] = -w[2 % n, 40 % k]
    wd = torch.from_numpy(w).to(DEV)
    q4 = quantize_int4_g32(wd)
    assert q4.packed.is_cuda and q4.scale.is_cuda
    p, s = O.quantize_int4_g32(w)
    assert np.array_equal(q4.packed.cpu().numpy(), p)
    assert np.array_equal(q4.scale.cpu().numpy().view(np.uint16), s.view(np.uint16))
    q8 = quantize_int8_row(wd)
    w8, s8 = O.quantize_int8_row(w)
    assert np.array_equal(q8.w.cpu().numpy(), w8)
    assert np.array_equal(q8.scale.cpu().numpy().view(np.uint32), s8.view(np.uint32))


def test_device_quantiser_saturates_instead_of_overflowing_fp16_and_refuses_non_finite_weights():
    from chadslab_amd.formats import quantize_int4_g32, quantize_int8_row

    w = np.zeros((2, 64), np.float32)
    w[0, 3] = 1.0e6      # absmax / 7 = 142857 > 65504: the scale is held at 65504 and the value saturates at 7
    w[0, 4] = -1.0e6
    w[1, 40] = 1.0
    q = quantize_int4_g32(torch.from_numpy(w).to(DEV))
    p, s = O.quantize_int4_g32(w)
    assert np.array_equal(q.packed.cpu().numpy(), p) and np.array_equal(q.scale.cpu().numpy().view(np.uint16), s.view(np.uint16))
    assert np.isfinite(q.scale.cpu().numpy().astype(np.float32)).all()
    u = O.unpack_int4(p)
    assert u[0, 3] == 7 and u[0, 4] == -8
    for bad in (np.nan, np.inf):
        w2 = w.copy()
        w2[1, 1] = bad
        with pytest.raises(ValueError):
            quantize_int4_g32(torch.from_numpy(w2).to(DEV))
        with pytest.raises(ValueError):
            quantize_int8_row(torch.from_numpy(w2).to(DEV))


def test_weight_file_loaded_to_the_gpu_feeds_gemv_and_gemm(tmp_path):
    from chadslab_amd import ops, wfile
    from chadslab_amd.formats import quantize_int4_g32, quantize_int8_row

    r = rng(71)
    w4 = (r.standard_normal((1536, 4096)) * 0.03).astype(np.float32)
    w8 = (r.standard_normal((640, 2048)) * 0.03).astype(np.float32)
    norm = (1 + 0.1 * r.standard_normal(4096)).astype(np.float32)
    path = str(tmp_path / "m.chadqw")
    wfile.save(path, {"up": quantize_int4_g32(torch.from_numpy(w4).to(DEV)), "proj": quantize_int8_row(torch.from_numpy(w8).to(DEV)),
                      "norm": torch.from_numpy(norm)}, meta={"note": "gpu round trip"})
    old_slab = wfile.SLAB_BYTES
    wfile.SLAB_BYTES = 1 << 20  # several slabs per array
    try:
        t = wfile.load(path, DEV)
    finally:
        wfile.SLAB_BYTES = old_slab
    up, proj = t["up"], t["proj"]
    assert up.packed.is_cuda and up.scale.is_cuda and proj.w.is_cuda and t["norm"].is_cuda
    p, s = O.quantize_int4_g32(w4)
    q8, s8 = O.quantize_int8_row(w8)
    assert np.array_equal(up.packed.cpu().numpy(), p) and np.array_equal(up.scale.cpu().numpy().view(np.uint16), s.view(np.uint16))
    assert np.array_equal(proj.w.cpu().numpy(), q8) and np.array_equal(proj.scale.cpu().numpy(), s8)
    assert np.array_equal(t["norm"].cpu().numpy(), norm)
    # the loaded containers feed the HIP path
    for m in (1, 8):
        xb = O.f32_to_bf16(r.standard_normal((m, 4096)).astype(np.float32))
        assert O.rel_l2(ops.qgemv(bf16_tensor(xb), up).cpu().numpy(), O.qgemm_int4g32_f64(xb, p, s)) <= 1e-3
    xb = O.f32_to_bf16(r.standard_normal((200, 4096)).astype(np.float32))
    assert O.rel_l2(O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb), up))), O.qgemm_int4g32_f64(xb, p, s)) <= 1e-2
    x8 = r.standard_normal((3, 2048)).astype(np.float32)
    assert O.rel_l2(ops.qgemv(torch.from_numpy(x8).to(DEV), proj).cpu().numpy(), O.qgemv_int8_f64(x8, q8, s8)) <= 1e-3
    xb8 = O.f32_to_bf16(r.standard_normal((130, 2048)).astype(np.float32))
    assert O.rel_l2(O.bf16_to_f32(bits(ops.qgemm(bf16_tensor(xb8), proj))), O.qgemm_int8_f64(xb8, q8, s8)) <= 1e-2


def test_decoder_saved_and_loaded_takes_the_same_steps(tmp_path):
    from chadslab_amd.decoder import DecoderConfig, QuantDecoder, load_weights, random_weights, save_weights

    cfg = DecoderConfig(n_layers=2, d=512, hq=4, dh=64, ffn=4096, vocab=3000, max_ctx=128)
    w = random_weights(cfg, 72, DEV)
    path = str(tmp_path / "dec.chadqw")
    save_weights(path, cfg, w)
    cfg2, w2 = load_weights(path, DEV)
    assert cfg2 == cfg
    a, b = QuantDecoder(cfg, w, DEV), QuantDecoder(cfg2, w2, DEV)
    b.capture()
    sa, sb = a.generate(7, 0, 10), b.generate(7, 0, 10)
    assert sa == sb
    assert np.array_equal(a.logits.cpu().numpy(), b.logits.cpu().numpy())  # same weights, same kernels: same bits

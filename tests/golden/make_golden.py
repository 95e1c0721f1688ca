"""Writes the golden fixtures in this folder from the CPU oracle (oracle/chadq_oracle.py).

The reference snapshot holds no implementation, test vector or fixture for this path, so these vectors are
the oracle's own outputs on seeded inputs (PCG64), frozen so that the oracle cannot drift unnoticed and so
that the GPU tests have inputs that do not depend on numpy's generator staying bit-stable.  Small on purpose
(N=64, K=128 and similar).  Run from the repo root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import chadq_oracle as O  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    rng = np.random.Generator(np.random.PCG64(20240001))
    # int4 group-32, N=64 K=128, M=8
    n, k, m = 64, 128, 8
    q = rng.integers(-8, 8, (n, k), dtype=np.int8)
    packed = O.pack_int4(q)
    scale = rng.lognormal(-5, 0.5, (n, k // 32)).astype(np.float16)
    x = O.f32_to_bf16(rng.standard_normal((m, k)).astype(np.float32))
    np.savez(
        os.path.join(HERE, "i4g32_n64_k128.npz"),
        q=q, packed=packed, scale=scale, x_bf16=x,
        dequant=O.dequant_int4g32(packed, scale),
        y_f64=O.qgemm_int4g32_f64(x, packed, scale),
        y_f32=O.qgemv_int4g32(x, packed, scale),
        y_bf16=O.qgemm_int4g32_bf16(x, packed, scale),
    )
    # int8 per-row, N=64 K=128, M=4
    w8 = rng.integers(-127, 128, (n, k), dtype=np.int8)
    s8 = rng.uniform(0.001, 0.02, n).astype(np.float32)
    x32 = rng.standard_normal((4, k)).astype(np.float32)
    xb = O.f32_to_bf16(x32)
    np.savez(
        os.path.join(HERE, "i8row_n64_k128.npz"),
        w=w8, scale=s8, x_f32=x32, x_bf16=xb,
        dequant=O.dequant_int8(w8, s8),
        y_f64=O.qgemv_int8_f64(x32, w8, s8),
        y_f32=O.qgemv_int8(x32, w8, s8),
        yb_f64=O.qgemm_int8_f64(xb, w8, s8),
        yb_bf16=O.qgemm_int8_bf16(xb, w8, s8),
    )
    # router + MoE, T=16 tokens, H=64, F=96, E=4
    t, h, f, e = 16, 64, 96, 4
    logits = rng.standard_normal((t, e)).astype(np.float32)
    logits[3, 1] = logits[3, 2]  # a constructed tie
    xm = O.f32_to_bf16(rng.standard_normal((t, h)).astype(np.float32))
    experts = []
    flat = {}
    for i in range(e):
        ws = []
        for name, shape in (("g", (f, h)), ("u", (f, h)), ("d", (h, f))):
            p, s = O.quantize_int4_g32((rng.standard_normal(shape) * 0.05).astype(np.float32))
            ws += [p, s]
            flat["e%d_%s_p" % (i, name)] = p
            flat["e%d_%s_s" % (i, name)] = s
        experts.append(tuple(ws))
    idx, w = O.moe_route(logits, 2, True)
    np.savez(
        os.path.join(HERE, "moe_t16_h64_f96_e4.npz"),
        logits=logits, x_bf16=xm, idx=idx, w=w, y_bf16=O.moe_qffn(xm, logits, experts, 2, True), **flat,
    )
    print("wrote fixtures to", HERE)


if __name__ == "__main__":
    main()

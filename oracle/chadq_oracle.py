"""CPU oracle for the quantized-weight matrix-product path.  TEST INFRASTRUCTURE ONLY.

This module is the checker: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it.  Nothing under chadslab_amd/ does.

What it restates
----------------
The reference snapshot (happycube/chadslab) holds no quantized-matmul code: no
numpy-gemma/, no reclank/, no int4/int8 unpack, dequant, GEMV or GEMM (its
top level is README, ancientARMS/, hsv2.c, kaggle/, m++/, m6502/, notebooks/,
nv-fansetup/, ppmproc.cxx, sand/, talks/).  So there is no reference file:line
for any function below.  Each one restates, in the plainest numpy a CPU runtime
would use, the closed form the benchmark configuration text gives:

  config 0  y = x . (W . s)^T, W int8 [N,K], s fp32 [N] per output row
  config 1  W int4 packed 2 per byte, group 32 along K, fp16 scale per group,
            symmetric (zero-point 8), fp32 out
  config 2  same weights, fp32 accumulate, bf16 out
  config 3  softmax top-2 routing, SiLU-gated experts, bf16 out
  config 4  Gemma-2B-shaped decoder step

Layout choices that the configuration text leaves open are this build's own
and are stated where they are made (nibble order, top-2 renormalisation, the
gate/up reading, the rounding of the MoE intermediate).  PARITY UNPINNED
against the reference for those choices: nothing in the snapshot can pin them.
What pins every function instead (tests/test_oracle_*.py): exhaustive
enumeration for pack/unpack, triple-loop brute force on tiny shapes, special
cases with exact answers, library cross-checks (scipy softmax, torch silu,
torch bf16 rounding, torch matmul), int64 brute force for the exact-integer
accumulation case, and the independent scalar C twin in chadq_oracle.c.
"""
from __future__ import annotations

import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

GROUP = 32          # int4 scale group length along K
ZERO_POINT = 8      # stored nibble u = q + 8, q in [-8, 7]


# --------------------------------------------------------------------------- bf16
def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    """uint16 bf16 bit patterns -> float32 (exact: bf16 is the top half of fp32)."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round-to-nearest-even; NaN stays a quiet NaN."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16), rounded)
    return rounded


# --------------------------------------------------------------------------- int4 pack
def pack_int4(q: np.ndarray) -> np.ndarray:
    """q int8 [N,K] with values in [-8,7] -> uint8 [N,K/2].

    BUILD CHOICE (nibble order): byte j of a row holds k=2j in its low nibble and
    k=2j+1 in its high nibble, K contiguous; stored nibble is q+8.
    """
    q = np.asarray(q)
    if q.ndim != 2 or q.shape[1] % 2:
        raise ValueError("pack_int4 wants [N,K] with even K")
    if q.min(initial=0) < -8 or q.max(initial=0) > 7:
        raise ValueError("int4 values must lie in [-8,7]")
    u = (q.astype(np.int16) + ZERO_POINT).astype(np.uint8)
    return (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)


def unpack_int4(wp: np.ndarray) -> np.ndarray:
    """uint8 [N,K/2] -> int8 [N,K] in [-8,7]; inverse of pack_int4."""
    wp = np.asarray(wp, dtype=np.uint8)
    n, kh = wp.shape
    q = np.empty((n, kh * 2), dtype=np.int8)
    q[:, 0::2] = (wp & 0x0F).astype(np.int8) - ZERO_POINT
    q[:, 1::2] = (wp >> 4).astype(np.int8) - ZERO_POINT
    return q


# --------------------------------------------------------------------------- tile order
def tile_int4g32(wp: np.ndarray, scale_f16: np.ndarray):
    """Row-major (wp uint8 [N,K/2], scale fp16 [N,K/32]) -> tile order, same shapes.

    BUILD CHOICE (a layout of this build, no reference counterpart).  Packed bytes: the matrix is cut into units of
    32 rows x 256 k; unit (b, c) occupies 4096 contiguous bytes at ((b * K/256) + c) * 4096, and inside it the 16-byte
    piece (one scale group) of row r and group g sits at (g * 32 + r) * 16.  Scales: block (b, c) = the same 32 rows x
    8 groups is 512 bytes at ((b * K/256) + c) * 512, the scale of row r and group g at
    ((g % 2) * 32 + r) * 8 + (g // 2) * 2.  N % 32 == 0, K % 256 == 0.
    """
    wp = np.ascontiguousarray(wp, dtype=np.uint8)
    sc = np.ascontiguousarray(scale_f16).view(np.uint16)
    n, kh = wp.shape
    k = kh * 2
    if n % 32 or k % 256 or sc.shape != (n, k // GROUP):
        raise ValueError("tile order needs N % 32 == 0, K % 256 == 0 and scales [N,K/32]")
    tiles = wp.reshape(n // 32, 32, k // 256, 8, 16).transpose(0, 2, 3, 1, 4)   # [band, unit, group, row, 16 B]
    st = sc.reshape(n // 32, 32, k // 256, 4, 2).transpose(0, 2, 4, 1, 3)       # [band, unit, parity, row, group // 2]
    return (np.ascontiguousarray(tiles).reshape(n, kh),
            np.ascontiguousarray(st).reshape(n, k // GROUP).view(np.float16))


def untile_int4g32(wp_tiles: np.ndarray, scale_tiles: np.ndarray):
    """Inverse of tile_int4g32."""
    wt = np.ascontiguousarray(wp_tiles, dtype=np.uint8)
    stl = np.ascontiguousarray(scale_tiles).view(np.uint16)
    n, kh = wt.shape
    k = kh * 2
    if n % 32 or k % 256 or stl.shape != (n, k // GROUP):
        raise ValueError("tile order needs N % 32 == 0, K % 256 == 0 and scales [N,K/32]")
    rows = wt.reshape(n // 32, k // 256, 8, 32, 16).transpose(0, 3, 1, 2, 4)    # [band, row, unit, group, 16 B]
    sr = stl.reshape(n // 32, k // 256, 2, 32, 4).transpose(0, 3, 1, 4, 2)      # [band, row, unit, group // 2, parity]
    return (np.ascontiguousarray(rows).reshape(n, kh),
            np.ascontiguousarray(sr).reshape(n, k // GROUP).view(np.float16))


# --------------------------------------------------------------------------- dequant
def dequant_int8(w: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """W int8 [N,K], scale fp32 [N] -> fp32 [N,K] = W[n,k] * s[n]."""
    return w.astype(np.float32) * np.asarray(scale, dtype=np.float32)[:, None]


def dequant_int4g32(wp: np.ndarray, scale_f16: np.ndarray) -> np.ndarray:
    """packed uint8 [N,K/2], scale fp16 [N,K/32] -> fp32 [N,K] = (u-8) * float(s[n,k//32]).

    The product is exact in fp32 (4-bit integer times 11-bit significand).
    """
    q = unpack_int4(wp).astype(np.float32)
    s = np.asarray(scale_f16, dtype=np.float16).astype(np.float32)
    if s.shape != (q.shape[0], q.shape[1] // GROUP):
        raise ValueError("scale must be [N, K/32]")
    return q * np.repeat(s, GROUP, axis=1)


# --------------------------------------------------------------------------- GEMV / GEMM
def qgemv_int8(x: np.ndarray, w: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """Config 0 as a numpy runtime computes it: y = x . (W . s)^T, all fp32.  x [M,K] -> [M,N]."""
    return np.asarray(x, dtype=np.float32) @ dequant_int8(w, scale).T


def qgemv_int8_f64(x, w, scale) -> np.ndarray:
    """Ground truth for config 0 in float64."""
    wd = w.astype(np.float64) * np.asarray(scale, dtype=np.float32).astype(np.float64)[:, None]
    return np.asarray(x, dtype=np.float32).astype(np.float64) @ wd.T


def qgemm_int4g32_f64(x_bf16: np.ndarray, wp: np.ndarray, scale_f16: np.ndarray) -> np.ndarray:
    """Ground truth: float64 product of the bf16 activations with the exactly dequantised weights."""
    x = bf16_to_f32(x_bf16).astype(np.float64)
    return x @ dequant_int4g32(wp, scale_f16).astype(np.float64).T


CHUNK_ELEMS = 1 << 20   # weights dequantised at a time: a worker's fp32 copy (4 MB) stays in its cache
WORKERS = min(8, os.cpu_count() or 1)


def qgemv_int4g32(x_bf16: np.ndarray, wp: np.ndarray, scale_f16: np.ndarray) -> np.ndarray:
    """Configs 1: x bf16 bits [M,K] -> fp32 [M,N]; dequantise to fp32, then an fp32 matmul.  A matrix of more than
    CHUNK_ELEMS weights is handled in blocks of whole rows, a few at a time on worker threads (numpy releases the
    interpreter lock inside its loops): each output column depends on its own weight row only, so the blocks are
    independent and the result does not depend on how many workers there are."""
    x = bf16_to_f32(x_bf16)
    n, k = wp.shape[0], wp.shape[1] * 2
    rows = max(1, CHUNK_ELEMS // max(1, k))
    if n <= rows:
        return x @ dequant_int4g32(wp, scale_f16).T

    def block(r):
        return x @ dequant_int4g32(wp[r: r + rows], scale_f16[r: r + rows]).T

    with ThreadPoolExecutor(WORKERS) as ex:
        return np.concatenate(list(ex.map(block, range(0, n, rows))), axis=1)


def qgemm_int4g32_bf16(x_bf16, wp, scale_f16) -> np.ndarray:
    """Config 2: fp32 accumulate, bf16 (RNE) out.  Returns bf16 bit patterns [M,N]."""
    return f32_to_bf16(qgemv_int4g32(x_bf16, wp, scale_f16))


def qgemm_int8_bf16(x_bf16, w, scale) -> np.ndarray:
    """Config 2's int8 variant: x bf16 [M,K], W int8 per-row scale, bf16 (RNE) out."""
    return f32_to_bf16(bf16_to_f32(x_bf16) @ dequant_int8(w, scale).T)


def qgemm_int8_f64(x_bf16, w, scale) -> np.ndarray:
    wd = w.astype(np.float64) * np.asarray(scale, dtype=np.float32).astype(np.float64)[:, None]
    return bf16_to_f32(x_bf16).astype(np.float64) @ wd.T


# --------------------------------------------------------------------------- MoE
def softmax(logits: np.ndarray) -> np.ndarray:
    z = np.asarray(logits, dtype=np.float32)
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)


def moe_route(logits: np.ndarray, top_k: int = 2, renorm: bool = True):
    """softmax over experts, then the top_k largest probabilities per token.

    Ties go to the lower expert index (a stable sort of -p).  BUILD CHOICE:
    renorm=True divides the selected weights by their sum (they then add to 1).
    Returns (idx int32 [T,top_k], w fp32 [T,top_k]).
    """
    p = softmax(logits)
    # softmax is monotonic, so the top_k probabilities belong to the top_k logits; ordering by the logits
    # themselves keeps the choice independent of the last bit of exp() (a CPU and a GPU exp may differ there)
    z = np.asarray(logits, dtype=np.float32)
    idx = np.argsort(-z, axis=-1, kind="stable")[:, :top_k].astype(np.int32)
    w = np.take_along_axis(p, idx, axis=-1)
    if renorm:
        w = w / w.sum(axis=-1, keepdims=True)
    return idx, w.astype(np.float32)


def silu(x: np.ndarray) -> np.ndarray:
    x = np.asarray(x, dtype=np.float32)
    return (x / (np.float32(1) + np.exp(-x))).astype(np.float32)


def moe_qffn(x_bf16, logits, experts, top_k: int = 2, renorm: bool = True) -> np.ndarray:
    """Config 3.  experts: list of (wg_p, wg_s, wu_p, wu_s, wd_p, wd_s), int4-g32.

    BUILD CHOICES: gate and up are two separate [F,H] matrices; the intermediate
    h = silu(x Wg^T) * (x Wu^T) is rounded to bf16 before the down projection
    (the down GEMM consumes bf16); the weighted sum over the selected experts is
    accumulated in fp32 and rounded to bf16 once.  Returns bf16 bits [T,H].
    """
    idx, w = moe_route(logits, top_k, renorm)
    t, h_dim = x_bf16.shape
    y = np.zeros((t, h_dim), dtype=np.float32)
    for e, (wg_p, wg_s, wu_p, wu_s, wd_p, wd_s) in enumerate(experts):
        tok, slot = np.nonzero(idx == e)
        if tok.size == 0:
            continue
        xe = x_bf16[tok]
        g = qgemv_int4g32(xe, wg_p, wg_s)
        u = qgemv_int4g32(xe, wu_p, wu_s)
        hmid = f32_to_bf16(silu(g) * u)
        d = qgemv_int4g32(hmid, wd_p, wd_s)
        y[tok] += w[tok, slot][:, None] * d
    return f32_to_bf16(y)


# --------------------------------------------------------------------------- quantiser (next-row helper)
def quantize_int4_g32(w: np.ndarray):
    """fp32 [N,K] -> (packed uint8 [N,K/2], scale fp16 [N,K/32]); min(absmax/7, 65504) per group, RNE, clamp to [-8,7]."""
    w = np.asarray(w, dtype=np.float32)
    n, k = w.shape
    g = w.reshape(n, k // GROUP, GROUP)
    s = np.minimum(np.abs(g).max(axis=2) / np.float32(7), np.float32(65504)).astype(np.float16)  # largest fp16: no inf scale
    sf = s.astype(np.float32)
    sf_safe = np.where(sf == 0, np.float32(1), sf)
    q = np.clip(np.rint(g / sf_safe[:, :, None]), -8, 7).astype(np.int8).reshape(n, k)
    return pack_int4(q), s


def quantize_int8_row(w: np.ndarray):
    """fp32 [N,K] -> (int8 [N,K], scale fp32 [N]); absmax/127 per row, RNE."""
    w = np.asarray(w, dtype=np.float32)
    s = (np.abs(w).max(axis=1) / np.float32(127)).astype(np.float32)
    s_safe = np.where(s == 0, np.float32(1), s)
    q = np.clip(np.rint(w / s_safe[:, None]), -127, 127).astype(np.int8)
    return q, s


def rel_l2(a: np.ndarray, ref: np.ndarray) -> float:
    a = np.asarray(a, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    d = np.linalg.norm(ref)
    return float(np.linalg.norm(a - ref) / (d if d > 0 else 1.0))


# --------------------------------------------------------------------------- decode step (config 4)
# Conventions (this build's plain choices; the benchmark text fixes shapes only, so parity with the
# reference is unpinned here): RMSNorm y = x / sqrt(mean(x^2) + eps) * w; rotate-half RoPE, base 10000;
# multi-query attention (one KV head), scores / sqrt(dh), KV cache in bf16; GeGLU with tanh-GELU; tied int4
# embedding / output table, no embedding scaling, no logit soft-cap; residual stream in fp32; every GEMV
# input rounded to bf16 (that is what the kernels consume).
def rmsnorm(x, w, eps):
    x = np.asarray(x, dtype=np.float32)
    return (x / np.sqrt(np.mean(x * x, dtype=np.float32) + np.float32(eps)) * np.asarray(w, dtype=np.float32)).astype(np.float32)


def rope_rotate_half(v, pos, base=10000.0):
    """v fp32 [..., dh]: pairs (j, j+dh/2) rotated by pos * base^(-2j/dh)."""
    v = np.asarray(v, dtype=np.float32)
    dh = v.shape[-1]
    half = dh // 2
    inv = np.power(np.float32(base), (-2.0 * np.arange(half, dtype=np.float32) / np.float32(dh)).astype(np.float32)).astype(np.float32)
    ang = (np.float32(pos) * inv).astype(np.float32)
    cs, sn = np.cos(ang.astype(np.float64)).astype(np.float32), np.sin(ang.astype(np.float64)).astype(np.float32)
    a, b = v[..., :half], v[..., half:]
    return np.concatenate([a * cs - b * sn, b * cs + a * sn], axis=-1).astype(np.float32)


def gelu_tanh(x):
    x = np.asarray(x, dtype=np.float32)
    return (0.5 * x * (1.0 + np.tanh(np.float32(0.7978845608028654) * (x + np.float32(0.044715) * x * x * x)))).astype(np.float32)


def decode_layer(L, x, pos, kcache, vcache, hq, dh, eps=1e-6, base=10000.0):
    """One decoder layer on the fp32 residual vector x [d]: attention block, then the gated FFN block.  L: {"ln1",
    "wqkv", "wo", "ln2", "wgu", "wd"} with weights as (packed, scale) tuples; kcache/vcache: this layer's bf16 bit
    arrays [max_ctx, dh], row `pos` is written.  Returns the residual vector after the layer."""
    xn = f32_to_bf16(rmsnorm(x, L["ln1"], eps))[None, :]
    qkv = qgemv_int4g32(xn, *L["wqkv"])[0]
    q = rope_rotate_half(qkv[: hq * dh].reshape(hq, dh), pos, base)
    k = rope_rotate_half(qkv[hq * dh: (hq + 1) * dh], pos, base)
    v = qkv[(hq + 1) * dh:]
    kcache[pos] = f32_to_bf16(k)
    vcache[pos] = f32_to_bf16(v)
    kk = bf16_to_f32(kcache[: pos + 1])
    vv = bf16_to_f32(vcache[: pos + 1])
    sc = (q @ kk.T) / np.float32(np.sqrt(dh))
    sc = sc - sc.max(axis=-1, keepdims=True)
    p = np.exp(sc)
    p = p / p.sum(axis=-1, keepdims=True)
    att = f32_to_bf16((p @ vv).astype(np.float32)).reshape(1, hq * dh)
    x = x + qgemv_int4g32(att, *L["wo"])[0]
    xn = f32_to_bf16(rmsnorm(x, L["ln2"], eps))[None, :]
    gu = qgemv_int4g32(xn, *L["wgu"])[0]
    f = gu.shape[0] // 2
    h = f32_to_bf16(gelu_tanh(gu[:f]) * gu[f:])[None, :]
    return x + qgemv_int4g32(h, *L["wd"])[0]


def decode_logits(model, x, eps=1e-6):
    """Final norm and the tied output table on the residual vector x [d]: fp32 logits [V]."""
    xn = f32_to_bf16(rmsnorm(x, model["lnf"], eps))[None, :]
    return qgemv_int4g32(xn, *model["emb"])[0]


def decode_step(model, token, pos, kcache, vcache, hq, dh, eps=1e-6, base=10000.0):
    """One token of a decoder-only transformer on int4 group-32 weights.  model: {"layers": [{"ln1","wqkv",
    "wo","ln2","wgu","wd"}], "lnf", "emb"} with weights as (packed, scale) tuples.  kcache/vcache: per layer
    bf16 bit arrays [max_ctx, dh], row `pos` is written.  Returns fp32 logits [V]."""
    ep, es = model["emb"]
    x = dequant_int4g32(ep[token:token + 1], es[token:token + 1])[0]
    for li, L in enumerate(model["layers"]):
        x = decode_layer(L, x, pos, kcache[li], vcache[li], hq, dh, eps, base)
    return decode_logits(model, x, eps)


def sample_topk(v: np.ndarray, k: int, temperature: float, u: float) -> int:
    """Top-k sampling as the product defines it: candidates are the k largest logits, larger first and lower index
    first among equals (NaN never a candidate); p_j = exp((v_j - v_0) / temperature); the token is the first candidate
    whose running sum of p exceeds u * sum(p).  float64 arithmetic."""
    v = np.asarray(v, dtype=np.float64)
    idx = np.arange(v.size)[~np.isnan(v)]
    if idx.size == 0:
        return 0
    order = idx[np.lexsort((idx, -v[idx]))][:k]
    top = v[order[0]]
    if np.isneginf(top):
        return int(order[0])
    c = np.cumsum(np.exp((v[order] - top) / temperature))
    hit = np.nonzero(c > u * c[-1])[0]
    return int(order[hit[0]] if hit.size else order[-1])

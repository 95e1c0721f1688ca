"""Operator entry points: what a numpy-style LLM runtime's quantized `x @ dequant(W).T` call sites bind to.

Every function runs hand-written HIP kernels from libchadq.so through its C ABI (chadslab_amd/_lib.py) on
torch's current stream.  torch is used for device memory and streams only.  Nothing here computes on the
CPU: tensors must already be on the GPU, and a missing library raises.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from . import _lib
from .formats import QWeightInt4G32, QWeightInt4G32Tiles, QWeightInt8

QWeight = Union[QWeightInt4G32, QWeightInt8]
GEMV_MAX_M = 16  # decode batch sizes served by the bandwidth kernel


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str, dtype: torch.dtype) -> torch.Tensor:
    if not t.is_cuda:
        raise ValueError("%s must be a GPU tensor (there is no CPU path)" % name)
    if t.dtype != dtype:
        raise ValueError("%s must be %s, got %s" % (name, dtype, t.dtype))
    return t if t.is_contiguous() else t.contiguous()


def _out(out: Optional[torch.Tensor], shape, dtype: torch.dtype, device) -> torch.Tensor:
    """A caller's result tensor, checked before its address goes to the library; a fresh one if none was given."""
    if out is None:
        return torch.empty(*shape, dtype=dtype, device=device)
    if not out.is_cuda or out.device != device:
        raise ValueError("out must live on %s, got %s" % (device, out.device))
    if out.dtype != dtype or tuple(out.shape) != tuple(shape) or not out.is_contiguous():
        raise ValueError("out must be a contiguous %s tensor of shape %s, got %s %s" % (dtype, tuple(shape), out.dtype, tuple(out.shape)))
    return out


def unpack_int4(packed: torch.Tensor) -> torch.Tensor:
    """uint8 [..., K/2] -> int8 [..., K] in [-8,7] (low nibble = even k)."""
    p = _dev(packed, "packed", torch.uint8)
    out = torch.empty(*p.shape[:-1], p.shape[-1] * 2, dtype=torch.int8, device=p.device)
    _lib.check(_lib.load().chadq_unpack_i4(p.data_ptr(), out.data_ptr(), p.numel(), _stream()), "chadq_unpack_i4")
    return out


def pack_int4(q: torch.Tensor) -> torch.Tensor:
    """int8 [..., K] in [-8,7] -> uint8 [..., K/2]; inverse of unpack_int4."""
    q = _dev(q, "q", torch.int8)
    if q.shape[-1] % 2:
        raise ValueError("K must be even")
    out = torch.empty(*q.shape[:-1], q.shape[-1] // 2, dtype=torch.uint8, device=q.device)
    _lib.check(_lib.load().chadq_pack_i4(q.data_ptr(), out.data_ptr(), out.numel(), _stream()), "chadq_pack_i4")
    return out


def dequantize(qw: QWeight) -> torch.Tensor:
    """fp32 [N,K] dequantised weights (exact)."""
    lib = _lib.load()
    if isinstance(qw, QWeightInt4G32):
        p, s = _dev(qw.packed, "packed", torch.uint8), _dev(qw.scale, "scale", torch.float16)
        out = torch.empty(qw.N, qw.K, dtype=torch.float32, device=p.device)
        _lib.check(lib.chadq_dequant_i4g32(p.data_ptr(), s.data_ptr(), out.data_ptr(), qw.N, qw.K, _stream()),
                   "chadq_dequant_i4g32")
        return out
    if isinstance(qw, QWeightInt8):
        w, s = _dev(qw.w, "w", torch.int8), _dev(qw.scale, "scale", torch.float32)
        out = torch.empty(qw.N, qw.K, dtype=torch.float32, device=w.device)
        _lib.check(lib.chadq_dequant_i8row(w.data_ptr(), s.data_ptr(), out.data_ptr(), qw.N, qw.K, _stream()),
                   "chadq_dequant_i8row")
        return out
    raise TypeError("unknown weight container %r" % type(qw))


def qgemv(x: torch.Tensor, qw: QWeight, out: Optional[torch.Tensor] = None, *, fp32_elements: bool = False) -> torch.Tensor:
    """Decode product, fp32 out [M,N], M <= 16.  x is bf16 [M,K] for int4 weights, fp32 [M,K] for int8 weights.

    fp32_elements (int8 weights only): fp32 arithmetic on every activation (chadq_gemv_i8row_fp32) instead of the
    matrix-core kernel's per-block fixed point, whose error on a small activation grows with the largest one of its
    2048-k block; the weights are then streamed once per pair of activation rows."""
    lib = _lib.load()
    if x.dim() != 2 or x.shape[1] != qw.K:
        raise ValueError("x must be [M,%d], got %s" % (qw.K, tuple(x.shape)))
    m = x.shape[0]
    if fp32_elements and not isinstance(qw, QWeightInt8):
        raise ValueError("fp32_elements applies to int8 weights (fp32 activations) only")
    if isinstance(qw, QWeightInt4G32):
        x = _dev(x, "x", torch.bfloat16)
        p, s = _dev(qw.packed, "packed", torch.uint8), _dev(qw.scale, "scale", torch.float16)
        y = _out(out, (m, qw.N), torch.float32, x.device)
        _lib.check(lib.chadq_gemv_i4g32(x.data_ptr(), p.data_ptr(), s.data_ptr(), y.data_ptr(), m, qw.N, qw.K,
                                        _stream()), "chadq_gemv_i4g32")
        return y
    if isinstance(qw, QWeightInt8):
        x = _dev(x, "x", torch.float32)
        w, s = _dev(qw.w, "w", torch.int8), _dev(qw.scale, "scale", torch.float32)
        y = _out(out, (m, qw.N), torch.float32, x.device)
        fn, name = (lib.chadq_gemv_i8row_fp32, "chadq_gemv_i8row_fp32") if fp32_elements else (lib.chadq_gemv_i8row, "chadq_gemv_i8row")
        _lib.check(fn(x.data_ptr(), w.data_ptr(), s.data_ptr(), y.data_ptr(), m, qw.N, qw.K, _stream()), name)
        return y
    raise TypeError("unknown weight container %r" % type(qw))


def qgemm(x: torch.Tensor, qw: QWeight, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Prefill product on the matrix cores: x bf16 [M,K] -> bf16 [M,N], fp32 accumulate."""
    lib = _lib.load()
    if x.dim() != 2 or x.shape[1] != qw.K:
        raise ValueError("x must be [M,%d], got %s" % (qw.K, tuple(x.shape)))
    x = _dev(x, "x", torch.bfloat16)
    m = x.shape[0]
    y = _out(out, (m, qw.N), torch.bfloat16, x.device)
    if isinstance(qw, QWeightInt4G32):
        p, s = _dev(qw.packed, "packed", torch.uint8), _dev(qw.scale, "scale", torch.float16)
        _lib.check(lib.chadq_gemm_i4g32_bf16(x.data_ptr(), p.data_ptr(), s.data_ptr(), y.data_ptr(), m, qw.N, qw.K,
                                             _stream()), "chadq_gemm_i4g32_bf16")
    elif isinstance(qw, QWeightInt8):
        w, s = _dev(qw.w, "w", torch.int8), _dev(qw.scale, "scale", torch.float32)
        _lib.check(lib.chadq_gemm_i8row_bf16(x.data_ptr(), w.data_ptr(), s.data_ptr(), y.data_ptr(), m, qw.N, qw.K,
                                             _stream()), "chadq_gemm_i8row_bf16")
    else:
        raise TypeError("unknown weight container %r" % type(qw))
    return y


def qlinear(x: torch.Tensor, qw: QWeight, *, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """y = x @ dequant(W).T over the last axis of x.

    Up to 16 rows go to the bandwidth-bound GEMV (fp32 result); more rows go to the MFMA GEMM (bf16 result).
    out_dtype picks the result type; asking for the other type than the kernel's native one casts.
    """
    lead, k = x.shape[:-1], x.shape[-1]
    x2 = x.reshape(-1, k)
    m = x2.shape[0]
    use_gemv = m <= GEMV_MAX_M and not (isinstance(qw, QWeightInt8) and x2.dtype == torch.bfloat16)
    if isinstance(qw, QWeightInt8) and x2.dtype == torch.float32 and not use_gemv:
        raise ValueError("int8 weights with fp32 activations are served for at most %d rows" % GEMV_MAX_M)
    y = qgemv(x2, qw) if use_gemv else qgemm(x2, qw)
    if out_dtype is not None and y.dtype != out_dtype:
        y = y.to(out_dtype)
    return y.reshape(*lead, qw.N)


def moe_route(logits: torch.Tensor, top_k: int = 2, renorm: bool = True):
    """softmax over experts, top_k by logit (lowest index wins ties) -> (idx int32 [T,top_k], w fp32 [T,top_k])."""
    z = _dev(logits, "logits", torch.float32)
    t, e = z.shape
    idx = torch.empty(t, top_k, dtype=torch.int32, device=z.device)
    w = torch.empty(t, top_k, dtype=torch.float32, device=z.device)
    _lib.check(_lib.load().chadq_moe_route(z.data_ptr(), idx.data_ptr(), w.data_ptr(), t, e, top_k, int(renorm), _stream()),
               "chadq_moe_route")
    return idx, w


_moe_ws = {}  # (device, stream, bytes) -> workspace tensor, reused between calls on that stream


def _repack(w, to_tiles: bool):
    lib = _lib.load()
    p, s = _dev(w.packed, "packed", torch.uint8), _dev(w.scale, "scale", torch.float16)
    if w.N % 32 or w.K % 256:
        raise ValueError("tile order needs N % 32 == 0 and K % 256 == 0 (N=%d, K=%d)" % (w.N, w.K))
    po, so = torch.empty_like(p), torch.empty_like(s)
    fn = lib.chadq_repack_i4g32_tiles if to_tiles else lib.chadq_unrepack_i4g32_tiles
    _lib.check(fn(p.data_ptr(), s.data_ptr(), po.data_ptr(), so.data_ptr(), w.N, w.K, _stream()),
               "chadq_repack_i4g32_tiles" if to_tiles else "chadq_unrepack_i4g32_tiles")
    return po, so


def to_tiles(w: QWeightInt4G32) -> QWeightInt4G32Tiles:
    """Row-major int4 group-32 matrix (on the GPU) -> tile order, for the experts of moe_ffn.  Done once at load time."""
    if not isinstance(w, QWeightInt4G32):
        raise TypeError("to_tiles wants a QWeightInt4G32")
    return QWeightInt4G32Tiles(*_repack(w, True))


def to_rows(w: QWeightInt4G32Tiles) -> QWeightInt4G32:
    """The exact inverse of to_tiles."""
    if not isinstance(w, QWeightInt4G32Tiles):
        raise TypeError("to_rows wants a QWeightInt4G32Tiles")
    return QWeightInt4G32(*_repack(w, False))


def moe_ffn(x: torch.Tensor, logits: torch.Tensor, experts, *, top_k: int = 2, renorm: bool = True) -> torch.Tensor:
    """SiLU-gated mixture of experts.  x bf16 [T,H], logits fp32 [T,E]; experts: sequence of (gate, up, down)
    triples with gate/up [F,H] and down [H,F], all QWeightInt4G32 or all QWeightInt4G32Tiles (to_tiles(): faster, fp16
    instead of bf16 dequantised weights, so the same results within rounding).  Returns bf16 [T,H]."""
    lib = _lib.load()
    x = _dev(x, "x", torch.bfloat16)
    z = _dev(logits, "logits", torch.float32)
    t, h = x.shape
    e = len(experts)
    if z.shape != (t, e):
        raise ValueError("logits must be [%d,%d]" % (t, e))
    f = experts[0][0].N
    kinds = {type(m) for tr in experts for m in tr}
    if kinds not in ({QWeightInt4G32}, {QWeightInt4G32Tiles}):
        raise TypeError("the experts' matrices must all be QWeightInt4G32 or all QWeightInt4G32Tiles")
    tiled = kinds == {QWeightInt4G32Tiles}
    arr = (_lib.MoeExpertI4G32 * e)()
    keep = []
    for i, (g, u, d) in enumerate(experts):
        if (g.N, g.K) != (f, h) or (u.N, u.K) != (f, h) or (d.N, d.K) != (h, f):
            raise ValueError("expert %d: gate/up must be [%d,%d] and down [%d,%d]" % (i, f, h, h, f))
        ts = [_dev(g.packed, "gate", torch.uint8), _dev(g.scale, "gate scale", torch.float16),
              _dev(u.packed, "up", torch.uint8), _dev(u.scale, "up scale", torch.float16),
              _dev(d.packed, "down", torch.uint8), _dev(d.scale, "down scale", torch.float16)]
        keep.append(ts)
        arr[i] = _lib.MoeExpertI4G32(*[v.data_ptr() for v in ts])
    need = lib.chadq_moe_ffn_i4g32_workspace_bytes(t, h, f, e, top_k)
    if need == 0:
        raise ValueError("unsupported MoE sizes T=%d H=%d F=%d E=%d top_k=%d" % (t, h, f, e, top_k))
    # The workspace holds the router's output and every intermediate of the call, so two calls in flight at once must
    # not share one: calls on one stream are ordered and reuse theirs, another stream gets its own.  A graph captured
    # on a stream keeps using that stream's workspace on every replay: do not run eager calls of the same sizes on the
    # capture stream while a replay is in flight.
    key = (x.device, _stream(), need)
    ws = _moe_ws.get(key)
    if ws is None:
        ws = _moe_ws[key] = torch.empty(need, dtype=torch.uint8, device=x.device)
    y = torch.empty(t, h, dtype=torch.bfloat16, device=x.device)
    fn = lib.chadq_moe_ffn_i4g32_tiled if tiled else lib.chadq_moe_ffn_i4g32
    _lib.check(fn(x.data_ptr(), z.data_ptr(), arr, y.data_ptr(), t, h, f, e, top_k, int(renorm), ws.data_ptr(), need, _stream()),
               "chadq_moe_ffn_i4g32_tiled" if tiled else "chadq_moe_ffn_i4g32")
    return y

"""Quantized-weight containers and the host-side tools that produce them.

Layouts (this build's choices; the benchmark text fixes only "2 per byte", "group 32 along K",
"fp16 scale per group", "zero-point 8" and "per-output-row fp32 scale"):

  QWeightInt8     w      int8  [N, K]    row-major          value = w[n,k] * scale[n]
                  scale  fp32  [N]
  QWeightInt4G32  packed uint8 [N, K/2]  row-major          byte j of a row = u[2j] | (u[2j+1] << 4), u = q + 8
                  scale  fp16  [N, K/32]                    value = (u - 8) * scale[n, k // 32]
  QWeightInt4G32Tiles  the same bytes regrouped into contiguous tiles for the mixture-of-experts kernel (a load-time
                  repack on the device; the row-major form stays the interchange format)

The tensors live wherever the caller puts them; the operators in chadslab_amd.ops want them on the GPU.
Quantising and packing are load-time tools, not the hot path, and are written with torch tensor ops.
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

GROUP = 32
ZERO_POINT = 8
FP16_MAX = 65504.0


@dataclass
class QWeightInt8:
    w: torch.Tensor      # int8 [N, K]
    scale: torch.Tensor  # float32 [N]

    def __post_init__(self):
        if self.w.dtype != torch.int8 or self.w.dim() != 2:
            raise ValueError("QWeightInt8.w must be int8 [N,K]")
        if self.scale.dtype != torch.float32 or self.scale.shape != (self.w.shape[0],):
            raise ValueError("QWeightInt8.scale must be float32 [N]")

    @property
    def N(self) -> int:
        return self.w.shape[0]

    @property
    def K(self) -> int:
        return self.w.shape[1]

    def to(self, device) -> "QWeightInt8":
        return QWeightInt8(self.w.to(device).contiguous(), self.scale.to(device).contiguous())


@dataclass
class QWeightInt4G32:
    packed: torch.Tensor  # uint8 [N, K/2]
    scale: torch.Tensor   # float16 [N, K/32]

    def __post_init__(self):
        if self.packed.dtype != torch.uint8 or self.packed.dim() != 2:
            raise ValueError("QWeightInt4G32.packed must be uint8 [N,K/2]")
        n, kh = self.packed.shape
        if (kh * 2) % GROUP:
            raise ValueError("K must be a multiple of 32")
        if self.scale.dtype != torch.float16 or self.scale.shape != (n, kh * 2 // GROUP):
            raise ValueError("QWeightInt4G32.scale must be float16 [N,K/32]")

    @property
    def N(self) -> int:
        return self.packed.shape[0]

    @property
    def K(self) -> int:
        return self.packed.shape[1] * 2

    def to(self, device) -> "QWeightInt4G32":
        return QWeightInt4G32(self.packed.to(device).contiguous(), self.scale.to(device).contiguous())


@dataclass
class QWeightInt4G32Tiles:
    """An int4 group-32 matrix in tile order (chadq_repack_i4g32_tiles): what ops.moe_ffn streams fastest.  The arrays
    have the shapes of the row-major container but hold 32-row x 256-k units of packed bytes (4 KiB each, group-major)
    and 32-row x 8-group blocks of scales (512 B each) contiguously.  Made with ops.to_tiles(); ops.to_rows() is the
    inverse.  Scales must stay below 64 in magnitude for the expert kernel."""
    packed: torch.Tensor  # uint8 [N, K/2], tile order
    scale: torch.Tensor   # float16 [N, K/32], tile order

    def __post_init__(self):
        QWeightInt4G32(self.packed, self.scale)  # same shape and dtype rules
        if self.N % 32 or self.K % 256:
            raise ValueError("tile order needs N % 32 == 0 and K % 256 == 0")

    @property
    def N(self) -> int:
        return self.packed.shape[0]

    @property
    def K(self) -> int:
        return self.packed.shape[1] * 2


def pack_int4(q: torch.Tensor) -> torch.Tensor:
    """int8 [N,K] in [-8,7] -> uint8 [N,K/2]: low nibble = even k, high nibble = odd k, stored value q+8."""
    if q.dim() != 2 or q.shape[1] % 2:
        raise ValueError("pack_int4 wants [N,K] with even K")
    if q.numel() and (int(q.min()) < -8 or int(q.max()) > 7):
        raise ValueError("int4 values must lie in [-8,7]")
    u = (q.to(torch.int16) + ZERO_POINT).to(torch.uint8)
    return (u[:, 0::2] | (u[:, 1::2] << 4)).contiguous()


def quantize_int4_g32(w: torch.Tensor) -> QWeightInt4G32:
    """fp32 [N,K] -> int4 group-32: scale = min(absmax/7, 65504) per group (stored fp16), q = clamp(rne(w/scale), -8, 7).
    Raises on NaN or infinite weights."""
    w = w.to(torch.float32)
    n, k = w.shape
    if k % GROUP:
        raise ValueError("K must be a multiple of 32")
    if not bool(torch.isfinite(w).all()):
        raise ValueError("quantize_int4_g32: the matrix holds NaN or infinite values")
    g = w.reshape(n, k // GROUP, GROUP)
    # a group whose absmax / 7 exceeds the largest fp16 (65504) keeps that scale and saturates at -8 / 7
    # the divisor is a tensor on purpose: torch turns a division by a Python scalar on the GPU into a multiplication by
    # its reciprocal, which is not the correctly rounded quotient a CPU runtime (and the oracle) computes
    amax = g.abs().amax(dim=2)
    s = (amax / torch.full_like(amax, 7.0)).clamp(max=FP16_MAX).to(torch.float16)
    sf = s.to(torch.float32)
    sf = torch.where(sf == 0, torch.ones_like(sf), sf)
    q = torch.clamp(torch.round(g / sf[:, :, None]), -8, 7).to(torch.int8).reshape(n, k)
    return QWeightInt4G32(pack_int4(q), s.contiguous())


def quantize_int8_row(w: torch.Tensor) -> QWeightInt8:
    """fp32 [N,K] -> int8 per-row: scale = absmax/127 per row (fp32), q = clamp(rne(w/scale), -127, 127)."""
    w = w.to(torch.float32)
    if not bool(torch.isfinite(w).all()):
        raise ValueError("quantize_int8_row: the matrix holds NaN or infinite values")
    amax = w.abs().amax(dim=1)
    s = (amax / torch.full_like(amax, 127.0)).to(torch.float32)  # a tensor divisor: see quantize_int4_g32
    ss = torch.where(s == 0, torch.ones_like(s), s)
    q = torch.clamp(torch.round(w / ss[:, None]), -127, 127).to(torch.int8)
    return QWeightInt8(q.contiguous(), s.contiguous())

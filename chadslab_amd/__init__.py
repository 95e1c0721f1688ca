"""chadslab_amd: MI355X-native quantized-weight matrix products (int8 per-row, int4 group-32).

Hand-written HIP kernels for gfx950 behind a C ABI (include/chadq.h, chadslab_amd/libchadq.so); the Python
layer only moves pointers.  Build the library with `python -m chadslab_amd.build`.
"""
from .formats import QWeightInt4G32, QWeightInt4G32Tiles, QWeightInt8, pack_int4, quantize_int4_g32, quantize_int8_row  # noqa: F401

__all__ = ["QWeightInt4G32", "QWeightInt8", "pack_int4", "quantize_int4_g32", "quantize_int8_row", "ops"]

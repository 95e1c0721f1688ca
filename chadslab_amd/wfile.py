"""On-disk container for quantized weights: one file, a JSON header and 256-byte aligned raw arrays, readable by
memory map so that a multi-GB checkpoint is paged in by the copy to the GPU and never held twice on the host.

Layout (little endian):
    bytes 0..7    magic  b"CHADQW01"
    bytes 8..15   uint64 header length H
    bytes 16..    H bytes of UTF-8 JSON: {"tensors": {name: {"kind": "i4g32" | "i8row" | "raw", "shape": [...],
                  "arrays": {array_name: {"dtype": numpy dtype string, "shape": [...], "offset": bytes from file start,
                  "nbytes": ...}}}}, "meta": {...}}
    then the arrays, each starting on a 256-byte boundary, in the layouts of chadslab_amd.formats
    (i4g32: "packed" uint8 [N,K/2], "scale" float16 [N,K/32];  i8row: "w" int8 [N,K], "scale" float32 [N];
     raw: "data" of any dtype, e.g. norm weights).

The reference snapshot defines no checkpoint format for this path; this one is the build's own.
"""
from __future__ import annotations

import json
import struct
from typing import Dict, Union

import numpy as np
import torch

from .formats import QWeightInt4G32, QWeightInt8

MAGIC = b"CHADQW01"
ALIGN = 256

Entry = Union[QWeightInt4G32, QWeightInt8, torch.Tensor, np.ndarray]


def _np(t) -> np.ndarray:
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu()
        if t.dtype == torch.bfloat16:
            raise ValueError("bf16 tensors are not stored; convert to float32 or keep the bit pattern as int16")
        return np.ascontiguousarray(t.numpy())
    return np.ascontiguousarray(t)


def _arrays(e: Entry):
    if isinstance(e, QWeightInt4G32):
        return "i4g32", [e.N, e.K], {"packed": _np(e.packed), "scale": _np(e.scale)}
    if isinstance(e, QWeightInt8):
        return "i8row", [e.N, e.K], {"w": _np(e.w), "scale": _np(e.scale)}
    a = _np(e)
    return "raw", list(a.shape), {"data": a}


def save(path: str, tensors: Dict[str, Entry], meta: Dict = None) -> None:
    """Writes `tensors` (name -> quantized weight or plain tensor) to `path`."""
    items = {name: _arrays(e) for name, e in tensors.items()}

    def header(offsets):
        out = {}
        for name, (kind, shape, arrs) in items.items():
            out[name] = {"kind": kind, "shape": shape, "arrays": {
                an: {"dtype": a.dtype.str, "shape": list(a.shape), "offset": offsets.get((name, an), 0), "nbytes": int(a.nbytes)}
                for an, a in arrs.items()}}
        return json.dumps({"tensors": out, "meta": meta or {}}, sort_keys=True).encode("utf-8")

    # the header's length depends on the offsets' digits: reserve room generously, then pad with spaces
    hlen = len(header({})) + 24 * sum(len(a[2]) for a in items.values()) + 64
    pos = -(-(16 + hlen) // ALIGN) * ALIGN
    offsets = {}
    for name, (_, _, arrs) in items.items():
        for an, a in arrs.items():
            offsets[(name, an)] = pos
            pos = -(-(pos + a.nbytes) // ALIGN) * ALIGN
    h = header(offsets)
    if len(h) > hlen:
        raise RuntimeError("header grew beyond its reservation")
    h = h + b" " * (hlen - len(h))
    with open(path, "wb") as f:
        f.write(MAGIC)
        f.write(struct.pack("<Q", hlen))
        f.write(h)
        for name, (_, _, arrs) in items.items():
            for an, a in arrs.items():
                f.seek(offsets[(name, an)])
                f.write(a.tobytes())
        f.truncate(max(pos, f.tell()))


def read_header(path: str) -> Dict:
    with open(path, "rb") as f:
        if f.read(8) != MAGIC:
            raise ValueError("%s is not a CHADQW01 weight file" % path)
        (hlen,) = struct.unpack("<Q", f.read(8))
        if hlen > (1 << 28):
            raise ValueError("implausible header length %d" % hlen)
        return json.loads(f.read(hlen).decode("utf-8"))


SLAB_BYTES = 64 << 20


def _copy_out(m: np.ndarray, shape, device) -> torch.Tensor:
    """The mapped flat array `m` as a tensor of `shape` on `device`, copied in slabs of at most 64 MiB so that the
    host never holds more than one slab of it outside the page cache."""
    n = m.shape[0]
    out = torch.empty(n, dtype=torch.from_numpy(np.empty(0, dtype=m.dtype)).dtype, device=device)
    step = max(1, SLAB_BYTES // max(1, m.dtype.itemsize))
    for a in range(0, n, step):
        b = min(n, a + step)
        out[a:b].copy_(torch.from_numpy(np.array(m[a:b])))  # np.array: the slab's one host copy (the map is read-only)
    return out.reshape(shape)


def load(path: str, device="cpu") -> Dict[str, Entry]:
    """Memory-maps `path` and returns name -> QWeightInt4G32 / QWeightInt8 / tensor on `device`.  Every array is
    copied out of the map in slabs of 64 MiB (to the GPU for a GPU device), so a multi-GB file is never held whole
    in host memory; the map is closed on return."""
    hdr = read_header(path)
    size = np.memmap(path, dtype=np.uint8, mode="r").shape[0]
    out: Dict[str, Entry] = {}
    for name, t in hdr["tensors"].items():
        arrs = {}
        for an, d in t["arrays"].items():
            dt = np.dtype(d["dtype"])
            n = int(np.prod(d["shape"])) if d["shape"] else 1
            if d["offset"] % ALIGN or d["offset"] + n * dt.itemsize > size or n * dt.itemsize != d["nbytes"]:
                raise ValueError("%s: array %s/%s does not fit the file" % (path, name, an))
            m = np.memmap(path, dtype=dt, mode="r", offset=d["offset"], shape=(n,))
            arrs[an] = _copy_out(m, tuple(d["shape"]), device)
            del m
        if t["kind"] == "i4g32":
            out[name] = QWeightInt4G32(arrs["packed"], arrs["scale"])
        elif t["kind"] == "i8row":
            out[name] = QWeightInt8(arrs["w"], arrs["scale"])
        elif t["kind"] == "raw":
            out[name] = arrs["data"]
        else:
            raise ValueError("%s: unknown tensor kind %r" % (path, t["kind"]))
        if t["kind"] != "raw" and [out[name].N, out[name].K] != t["shape"]:
            raise ValueError("%s: %s has shape %s, header says %s" % (path, name, [out[name].N, out[name].K], t["shape"]))
    return out

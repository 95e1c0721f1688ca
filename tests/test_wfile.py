"""The weight container: round trip, alignment, and refusal of damaged files (CPU only)."""
import json
import struct

import numpy as np
import pytest
import torch

from chadslab_amd import QWeightInt4G32, QWeightInt8, wfile
from chadslab_amd.formats import quantize_int4_g32, quantize_int8_row


def _model():
    g = torch.Generator().manual_seed(5)
    return {
        "layer0.wqkv": quantize_int4_g32(torch.randn(48, 64, generator=g)),
        "layer0.wo": quantize_int8_row(torch.randn(20, 32, generator=g)),
        "layer0.ln": torch.randn(64, generator=g),
        "ids": np.arange(7, dtype=np.int32),
    }


def test_round_trip_and_alignment(tmp_path):
    m = _model()
    p = str(tmp_path / "m.chadq")
    wfile.save(p, m, meta={"d": 64})
    hdr = wfile.read_header(p)
    assert hdr["meta"] == {"d": 64}
    for t in hdr["tensors"].values():
        for a in t["arrays"].values():
            assert a["offset"] % 256 == 0
    back = wfile.load(p)
    assert isinstance(back["layer0.wqkv"], QWeightInt4G32) and isinstance(back["layer0.wo"], QWeightInt8)
    assert torch.equal(back["layer0.wqkv"].packed, m["layer0.wqkv"].packed)
    assert torch.equal(back["layer0.wqkv"].scale, m["layer0.wqkv"].scale)
    assert torch.equal(back["layer0.wo"].w, m["layer0.wo"].w) and torch.equal(back["layer0.wo"].scale, m["layer0.wo"].scale)
    assert torch.equal(back["layer0.ln"], m["layer0.ln"])
    assert np.array_equal(back["ids"].numpy(), m["ids"])


def test_refuses_foreign_and_truncated_files(tmp_path):
    p = str(tmp_path / "x.bin")
    open(p, "wb").write(b"NOTCHADQ" + b"\0" * 100)
    with pytest.raises(ValueError):
        wfile.load(p)
    m = _model()
    q = str(tmp_path / "m.chadq")
    wfile.save(q, m)
    data = open(q, "rb").read()
    open(q, "wb").write(data[: len(data) - 300])  # cut into the last array
    with pytest.raises(ValueError):
        wfile.load(q)


def test_refuses_inconsistent_header(tmp_path):
    q = str(tmp_path / "m.chadq")
    wfile.save(q, {"w": quantize_int4_g32(torch.ones(4, 32))})
    raw = bytearray(open(q, "rb").read())
    (hlen,) = struct.unpack("<Q", raw[8:16])
    hdr = json.loads(raw[16:16 + hlen].decode())
    hdr["tensors"]["w"]["arrays"]["packed"]["offset"] += 8  # no longer aligned
    h = json.dumps(hdr, sort_keys=True).encode()
    raw[16:16 + hlen] = h + b" " * (hlen - len(h))
    open(q, "wb").write(bytes(raw))
    with pytest.raises(ValueError):
        wfile.load(q)


def test_bf16_is_refused_loudly(tmp_path):
    with pytest.raises(ValueError):
        wfile.save(str(tmp_path / "b.chadq"), {"x": torch.zeros(4, dtype=torch.bfloat16)})


def test_decoder_weights_round_trip(tmp_path):
    from chadslab_amd.decoder import DecoderConfig, load_weights, random_weights, save_weights

    cfg = DecoderConfig(n_layers=2, d=64, hq=2, dh=16, ffn=96, vocab=50, max_ctx=32)
    w = random_weights(cfg, 3, "cpu")
    p = str(tmp_path / "dec.chadq")
    save_weights(p, cfg, w)
    cfg2, w2 = load_weights(p, "cpu")
    assert cfg2 == cfg and len(w2["layers"]) == 2
    assert torch.equal(w2["emb"].packed, w["emb"].packed) and torch.equal(w2["lnf"], w["lnf"])
    for a, b in zip(w["layers"], w2["layers"]):
        assert torch.equal(a["wgu"].packed, b["wgu"].packed) and torch.equal(a["wd"].scale, b["wd"].scale)
        assert torch.equal(a["ln1"], b["ln1"])

"""Packed-weight containers: the GGUF reader/writer and the safetensors U8 convention
(host logic; the GPU part checks that a loaded layer computes what the in-memory one does)."""
import json
import struct

import numpy as np
import pytest

from tattletale_amd import formats as F
from tattletale_amd import gguf as G
from tattletale_amd import quantize as Q


def _hand_made_file(tmp_path):
    """A GGUF v3 file assembled byte by byte from the published layout, independent of write_gguf."""
    def s(x):
        b = x.encode()
        return struct.pack("<Q", len(b)) + b
    kv = s("general.architecture") + struct.pack("<I", 8) + s("llama")
    kv += s("general.alignment") + struct.pack("<II", 4, 64)
    kv += s("llama.block_count") + struct.pack("<II", 4, 32)
    kv += s("tokenizer.ggml.tokens") + struct.pack("<IIQ", 9, 8, 2) + s("a") + s("bc")
    kv += s("some.float") + struct.pack("<If", 6, 0.5)
    t0 = np.arange(2 * 144, dtype=np.uint8)                      # 2 x 256 Q4_K: ne = [256, 2]
    t1 = np.arange(3, dtype=np.float32)
    ti = s("blk.0.ffn_up.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 256, 2) + struct.pack("<IQ", 12, 0)
    ti += s("blk.0.bias") + struct.pack("<I", 1) + struct.pack("<Q", 3) + struct.pack("<IQ", 0, 320)
    head = struct.pack("<IIQQ", 0x46554747, 3, 2, 5) + kv + ti
    head += b"\0" * ((-len(head)) % 64)
    data = t0.tobytes() + b"\0" * (320 - t0.size) + t1.tobytes()
    p = tmp_path / "hand.gguf"
    p.write_bytes(head + data)
    return str(p), t0, t1


def test_reader_against_hand_made_bytes(tmp_path):
    path, t0, t1 = _hand_made_file(tmp_path)
    with G.GGUFFile(path) as g:
        assert g.version == 3 and g.alignment == 64
        assert g.metadata["general.architecture"] == "llama"
        assert g.metadata["llama.block_count"] == 32
        assert g.metadata["tokenizer.ggml.tokens"] == ["a", "bc"]
        assert g.metadata["some.float"] == 0.5
        w = g.tensors["blk.0.ffn_up.weight"]
        # GGUF lists the contiguous dimension first; the matrix is (n_out, n_in) = (2, 256)
        assert w.shape == (2, 256) and w.format == F.Q4_K and w.nbytes == 288
        assert w.offset % 64 == 0 and g.data_offset % 64 == 0
        assert np.array_equal(g.data("blk.0.ffn_up.weight"), t0)
        b = g.tensors["blk.0.bias"]
        assert b.shape == (3,) and b.format is None
        assert np.array_equal(g.data("blk.0.bias").view(np.float32), t1)


def test_writer_reader_round_trip(tmp_path):
    w = Q.fill_normal(9, 0, 0.02, 48 * 512).reshape(48, 512)
    tensors, packed = [], {}
    for fmt in (F.Q8_0, F.Q4_K, F.Q6_K):
        p = Q.quantize(fmt, w)
        packed[fmt] = p
        tensors.append(("w%d" % fmt, G.ggml_type_of(fmt), (48, 512), p))
    tensors.append(("bias", G.GGML_F32, (48,), np.arange(48, dtype=np.float32)))
    path = str(tmp_path / "rt.gguf")
    G.write_gguf(path, tensors, {"general.name": "round trip", "x.count": 7, "x.big": 2 ** 40, "x.flag": True,
                                 "x.list": [1, -2, 3]})
    with G.GGUFFile(path) as g:
        assert g.metadata["general.name"] == "round trip" and g.metadata["x.count"] == 7
        assert g.metadata["x.big"] == 2 ** 40 and g.metadata["x.flag"] is True and g.metadata["x.list"] == [1, -2, 3]
        for fmt in (F.Q8_0, F.Q4_K, F.Q6_K):
            t = g.tensors["w%d" % fmt]
            assert t.shape == (48, 512) and t.format == fmt and t.offset % 32 == 0
            assert np.array_equal(g.data("w%d" % fmt), packed[fmt])
            assert t.nbytes == F.lib().ttq_packed_nbytes(fmt, 48, 512, 0)
        assert np.array_equal(g.data("bias").view(np.float32), np.arange(48, dtype=np.float32))


def test_malformed_files_are_rejected(tmp_path):
    path, _, _ = _hand_made_file(tmp_path)
    raw = open(path, "rb").read()
    def write(name, b):
        q = tmp_path / name
        q.write_bytes(b)
        return str(q)
    with pytest.raises(G.GGUFError):
        G.GGUFFile(write("magic.gguf", b"GGUX" + raw[4:]))
    with pytest.raises(G.GGUFError):
        G.GGUFFile(write("version.gguf", raw[:4] + struct.pack("<I", 9) + raw[8:]))
    with pytest.raises(G.GGUFError):
        G.GGUFFile(write("short.gguf", raw[:100]))
    with pytest.raises(G.GGUFError):
        G.GGUFFile(write("data.gguf", raw[:-8]))            # last tensor runs past the end
    with pytest.raises(G.GGUFError):
        G.GGUFFile(write("tiny.gguf", raw[:10]))
    # a row length that is not a multiple of the block size
    with pytest.raises(G.GGUFError):
        G.write_gguf(str(tmp_path / "bad.gguf"), [("w", G.GGML_Q4_K, (2, 100), np.zeros(10, np.uint8))])
    # unsupported tensor types are listed but cannot be read
    bad = raw.replace(struct.pack("<IQ", 12, 0), struct.pack("<IQ", 2, 0), 1)
    with G.GGUFFile(write("q4_0.gguf", bad)) as g:
        assert g.tensors["blk.0.ffn_up.weight"].nbytes == -1
        with pytest.raises(G.GGUFError):
            g.data("blk.0.ffn_up.weight")


def test_safetensors_entry_is_json():
    k, v = G.safetensors_entry("mlp.down", F.Q6_K, 4096, 14336)
    assert k == "ttq.mlp.down" and json.loads(v) == {"format": F.Q6_K, "n_out": 4096, "n_in": 14336}


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [F.Q8_0, F.Q4_K, F.Q6_K])
def test_loaded_layer_matches_in_memory_layer(tmp_path, fmt):
    import torch
    from safetensors.torch import save_file
    from tattletale_amd import QuantLinear
    from util import DEV, packed_to_dev, x_to_dev
    n_out, n_in = 300, 1024
    w = Q.fill_normal(21 + fmt, 0, 0.02, n_out * n_in).reshape(n_out, n_in)
    p = Q.quantize(fmt, w)
    bias = np.linspace(-1, 1, n_out).astype(np.float32)
    path = str(tmp_path / "layer.gguf")
    G.write_gguf(path, [("w", G.ggml_type_of(fmt), (n_out, n_in), p), ("b", G.GGML_F32, (n_out,), bias)])
    xd, _ = x_to_dev(Q.fill_normal(5, 1, 1.0, 2 * n_in).reshape(2, n_in), "bf16")
    want = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out, bias=torch.from_numpy(bias).to(DEV)).forward(xd)
    with G.GGUFFile(path) as g:
        layer = G.load_quant_linear(g, "w", DEV, bias_name="b")
    assert torch.equal(layer.forward(xd), want)
    # the safetensors convention: a U8 tensor plus a metadata entry
    st = str(tmp_path / "layer.safetensors")
    k, v = G.safetensors_entry("w", fmt, n_out, n_in)
    save_file({"w.qweight": torch.from_numpy(p.copy())}, st, metadata={k: v})
    layer2 = G.load_quant_linear_safetensors(st, "w", DEV)
    want2 = QuantLinear.init(packed_to_dev(p), fmt, n_in, n_out).forward(xd)
    assert torch.equal(layer2.forward(xd), want2)

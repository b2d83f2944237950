"""Writes tests/golden/qlinear_layer_fixture.safetensors: a small layer fixture in the shape of the
reference's own (workspace/transformers/tests/fixtures/layers/...: inputs and expected outputs of one
layer as bf16 tensors in a safetensors file, read by test_fixtures_layers.nim), for the quantized
layers of this library.  Packed weights are stored as U8 tensors `<name>.qweight` with a
`ttq.<name>` metadata entry (format, n_out, n_in); expected outputs come from the CPU oracle:
float64 products over oracle-dequantized weights, rounded to bf16 where the reference's layer
rounds (after every Linear and after silu_and_mul, mlp.nim:56-60).

    python tests/golden/make_layer_fixture.py

The file is read by tests/test_layer_fixture.py (CPU: fixture against the oracle; GPU: the layers
against the fixture) and by tattletale_amd/nim/test_qlinear.nim."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from tattletale_amd import formats as F  # noqa: E402
from tattletale_amd import quantize as Q  # noqa: E402
from tattletale_amd.gguf import safetensors_entry  # noqa: E402

HIDDEN, FF = 256, 256
SEED = 4242
CASES = {"decode": (1, 1), "prefill": (2, 9), "zeros": (1, 3)}     # name -> (batch, seq)
PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "qlinear_layer_fixture.safetensors")


def bf16(a):
    """float -> bf16 bit patterns (uint16) and the float32 values they stand for."""
    bits = oracle.f32_to_bf16(np.asarray(a, np.float32))
    return bits, oracle.bf16_to_f32(bits)


def build():
    """name -> (numpy array, safetensors dtype string); metadata dict."""
    tensors, meta = {}, {}
    dense = {
        "mlp.gate_up_proj": (F.Q4_K, 2 * FF, HIDDEN), "mlp.down_proj": (F.Q4_K, HIDDEN, FF),
        "attn.o_proj": (F.Q6_K, HIDDEN, HIDDEN), "attn.q_proj": (F.Q8_0, HIDDEN, HIDDEN),
    }
    what = {}
    for i, (name, (fmt, n_out, n_in)) in enumerate(sorted(dense.items())):
        w = Q.fill_normal(SEED + i, 0, 0.05, n_out * n_in).reshape(n_out, n_in)
        p = Q.quantize(fmt, w)
        tensors[name + ".qweight"] = (p, "U8")
        k, v = safetensors_entry(name, fmt, n_out, n_in)
        meta[k] = v
        what[name] = oracle.dequant(fmt, p, n_out, n_in)
    for ci, (case, (b, s)) in enumerate(sorted(CASES.items())):
        m = b * s
        x = np.zeros((m, HIDDEN), np.float32) if case == "zeros" else \
            Q.fill_normal(SEED + 100 + ci, 1, 1.0, m * HIDDEN).reshape(m, HIDDEN)
        xb, xf = bf16(x)
        tensors[case + ".input_hidden_states"] = (xb.reshape(b, s, HIDDEN), "BF16")
        # GatedMLP.forward: gate_up -> bf16, silu_and_mul -> bf16, down -> bf16
        _, gu = bf16(oracle.linear_f64(what["mlp.gate_up_proj"], xf))
        _, act = bf16(oracle.silu_and_mul_f64(gu))
        yb, _ = bf16(oracle.linear_f64(what["mlp.down_proj"], act))
        tensors[case + ".mlp.output"] = (yb.reshape(b, s, HIDDEN), "BF16")
        for name in ("attn.o_proj", "attn.q_proj"):
            yb, _ = bf16(oracle.linear_f64(what[name], xf))
            tensors[case + "." + name + ".output"] = (yb.reshape(b, s, HIDDEN), "BF16")
    return tensors, meta


def write(path=PATH):
    import json
    import struct
    tensors, meta = build()
    header, blobs, off = {"__metadata__": meta}, [], 0
    for name in sorted(tensors):
        a, dt = tensors[name]
        raw = np.ascontiguousarray(a).tobytes()
        header[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    hj = json.dumps(header, sort_keys=True).encode()
    hj += b" " * (-len(hj) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(hj)))
        f.write(hj)
        for raw in blobs:
            f.write(raw)
    return path


if __name__ == "__main__":
    print("wrote", write(), os.path.getsize(PATH), "bytes")

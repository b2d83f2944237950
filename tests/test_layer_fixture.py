"""The layer fixture tests/golden/qlinear_layer_fixture.safetensors (inputs, packed weights and
expected outputs of a gated MLP and two projections, in the shape of the reference's layer fixtures,
workspace/transformers/tests/test_fixtures_layers.nim:63-93).

CPU: the committed file is what the generator produces from the oracle today.  GPU: the library's
layers, loaded from the file the way a caller would, reproduce the expected outputs within the
reference's own layer tolerance (assertAllClose rtol = abstol = 2e-2, common_utils.nim:53-66)."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import make_layer_fixture as MLF  # noqa: E402


def _read(path):
    from safetensors import safe_open
    out = {}
    with safe_open(path, framework="pt", device="cpu") as f:
        md = f.metadata()
        for k in f.keys():
            out[k] = f.get_tensor(k)
    return out, md


def test_fixture_file_matches_the_oracle(tmp_path):
    fresh = MLF.write(str(tmp_path / "fresh.safetensors"))
    with open(fresh, "rb") as a, open(MLF.PATH, "rb") as b:
        assert a.read() == b.read()


def test_fixture_outputs_are_not_trivial():
    t, md = _read(MLF.PATH)
    assert set(md) == {"ttq.mlp.gate_up_proj", "ttq.mlp.down_proj", "ttq.attn.o_proj", "ttq.attn.q_proj"}
    for case in MLF.CASES:
        y = t[case + ".mlp.output"].float()
        assert y.shape == t[case + ".input_hidden_states"].shape
        assert bool(torch.isfinite(y).all())
        assert (case == "zeros") == bool((y == 0).all())


@pytest.mark.gpu
@pytest.mark.parametrize("case", sorted(MLF.CASES))
def test_layers_reproduce_the_fixture(case):
    from tattletale_amd import QuantGatedMLP
    from tattletale_amd.gguf import load_quant_linear_safetensors
    dev = torch.device("cuda:0")
    t, _ = _read(MLF.PATH)
    x = t[case + ".input_hidden_states"].to(dev)
    mlp = QuantGatedMLP.init(load_quant_linear_safetensors(MLF.PATH, "mlp.gate_up_proj", dev),
                             load_quant_linear_safetensors(MLF.PATH, "mlp.down_proj", dev))
    y = mlp.forward(x)
    assert y.dtype == torch.bfloat16 and y.shape == x.shape
    assert torch.allclose(y.float().cpu(), t[case + ".mlp.output"].float(), rtol=2e-2, atol=2e-2)
    for name in ("attn.o_proj", "attn.q_proj"):
        layer = load_quant_linear_safetensors(MLF.PATH, name, dev)
        y = layer.forward(x)
        assert y.dtype == torch.bfloat16
        assert torch.allclose(y.float().cpu(), t[case + "." + name + ".output"].float(), rtol=2e-2, atol=2e-2)

# Layer test for the quantized Linear / GatedMLP in the reference's test idiom
# (workspace/transformers/tests/test_fixtures_layers.nim: runTest sections, fixtures as small
# safetensors files, assertAllClose with the 2e-2 tolerances of common_utils.nim:53-66).
#
# Fixture: tests/golden/qlinear_layer_fixture.safetensors of this repository (written by
# tests/golden/make_layer_fixture.py from the CPU oracle): packed weights as U8 tensors
# "<name>.qweight" with a "ttq.<name>" metadata entry {"format", "n_out", "n_in"}, and per case
# ("decode", "prefill", "zeros") the bf16 input and expected outputs.
#
# NOT compiled in this repository: no Nim toolchain is available where it is built.  The same
# fixture is checked through the same C ABI by tests/test_layer_fixture.py.  To run inside the
# reference tree: copy this file and qlinear.nim next to the layer tests, point FixtureFile at the
# fixture, put libttq_hip.so on the loader path, and `nim cpp -r test_qlinear.nim` on a machine
# with a GPU (the test_transformers task of config.nims picks up test_*.nim files).

import
  std/json,
  std/memfiles,
  std/options,
  std/os,
  std/tables,
  workspace/safetensors,
  workspace/libtorch as F,
  ./common_utils,
  ./qlinear

const
  FixtureFile = currentSourcePath().parentDir() / "fixtures" / "qlinear_layer_fixture.safetensors"
  Cases = ["decode", "prefill", "zeros"]

proc loadQuantLinear(st: var Safetensor, md: Table[string, string], name: string): QuantLinear =
  ## Packed weight `<name>.qweight` + its metadata entry -> QuantLinear on the GPU.
  let info = parseJson(md["ttq." & name])
  let q = st.getTensorOwned(name & ".qweight").to(kCUDA)
  QuantLinear.init(q, QuantFormat(info["format"].getInt()), info["n_in"].getInt(), info["n_out"].getInt())

proc main() =
  runTest "QuantLinear fixtures (Q6_K o_proj, Q8_0 q_proj)":
    proc(): bool =
      var mf = memfiles.open(FixtureFile, mode = fmRead)
      defer: close(mf)
      var st = safetensors.load(mf)
      let md = st.metadata.unsafeGet()
      for name in ["attn.o_proj", "attn.q_proj"]:
        let layer = loadQuantLinear(st, md, name)
        for c in Cases:
          let x = st.getTensorOwned(c & ".input_hidden_states").to(kCUDA)
          let expected = st.getTensorOwned(c & "." & name & ".output")
          let y = layer.forward(x)           # seq_len == 1: GEMV, otherwise GEMM; same call
          assertAllClose(y.to(kCPU), expected, msg = name & " case " & c & " failed")
      true

  runTest "QuantGatedMLP fixtures (Q4_K gate_up / down, fused silu_and_mul at decode)":
    proc(): bool =
      var mf = memfiles.open(FixtureFile, mode = fmRead)
      defer: close(mf)
      var st = safetensors.load(mf)
      let md = st.metadata.unsafeGet()
      let mlp = QuantGatedMLP.init(loadQuantLinear(st, md, "mlp.gate_up_proj"),
                                   loadQuantLinear(st, md, "mlp.down_proj"))
      for c in Cases:
        let x = st.getTensorOwned(c & ".input_hidden_states").to(kCUDA)
        let expected = st.getTensorOwned(c & ".mlp.output")
        let y = mlp.forward(x)
        assertAllClose(y.to(kCPU), expected, msg = "MLP case " & c & " failed")
      true

  runTest "QuantLinear rejects a packed buffer of the wrong size":
    proc(): bool =
      var mf = memfiles.open(FixtureFile, mode = fmRead)
      defer: close(mf)
      var st = safetensors.load(mf)
      let q = st.getTensorOwned("attn.q_proj.qweight").to(kCUDA)
      try:
        discard QuantLinear.init(q, kQ8_0, 256, 257)
        false
      except QuantLinearError:
        true

when isMainModule:
  main()

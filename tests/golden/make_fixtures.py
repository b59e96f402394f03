"""Extract the golden vectors the reference's own tests hold for this path.

Run in a container where the reference checkout is mounted:

    python tests/golden/make_fixtures.py [/root/reference]

Reads DATA only (a JSON fixture, and the literal tables of a generated Rust
test-data file) and writes small JSON fixtures beside this script:

  ggml_kquant_golden.json   llama.cpp's own encoder+decoder on 512 inputs:
                            q8_0 / q6_K / q4_K bytes and the decoded f32 bit
                            patterns.  Source (copied verbatim, it is data):
                            crates/larql-vindex/src/format/vindex3/represent/fixtures/ggml_kquant_golden.json
  q8_0_ggml_golden.json     ggml quantize_row_q8_0_ref blocks for edge-case
                            inputs: name, 32 input bit patterns, 34-byte block.
                            Source tables:
                            crates/larql-models/src/quant/ggml/tests/q8_0_ggml_golden.rs
  situ_glu_golden.json      SiTU-GLU (Kimi-K3's SituAndMul.forward run in PyTorch): per arm beta, linear_beta and 88
                            (gate, up, out) points.  Source (the arms' data, without the measured controls):
                            crates/larql-compute/src/ffn/expert_weight/tests/situ_oracle.json

Nothing of the reference is imported or executed.
"""
import json
import os
import re
import shutil
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def main(ref: str) -> None:
    src = os.path.join(ref, "crates/larql-vindex/src/format/vindex3/represent/fixtures/ggml_kquant_golden.json")
    shutil.copyfile(src, os.path.join(HERE, "ggml_kquant_golden.json"))

    rs = open(os.path.join(ref, "crates/larql-models/src/quant/ggml/tests/q8_0_ggml_golden.rs")).read()
    cases = []
    for m in re.finditer(r'Q8Golden\s*\{\s*name:\s*"([^"]*)",\s*input_bits:\s*\[(.*?)\],\s*block_hex:\s*"([0-9a-fA-F]*)"',
                         rs, re.S):
        bits = [int(t, 16) for t in re.findall(r"0x([0-9a-fA-F]+)", m.group(2))]
        assert len(bits) == 32 and len(m.group(3)) == 68
        cases.append({"name": m.group(1), "input_bits": bits, "block_hex": m.group(3)})
    assert cases, "no Q8Golden entries parsed"
    header = re.search(r"// Expected bytes: (.*)", rs)
    with open(os.path.join(HERE, "q8_0_ggml_golden.json"), "w") as f:
        json.dump({"source": header.group(1) if header else "", "cases": cases}, f, indent=0)
    situ = json.load(open(os.path.join(ref, "crates/larql-compute/src/ffn/expert_weight/tests/situ_oracle.json")))
    arms = {name: {k: arm[k] for k in ("beta", "linear_beta", "gate", "up", "out")} for name, arm in situ["arms"].items()}
    with open(os.path.join(HERE, "situ_glu_golden.json"), "w") as f:
        json.dump({"source": situ["_source"], "precision": situ["_precision"], "arms": arms}, f, indent=0)
    print(f"wrote {len(cases)} Q8_0 golden blocks, ggml_kquant_golden.json and {len(arms)} SiTU-GLU arms")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")

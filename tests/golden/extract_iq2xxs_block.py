"""Writes tests/golden/iq2xxs_ggml_block.json from the data the reference's own test holds.

The reference keeps one IQ2_XXS block that ggml made (66 bytes) and the 256 f32 bit patterns ggml decodes it
to, as literals inside crates/gguf/src/quant.rs (test `iq2_xxs_matches_a_ggml_made_block`, lines 3678-3745).
This script reads that file as text and copies the two literals out; nothing of the reference is run.
Run it from the repository root in a container that has /root/reference mounted.
"""
import json
import re

SRC = "/root/reference/crates/gguf/src/quant.rs"


def main():
    text = open(SRC).read()
    at = text.index("fn iq2_xxs_matches_a_ggml_made_block")
    body = text[at:at + 12000]
    block = re.search(r"const BLOCK: \[u8; 66\] = \[(.*?)\];", body, re.S).group(1)
    want = re.search(r"const WANT: \[u32; 256\] = \[(.*?)\];", body, re.S).group(1)
    block = [int(v) for v in re.findall(r"\d+", block)]
    want = [int(v.replace("_", ""), 16) for v in re.findall(r"0x[0-9a-f_]+", want)]
    assert len(block) == 66 and len(want) == 256
    with open("tests/golden/iq2xxs_ggml_block.json", "w") as f:
        json.dump({"source": "crates/gguf/src/quant.rs:3678-3745", "block": block, "want_f32_bits": want}, f)


if __name__ == "__main__":
    main()

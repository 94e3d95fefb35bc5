"""Transcribe the reference's SDPA golden table into a JSON fixture.

Source of the vectors: /root/reference/tests/attention_golden.rs (a generated
table of literals: six cases with q/k/v/mask inputs and the expected output,
consumed by tests/nn_attention.rs:33-56 with tolerance 1e-5*max(|want|,1)).
Only the numbers are carried over; nothing is executed from the reference.

Run once in the build container:  python tests/golden/make_sdpa_golden.py
"""
import json
import os
import re
import sys

SRC = "/root/reference/tests/attention_golden.rs"
DST = os.path.join(os.path.dirname(os.path.abspath(__file__)), "sdpa_golden.json")

LIST_FIELDS = ["q_shape", "q", "k_shape", "k", "v_shape", "v", "mask_shape", "mask", "out_shape", "out"]
BOOL_FIELDS = ["mask_bool", "is_causal", "enable_gqa"]


def main():
    text = open(SRC).read()
    body = text[text.index("pub static SDPA_GOLDEN"):]
    cases = []
    for chunk in body.split("SdpaGolden {")[1:]:
        case = {"name": re.search(r'name:\s*"([^"]+)"', chunk).group(1)}
        for f in LIST_FIELDS:
            m = re.search(r"\b%s:\s*&\[(.*?)\]" % f, chunk, re.S)
            vals = [x.strip() for x in m.group(1).replace("\n", " ").split(",") if x.strip()]
            if f.endswith("_shape"):
                case[f] = [int(x) for x in vals]
            else:
                case[f] = [float(x) for x in vals]
        for f in BOOL_FIELDS:
            case[f] = re.search(r"\b%s:\s*(true|false)" % f, chunk).group(1) == "true"
        cases.append(case)
    assert [c["name"] for c in cases] == ["basic", "multihead", "causal", "bool_mask", "float_mask", "gqa"], cases
    with open(DST, "w") as fh:
        json.dump({"source": "tests/attention_golden.rs", "tolerance": "abs(a-b) <= 1e-5*max(abs(b),1)", "cases": cases}, fh)
    print("wrote", DST, os.path.getsize(DST), "bytes")


if __name__ == "__main__":
    sys.exit(main())

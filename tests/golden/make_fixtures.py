"""Extracts the golden DATA this repo's tests use from the reference checkout.

Run once in the authoring container (the reference is not present on the GPU box):

    python tests/golden/make_fixtures.py /root/reference

Only data records are copied, no source text:
  * scripts/oracle/vectors.txt -> ggml_vectors.txt: the N / INPUT records and the
    TYPE / QUANT / DEQUANT records of q4_0, q4_1, q5_0, q5_1, q8_0, q2_K, q3_K, q4_K, q5_K, q6_K, q8_K, mxfp4 (ggml's own scalar quantize and
    dequantize outputs on a 1024-value input; floats are 8-hex-digit bit patterns).
  * tests/vectors/ggml_encode.json -> ggml_encode_subset.json: rows, cols, read, x and the
    `blocks` / `expected` hex strings of q4_0, q4_1, q5_0, q5_1, q2_k, q3_k, q4_k, q5_k, q6_k, q8_0, iq4_nl, iq4_xs, mxfp4 and
    the codebook formats iq2_xxs, iq3_xxs, iq3_s, iq2_s, q2_0 (ggml-written blocks of an 8x512 matrix and the
    first two rows as ggml decodes them).
  * tests/vectors/ggml_low_bit_blocks.json -> low_bit_blocks.json, whole: one block of IQ4_NL, IQ4_XS, IQ3_XXS,
    IQ3_S, IQ2_S and Q2_0 cut out of a real file, with the values that file's reader gives.
"""
import json
import sys
from pathlib import Path

KEEP_TYPES = {"q4_0", "q4_1", "q5_0", "q5_1", "q8_0", "q2_K", "q3_K", "q4_K", "q5_K", "q6_K", "q8_K", "mxfp4"}


def main(ref: str) -> None:
    ref = Path(ref)
    here = Path(__file__).resolve().parent

    out = []
    keep = False
    for line in (ref / "scripts/oracle/vectors.txt").read_text().splitlines():
        if line.startswith("#"):
            continue
        tag = line.split(" ", 1)[0]
        if tag in ("N", "INPUT"):
            out.append(line)
        elif tag == "TYPE":
            keep = line.split()[1] in KEEP_TYPES
            if keep:
                out.append(line)
        elif keep:
            out.append(line)
    (here / "ggml_vectors.txt").write_text("\n".join(out) + "\n")

    j = json.loads((ref / "tests/vectors/ggml_encode.json").read_text())
    sub = {k: j[k] for k in ("rows", "cols", "read", "x")}
    sub["formats"] = {
        f: {"blocks": j["formats"][f]["blocks"], "expected": j["formats"][f]["expected"]}
        for f in ("q4_0", "q4_1", "q5_0", "q5_1", "q2_k", "q3_k", "q4_k", "q5_k", "q6_k", "q8_0", "iq4_nl", "iq4_xs", "mxfp4",
                  "iq2_xxs", "iq3_xxs", "iq3_s", "iq2_s", "q2_0")
    }
    (here / "ggml_encode_subset.json").write_text(json.dumps(sub))
    (here / "low_bit_blocks.json").write_text((ref / "tests/vectors/ggml_low_bit_blocks.json").read_text())


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")

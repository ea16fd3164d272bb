"""Writes tests/golden/kat_fixtures.json from the oracle's restatement of the reference's known-answer
generator (reference: test/blkq4_fp16_quant_sm80_test.cu:72-112, shapes :313-347).

The digests in the output are compared in tests/test_oracle.py against a second, independently
derived table (tests/golden/kat_digests_independent.json) that was computed from the reference's
layout specification with a separate numpy program while the reference was being studied; neither
program runs any reference code.

Usage: python tests/golden/make_kat_fixtures.py
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import blkq4_oracle as O  # noqa: E402

SHAPES = [(64, 32), (64, 64), (64, 128), (64, 256), (128, 32), (256, 32), (256, 256)]


def digest(a) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()[:16]


def main():
    out = {"block_size": 32, "cases": []}
    for column_wise in (True, False):
        for rows, columns in SHAPES:
            kat = O.kat_generate(32, column_wise, rows, columns, True)
            pw, ps, pz = O.quant_sm80(32, column_wise, kat["weights"], True)
            case = {
                "column_wise": column_wise, "rows": rows, "columns": columns,
                "canonW": digest(kat["canon_w"]), "packedW": digest(pw),
                "packedS": digest(ps.view(np.uint16)), "packedZ": digest(pz),
                "nativeW": digest(O.native_from_canonical(kat["canon_w"])),
            }
            if (rows, columns) == (64, 32):
                # the smallest case in full, as hex
                case["hex"] = {
                    "weights_fp16": kat["weights"].view(np.uint16).astype("<u2").tobytes().hex(),
                    "canonW": kat["canon_w"].tobytes().hex(),
                    "packedW": pw.tobytes().hex(),
                    "packedS": ps.view(np.uint16).astype("<u2").tobytes().hex(),
                    "packedZ": pz.tobytes().hex(),
                    "nativeW": O.native_from_canonical(kat["canon_w"]).tobytes().hex(),
                }
            out["cases"].append(case)
    with open(os.path.join(HERE, "kat_fixtures.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote kat_fixtures.json with", len(out["cases"]), "cases")


if __name__ == "__main__":
    main()

"""Writes tests/golden/plan_times_mi355x.json from the output of

    python3 -m bench_probe.plan_check --quick --every-plan --shapes <variant:m:n:k,...> > times.jsonl

(run on an MI355X): for every shape the measured microseconds of every plan that exists for it, by the plan's text
form as blkq4_gemm_with_plan_sm80 takes it.  Plans more than 1.6 times slower than the shape's best are left out.
tests/test_kernel_choice.py holds the kernel choice against these times on the CPU.

    python3 tests/golden/make_plan_times.py times.jsonl [more.jsonl ...]
"""

import json
import os
import sys

VARIANTS = {"fp16/bs64": (False, 64, True, True), "bf16/bs64": (True, 64, True, True), "fp16/bs16": (False, 16, True, True),
            "fp16/bs32/sym": (False, 32, True, False), "fp16/bs64/along-N": (False, 64, False, True),
            "bf16/bs16": (True, 16, True, True), "bf16/bs64/along-N": (True, 64, False, True)}


def main(paths):
    rows = []
    for path in paths:
        for line in open(path):
            try:
                r = json.loads(line)
            except ValueError:
                continue
            if "us_by_plan" not in r or r.get("wrong_results"):
                continue
            bf16, bs, column_wise, has_zp = VARIANTS[r["variant"]]
            best = min(r["us_by_plan"].values())
            rows.append({"bf16": bf16, "block_size": bs, "column_wise": column_wise, "has_offsets": has_zp,
                         "m": r["m"], "n": r["n"], "k": r["k"],
                         "us": {p: round(v, 2) for p, v in sorted(r["us_by_plan"].items()) if v <= 1.6 * best}})
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "plan_times_mi355x.json")
    with open(out, "w") as f:
        f.write("[\n" + ",\n".join(json.dumps(r, separators=(",", ":")) for r in rows) + "\n]\n")
    print(f"{len(rows)} shapes -> {out} ({os.path.getsize(out)} bytes)")


if __name__ == "__main__":
    main(sys.argv[1:])

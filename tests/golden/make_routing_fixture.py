#!/usr/bin/env python3
"""Writes tests/golden/routing_first_real_prompt_layer0.csv: the layer-0 prefill histogram of the
reference's recorded routing profile (routing-profile/first-real-prompt/counts.csv, the fixture
its tests/bench_expert_pair_ab.cpp:189-216,640 draws chunks from), 256 counts, data only. Run from
the repo root where the reference tree is mounted:
    python tests/golden/make_routing_fixture.py
"""
import csv
import os

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
SOURCE = "/root/reference/routing-profile/first-real-prompt/counts.csv"


def main():
    counts = [0] * 256
    with open(SOURCE, newline="") as f:
        for row in csv.DictReader(f):
            if row["phase"] == "prefill" and int(row["layer_id"]) == 0:
                counts[int(row["expert_id"])] = int(row["selection_count"])
    assert sum(counts) > 0
    path = os.path.join(ROOT, "tests", "golden", "routing_first_real_prompt_layer0.csv")
    with open(path, "w") as f:
        f.write("expert_id,selection_count\n")
        for e, c in enumerate(counts):
            f.write("%d,%d\n" % (e, c))
    print("wrote", path, "total selections", sum(counts), "experts never selected", counts.count(0))


if __name__ == "__main__":
    main()

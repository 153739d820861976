#!/usr/bin/env python3
"""Extract the reference-held golden checksums into tests/golden/checksums.json.

The reference's `knn` binary prints `Checksum: S` on stderr once per iteration, where
S = sum of the k result indices of query 0 modulo 2^32 (reference src/main.cpp:410-417).
The authors committed the stderr of their measurement runs as data/*.err next to the
stdout CSV data/*.csv; the i-th `Checksum:` line belongs to the i-th row of the CSV whose
phase is `finish` (one such row per iteration, reference src/main.cpp:402-406).

This script only READS those text files (nothing of the reference is imported or executed)
and writes a small JSON fixture: for every distinct experiment shape
(generator, preprocessor, n, q, d, k) the multiset of checksums that were printed, with the
set of algorithms that printed them.  Run it in the build container, where the reference
is mounted:

    python tests/golden/extract_checksums.py /root/reference/data

The fixture is data (inputs' shape + expected outputs), committed as
tests/golden/checksums.json, and is what the parity tests read on the GPU box.
"""
import csv
import json
import os
import sys
from collections import defaultdict

# experiment families whose stderr/CSV pairs line up one checksum per finish row
FAMILIES = ("kselection", "fused", "buffer")


def pair_file(err_path, csv_path):
    with open(err_path, "r", errors="replace") as f:
        sums = [int(line.split(":")[1]) for line in f if line.startswith("Checksum:")]
    rows = []
    with open(csv_path, newline="") as f:
        for row in csv.DictReader(f):
            if row.get("phase") == "finish":
                rows.append(row)
    if len(sums) != len(rows):
        return None
    return list(zip(rows, sums))


def main():
    data_dir = sys.argv[1] if len(sys.argv) > 1 else "/root/reference/data"
    out_path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "checksums.json")
    table = defaultdict(lambda: {"checksums": defaultdict(int), "algorithms": set(), "files": set()})
    skipped = []
    for name in sorted(os.listdir(data_dir)):
        if not name.endswith(".err"):
            continue
        family = next((fam for fam in FAMILIES if name.startswith(fam + "-")), None)
        if family is None:
            continue
        csv_path = os.path.join(data_dir, name[:-4] + ".csv")
        if not os.path.exists(csv_path):
            continue
        pairs = pair_file(os.path.join(data_dir, name), csv_path)
        if pairs is None:
            skipped.append(name)
            continue
        for row, checksum in pairs:
            key = (family, row["generator"], row["preprocessor"], int(row["point_count"]),
                   int(row["query_count"]), int(row["dim"]), int(row["k"]))
            entry = table[key]
            entry["checksums"][checksum] += 1
            entry["algorithms"].add(row["algorithm"])
            entry["files"].add(name)
    records = []
    for key in sorted(table):
        family, gen, pre, n, q, d, k = key
        entry = table[key]
        records.append({
            "family": family, "generator": gen, "preprocessor": pre, "seed": 24,
            "n": n, "q": q, "d": d, "k": k,
            "checksums": {str(c): cnt for c, cnt in sorted(entry["checksums"].items(),
                                                            key=lambda kv: -kv[1])},
            "unanimous": len(entry["checksums"]) == 1,
            "algorithms": sorted(entry["algorithms"]),
            "n_files": len(entry["files"]),
        })
    with open(out_path, "w") as f:
        json.dump({"source": "reference data/*.err paired with data/*.csv finish rows",
                   "seed_note": "all runs use --seed 24 (reference scripts/run-*.sh)",
                   "skipped_files_line_mismatch": skipped,
                   "records": records}, f, indent=0, separators=(",", ":"))
        f.write("\n")
    print(f"{len(records)} records -> {out_path}; skipped {skipped}")


if __name__ == "__main__":
    main()

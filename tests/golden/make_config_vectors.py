#!/usr/bin/env python3
"""Writes config_vectors.json: what the reference's own lookup (the awk program of
scripts/config.sh, `config_generic`) answers for a list of requests on optima_sample.csv.

Run in a container that holds the reference checkout (default /root/reference); the output is
committed so that the tests need neither the reference nor a shell.
"""
import json
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
SAMPLE = os.path.join(HERE, "optima_sample.csv")

REQUESTS = []
for host in ("hostA", "hostB", "None"):
    for q, k in ((1, 1), (64, 16), (100, 100), (1000, 20), (1024, 128), (5000, 200), (8192, 2048),
                 (100000, 4096), (700, 16), (64, 2048)):
        REQUESTS.append(("bits", host, q, k, "None"))
for q, k, dim in ((2048, 8, 4), (2000, 10, 16), (4096, 32, 32), (10000, 64, 64), (1, 1, 1),
                  (8192, 64, 128), (3000, 9, 5)):
    REQUESTS.append(("fused-cache", "hostA", q, k, dim))
for k in (1, 32, 33, 512, 1000):
    REQUESTS.append(("partial-bitonic-regs", "hostA", 1024, k, "None"))
    REQUESTS.append(("partial-bitonic-regs", "None", "None", k, "None"))
REQUESTS.append(("unknown-algorithm", "hostA", 10, 10, "None"))
REQUESTS.append(("bits", "hostC", 10, 10, "None"))


def main():
    out = []
    for algorithm, host, q, k, dim in REQUESTS:
        script = (f'worker={host}; root_dir={REFERENCE}; build_dir=/tmp; '
                  f'. {REFERENCE}/scripts/config.sh 2>/dev/null; worker={host}; '
                  f'config_generic {SAMPLE} {algorithm} {q} {k} {dim}')
        answer = subprocess.run(["bash", "-c", script], check=True, capture_output=True, text=True).stdout
        out.append({"algorithm": algorithm, "hostname": host, "query_count": q, "k": k, "dim": dim,
                    "answer": answer.rstrip("\n").split(" ")})
    with open(os.path.join(HERE, "config_vectors.json"), "w") as handle:
        json.dump(out, handle, indent=0)
        handle.write("\n")


if __name__ == "__main__":
    main()

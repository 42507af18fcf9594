"""Keeps the N best rows (highest perf, failed measurements dropped) of a records.txt:

    python keep_best.py <run>/records.txt tuned/<CASE>/records.txt [N=32]

The files under tuned/ are what ``run.py -t`` and the benchmark load through Task.apply_best.
"""
import json
import os
import sys


def keep_best(src, dst, n=32):
    rows = [json.loads(line) for line in open(src) if line.strip()]
    rows = sorted((r for r in rows if r["perf"] > 0), key=lambda r: -r["perf"])[:n]
    os.makedirs(os.path.dirname(os.path.abspath(dst)), exist_ok=True)
    with open(dst, "w") as out:
        for r in rows:
            out.write(json.dumps(r) + "\n")
    return len(rows)


if __name__ == "__main__":
    print(keep_best(sys.argv[1], sys.argv[2], int(sys.argv[3]) if len(sys.argv) > 3 else 32), "rows kept")

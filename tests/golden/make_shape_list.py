"""Writes tests/golden/reference_sweep_shapes.csv: every distinct (m, n, k, transA, transB, alpha, beta) row of the shape
lists the reference's GEMM benchmark driver sweeps (/root/reference/tools/benchmarkers/gemm_*.csv, read by
accera_gemm.py / gpu_benchmark_tool.py).  Data only: the sizes and flags, no code.  Run where /root/reference exists:

    python tests/golden/make_shape_list.py
"""
import csv
import glob
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def main(src="/root/reference/tools/benchmarkers"):
    rows = set()
    for path in sorted(glob.glob(os.path.join(src, "gemm_*.csv"))):
        for r in csv.DictReader(open(path)):
            rows.add((int(r["m"]), int(r["n"]), int(r["k"]), int(r["transA"]), int(r["transB"]), float(r["alpha"]), float(r["beta"])))
    out = os.path.join(HERE, "reference_sweep_shapes.csv")
    with open(out, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["m", "n", "k", "transA", "transB", "alpha", "beta"])
        for r in sorted(rows):
            w.writerow(r)
    print(len(rows), "rows ->", out)


if __name__ == "__main__":
    main()

"""Turns rocprofv3 counter output into the figures the benchmark reports.

    python -m accera_amd.profiling traffic <config> <fetch_csv> <write_csv> [--out profiles/traffic.json]

reads the `*_counter_collection.csv` files of two `rocprofv3 --pmc` runs of `bench.py`
(one with FETCH_SIZE, one with WRITE_SIZE; both counters are KiB per dispatch), scales them
by what the same counter reads for the library's plain copy kernel of known size (64 MiB
read, 64 MiB written, launched once by bench.py), and stores the HBM bytes per launch of
the dominant kernel.

    python -m accera_amd.profiling summary <csv> ...

prints per-kernel averages of every counter in the given files.
"""
import argparse
import collections
import csv
import re
import json
import os
import sys

COPY_KERNEL = "acc950_copy_kernel"
COPY_BYTES = 64 << 20


def read_counters(path):
    """{kernel name: {counter: [values per dispatch]}}"""
    acc = collections.defaultdict(lambda: collections.defaultdict(list))
    with open(path) as f:
        for r in csv.DictReader(f):
            acc[r["Kernel_Name"]][r["Counter_Name"]].append(float(r["Counter_Value"]))
    return acc


def _dominant(acc, counter):
    """Kernel (other than the probes) with the largest total of `counter`."""
    best = None
    for k, cs in acc.items():
        if "acc950_copy_kernel" in k or "acc950_stream_read_kernel" in k or "mfma_ceiling" in k or counter not in cs:
            continue
        if not any(s in k for s in ("gemm_mfma_kernel", "gemm_mfma16_kernel", "gemm_mfma16w4_kernel", "gemm_skinny", "gemm_f32_kernel", "gemm_generic_kernel")):
            continue
        # the builds with clock stamps, run by the phase probe: third argument of Mfma16W4Config, last one of the others
        if re.search(r"Mfma16W4Config<[^,>]*,[^,>]*, true\b", k) or (
                "Mfma16W4Config" not in k and re.search(r"Config<[^>]*, true>\s*>", k)):
            continue
        tot = sum(cs[counter])
        if best is None or tot > best[1]:
            best = (k, tot)
    return best[0] if best else None


def traffic(config, fetch_csv, write_csv, out):
    res = {}
    for counter, path in (("FETCH_SIZE", fetch_csv), ("WRITE_SIZE", write_csv)):
        acc = read_counters(path)
        copy = [k for k in acc if COPY_KERNEL in k]
        if not copy:
            raise SystemExit(f"{path}: the copy probe kernel is not in this trace")
        copy_kib = sum(acc[copy[0]][counter]) / len(acc[copy[0]][counter])
        factor = (COPY_BYTES / 1024.0) / copy_kib  # true KiB per counted KiB
        kern = _dominant(acc, counter)
        vals = acc[kern][counter]
        # skip the first dispatches (cold caches / warm-up)
        steady = vals[len(vals) // 3:] or vals
        res[counter] = dict(kernel=kern, kib_per_dispatch=sum(steady) / len(steady), copy_kernel_kib=copy_kib, scale=factor)
    total = sum(r["kib_per_dispatch"] * r["scale"] for r in res.values()) * 1024
    doc = {}
    if os.path.exists(out):
        with open(out) as f:
            doc = json.load(f)
    doc[config] = dict(hbm_bytes_per_launch=int(total), fetch=res["FETCH_SIZE"], write=res["WRITE_SIZE"])
    with open(out, "w") as f:
        json.dump(doc, f, indent=1, sort_keys=True)
    print(json.dumps(doc[config], indent=1))


def summary(paths):
    for p in paths:
        for k, cs in read_counters(p).items():
            print(os.path.basename(os.path.dirname(p)), k[:100])
            for c, v in sorted(cs.items()):
                print(f"    {c:36s} mean {sum(v) / len(v):16.1f}  dispatches {len(v)}")


def main(argv=None):
    ap = argparse.ArgumentParser()
    sub = ap.add_subparsers(dest="cmd", required=True)
    t = sub.add_parser("traffic")
    t.add_argument("config")
    t.add_argument("fetch_csv")
    t.add_argument("write_csv")
    t.add_argument("--out", default=os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "profiles", "traffic.json"))
    s = sub.add_parser("summary")
    s.add_argument("csv", nargs="+")
    a = ap.parse_args(argv)
    if a.cmd == "traffic":
        traffic(a.config, a.fetch_csv, a.write_csv, a.out)
    else:
        summary(a.csv)


if __name__ == "__main__":
    main(sys.argv[1:])

"""Geometric-mean table from a sweep result file.

    python -m vectorsparse_amd.plot --csv results.csv [--geo spmm_geo.csv]

The numbers behind the reference's figure (plot_spmm.py:43-58: geometric mean of the speed-up over the dense fp16
product per sparsity bucket, vector length, k and kernel path; "fpu" = the fine-grained path, "mma" = the MFMA
path) for the rows `vectorsparse_amd.sweep` writes.  --geo writes them as `label, V, k, mean per bucket...` rows (the
reference's spmm_geo.csv).  The figure itself is not drawn here.
"""
import argparse
import csv
import math
import sys

PATHS = (("cuda", "fpu"), ("wmma", "mma"))


def load(path):
    """{(V, k): {kernel: {bucket: [speed-ups]}}} and the sorted buckets; k (column `k`) is the dense width of
    an SpMM row or the contraction length of an SDDMM row."""
    with open(path) as f:
        rows = list(csv.DictReader(f))
    if not rows:
        raise SystemExit("no rows in %s" % path)
    table, buckets = {}, sorted({float(r["sparsity"]) for r in rows})
    for r in rows:
        key = (int(r["V"]), int(r["k"]))
        table.setdefault(key, {}).setdefault(r["kernel"], {}).setdefault(float(r["sparsity"]), []).append(
            float(r["speedup"]))
    return table, buckets


def geomean(xs):
    xs = [x for x in xs if x > 0]
    return math.exp(sum(math.log(x) for x in xs) / len(xs)) if xs else float("nan")


def geo_rows(table, buckets):
    out = []
    for (V, k) in sorted(table):
        for kernel, label in PATHS:
            if kernel in table[(V, k)]:
                out.append([label, V, k] + [geomean(table[(V, k)][kernel].get(b, [])) for b in buckets])
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--csv", required=True, help="result file written by vectorsparse_amd.sweep --out")
    ap.add_argument("--geo", default=None, help="geometric means to write as CSV")
    args = ap.parse_args(argv)
    table, buckets = load(args.csv)
    rows = geo_rows(table, buckets)
    print("%-6s %3s %5s " % ("path", "V", "k") + "".join("%8s" % ("s=%g" % b) for b in buckets))
    for r in rows:
        print("%-6s %3d %5d " % tuple(r[:3]) + "".join("%8.2f" % x for x in r[3:]))
    if args.geo:
        with open(args.geo, "w", newline="") as f:
            w = csv.writer(f)
            w.writerow(["path", "V", "k"] + ["%g" % b for b in buckets])
            w.writerows(rows)
    return 0


if __name__ == "__main__":
    sys.exit(main())

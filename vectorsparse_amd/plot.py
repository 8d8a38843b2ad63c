"""Speed-up figure and geometric-mean table from a sweep result file.

    python -m vectorsparse_amd.plot --csv results.csv --out spmm_speedup.pdf [--geo spmm_geo.csv]

The counterpart of the reference's plot_spmm.py:60-175 / plot_sddmm.py for the rows `vectorsparse_amd.sweep`
writes: one panel per (vector length, k), sparsity buckets on the x axis, a notched box per kernel path
("fpu" = the fine-grained path, "mma" = the MFMA path) of speed-up over the dense fp16 product, the
geometric means joined by a line, and the break-even line at 1.  --geo writes the geometric means as
`label, V, k, mean per bucket...` rows (the reference's spmm_geo.csv).
"""
import argparse
import csv
import math
import sys

PATHS = (("cuda", "fpu", "steelblue", 0.0), ("wmma", "mma", "lightcoral", 0.35))


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
        for kernel, label, _, _ in PATHS:
            if kernel in table[(V, k)]:
                out.append([label, V, k] + [geomean(table[(V, k)][kernel].get(b, [])) for b in buckets])
    return out


def draw(table, buckets, out_path, title):
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt

    vs = sorted({V for V, _ in table})
    ks = sorted({k for _, k in table})
    fig, axs = plt.subplots(len(vs), len(ks), figsize=(4 * len(ks), 2.8 * len(vs)), squeeze=False)
    xs = list(range(1, len(buckets) + 1))
    for i, V in enumerate(vs):
        for j, k in enumerate(ks):
            ax = axs[i][j]
            ax.plot([0.5, len(buckets) + 0.8], [1, 1], color="purple", linewidth=0.8)
            handles, labels = [], []
            for kernel, label, color, bias in PATHS:
                data = table.get((V, k), {}).get(kernel)
                if not data:
                    continue
                series = [data.get(b, [float("nan")]) for b in buckets]
                ax.plot([x + bias for x in xs], [geomean(s) for s in series], color=color)
                box = ax.boxplot(series, positions=[x + bias for x in xs], notch=True, patch_artist=True, widths=0.28,
                                 boxprops=dict(facecolor=color), capprops=dict(color=color),
                                 whiskerprops=dict(color=color), flierprops=dict(markeredgecolor=color, markersize=2),
                                 medianprops=dict(color="black"), manage_ticks=False)
                handles.append(box["boxes"][0])
                labels.append(label)
            ax.set_xticks(xs)
            ax.set_xticklabels(["%g" % b for b in buckets])
            ax.set_title("V=%d, k=%d" % (V, k), fontsize=9)
            if handles:
                ax.legend(handles, labels, loc="upper left", fontsize=7)
    fig.supxlabel("Sparsity")
    fig.supylabel(title)
    fig.tight_layout()
    fig.savefig(out_path, bbox_inches="tight")
    plt.close(fig)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--csv", required=True, help="result file written by vectorsparse_amd.sweep --out")
    ap.add_argument("--out", default=None, help="figure to write (.pdf, .png, ...)")
    ap.add_argument("--geo", default=None, help="geometric means to write as CSV")
    ap.add_argument("--title", default="Speedup over dense fp16 GEMM (hipBLASLt)")
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
    if args.out:
        draw(table, buckets, args.out, args.title)
    return 0


if __name__ == "__main__":
    sys.exit(main())

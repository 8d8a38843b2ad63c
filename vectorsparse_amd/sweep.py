"""SpMM and SDDMM sweeps against dense fp16 GEMM: a synthetic ResNet-50-shaped grid, or a tree of .smtx files.

    python -m vectorsparse_amd.sweep --out results.csv [--quick] [--op spmm|sddmm] [--hint]
    python -m vectorsparse_amd.sweep --smtx-dir /data/dlmc --matrix-list /data/dlmc/rn50_matrices.txt \\
           --start 0 --end 323 --dimK 64,128,256 --dimV 1,2,4,8 --csv-dir csv --out rn50.csv

The counterpart of the reference's experiment driver (launch.py:11-36 -> job_launcher.py:38-63 ->
ncu_profile.py:80-96, then plot_spmm.py:43-58 / plot_sddmm.py): for every (benchmark, k, V) it times the MFMA
path and the fine-grained path, times hipBLASLt's dense fp16 product of the same shape once, and reports
speed-up = dense duration / kernel duration with the geometric mean per (V, sparsity) bucket.

Benchmarks: without --smtx-dir a synthetic grid (uniform vector placement, exactly round((1-s) n) vectors per
row; the DLMC files are not available offline) - SpMM: M x K of the ResNet-50 layer shapes with N = 256,
SDDMM: square masks M = N in {512..4096} with K in {64, 128, 256}.  With --smtx-dir every .smtx below it, or
the entries [--start, --end) of --matrix-list (one path per line, relative to --smtx-dir, as in the
reference's rn50_matrices.txt); the file's pattern is the sparse operand (SpMM) or the mask (SDDMM), --dimK
the dense width / contraction length (job_launcher.py:41-50: a value <= 0 looks the layer up in --batchsizes,
lines `layer,k`; --dimK-mul scales it), --dimV the vector lengths.
Every point is verified before it is timed (the reference runs its own check on every benchmark it launches with
func = 1, spmm_benchmark.cpp:206-225, sddmm_benchmark.cpp:279-301): one launch per kernel is compared with a
float64 product on a sample of vector rows, by the reference's criterion (no element off by more than 0.5) and by
the maximum relative error (denominator floored at 1e-2 rms); the result file carries `verified` and
`max_rel_err` columns and the run ends with a non-zero status if any point failed.
Durations are device time per launch (HIP events around a HIP-graph replay).  --csv-dir also writes one
duration file per (benchmark, k, v, kernel) point under the names and in the record layout the reference's
plot scripts read (file_name_server.py:6-45, :57-81), dense baseline included.
"""
import argparse
import csv
import glob
import math
import os
import sys

import numpy as np

MS = (64, 128, 256, 512, 1024, 2048)
KS = (64, 147, 256, 576, 1152, 2304, 4608)
SPARSITIES = (0.5, 0.7, 0.8, 0.9, 0.95, 0.98)
VS = (1, 2, 4, 8)
N_DENSE = 256


def spmm_bytes(pat, n_dense):
    k_ref = int(np.unique(pat.column_indices[:pat.nnz_vec]).size)
    return (2 * pat.nnz + 4 * pat.nnz_vec + 4 * (pat.m_vec + 1) + 4 * pat.m_vec
            + 2 * k_ref * n_dense + 2 * pat.m * n_dense)


def sddmm_bytes(pat, k):
    n_ref = int(np.unique(pat.column_indices[:pat.nnz_vec]).size)
    return 2 * pat.m * k + 2 * n_ref * k + 4 * pat.nnz_vec + 4 * (pat.m_vec + 1) + 4 * pat.m_vec + 2 * pat.nnz


SDDMM_SIZES = (512, 1024, 2048, 4096)
SDDMM_KS = (64, 128, 256)


def spmm_grid_pattern(M, K, s, V):
    """The synthetic SpMM point (M x K, sparsity s, vector length V): pattern with values, seeded by the point."""
    from . import colvec_csr as cv
    seed = (M * 1000003 + K * 10007 + int(round(s * 100)) * 101 + V) % (2 ** 31)
    return cv.random_values(cv.uniform_pattern(M // V, K, s, seed, V), seed=V + 7)


def sddmm_grid_pattern(M, s, V):
    """The synthetic SDDMM mask (M x M, sparsity s, vector length V), seeded by the point."""
    from . import colvec_csr as cv
    seed = (M * 1000003 + int(round(s * 100)) * 101 + V) % (2 ** 31)
    return cv.random_values(cv.uniform_pattern(M // V, M, s, seed, V), seed=V + 7)


def sample_rows(m_vec, count=24):
    """Vector rows a verification looks at: the first, the last and an even spread in between."""
    if m_vec <= count:
        return np.arange(m_vec)
    return np.unique(np.linspace(0, m_vec - 1, count).round().astype(np.int64))


def _verdict(got, ref):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    ref = np.asarray(ref, dtype=np.float64).reshape(-1)
    if ref.size == 0:
        return True, 0.0
    floor = max(1e-2 * float(np.sqrt(np.mean(ref * ref))), 1e-30)
    rel = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)))
    ok = bool(np.all(np.isfinite(got))) and int(np.sum(np.abs(got - ref) > 0.5)) == 0 and rel <= 1e-2
    return ok, rel


def verify_spmm(pat, B, out_host):
    """(passed, max relative error) of an SpMM result on a sample of vector rows against a float64 product."""
    V = pat.vec_length
    rows = sample_rows(pat.m_vec)
    Bd = np.asarray(B, dtype=np.float64)
    got, ref = [], []
    for i in rows:
        lo, hi = int(pat.row_offsets[i]), int(pat.row_offsets[i + 1])
        vals = np.asarray(pat.values[lo:hi], dtype=np.float64).reshape(hi - lo, V)
        ref.append(vals.T @ Bd[pat.column_indices[lo:hi]])
        got.append(out_host[i * V:(i + 1) * V])
    return _verdict(np.concatenate(got), np.concatenate(ref))


def verify_sddmm(pat, A, B, out_host):
    """(passed, max relative error) of an SDDMM result on a sample of vector rows against float64 dot products."""
    V = pat.vec_length
    rows = sample_rows(pat.m_vec)
    Ad, Bd = np.asarray(A, dtype=np.float64), np.asarray(B, dtype=np.float64)
    out_host = np.asarray(out_host).reshape(-1, V)
    got, ref = [], []
    for i in rows:
        lo, hi = int(pat.row_offsets[i]), int(pat.row_offsets[i + 1])
        ref.append(Bd[pat.column_indices[lo:hi]] @ Ad[i * V:(i + 1) * V].T)    # [nonzero][v]
        got.append(out_host[lo:hi])
    return _verdict(np.concatenate(got), np.concatenate(ref))


def geomean(xs):
    xs = [x for x in xs if x > 0]
    return math.exp(sum(math.log(x) for x in xs) / len(xs)) if xs else float("nan")


def int_list(text):
    return tuple(int(x) for x in str(text).split(",") if x.strip())


def sparsity_bucket(name, sparsity):
    """The reference's plot scripts bucket a DLMC file by the sparsity directory in its path
    (plot_spmm.py:45-58, '0.95' and '0.98' looked for before '0.9'); other names fall back to the
    pattern's own sparsity."""
    parts = name.replace("\\", "/").split("/")
    for tag in ("0.95", "0.98", "0.9", "0.8", "0.7", "0.5"):
        if tag in parts:
            return float(tag)
    return round(float(sparsity), 2)


def file_benchmarks(smtx_dir, matrix_list=None, start=0, end=None):
    """[(name below smtx_dir without extension, path)] - every .smtx below smtx_dir, or the entries
    [start, end) of a list file (job_launcher.py:34-40: one benchmark per line, '.smtx' optional)."""
    if matrix_list:
        with open(matrix_list) as f:
            names = [line.strip() for line in f if line.strip()]
        names = names[start:end]
        names = [n[:-len(".smtx")] if n.endswith(".smtx") else n for n in names]
        return [(n, os.path.join(smtx_dir, n + ".smtx")) for n in names]
    paths = sorted(glob.glob(os.path.join(smtx_dir, "**", "*.smtx"), recursive=True))
    return [(os.path.relpath(p, smtx_dir)[:-len(".smtx")], p) for p in paths][start:end]


def layer_widths(path):
    """`layer,k` lines (the reference's rn50_batchsizes.txt, job_launcher.py:25-31) -> {layer: k}."""
    table = {}
    if path:
        with open(path) as f:
            for line in f:
                if "," in line:
                    layer, k = line.strip().split(",")[:2]
                    table[layer] = int(k)
    return table


def widths_for(name, dim_ks, dim_k_mul, table):
    """The k values to run for one benchmark: the requested ones, a value <= 0 replaced by the layer's own."""
    out = []
    for k in dim_ks:
        if k <= 0:
            layer = name.split("/")[-1]
            if layer not in table:
                raise SystemExit("--dimK <= 0 needs a --batchsizes entry for layer %s" % layer)
            k = table[layer]
        out.append(k * dim_k_mul)
    return out


def report(path, rows, title):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
        w.writeheader()
        w.writerows(rows)
    print("\n" + title + ", by vector length and sparsity")
    buckets = sorted({r["sparsity"] for r in rows})
    print("%-12s" % "kernel/V" + "".join("%9s" % ("s=%.2f" % b) for b in buckets))
    for kernel in ("wmma", "cuda"):
        for V in sorted({r["V"] for r in rows}):
            line = "%-12s" % ("%s V=%d" % (kernel, V))
            for b in buckets:
                xs = [r["speedup"] for r in rows if r["kernel"] == kernel and r["V"] == V and r["sparsity"] == b]
                line += "%9.2f" % geomean(xs)
            print(line)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--out", default="spmm_sweep.csv")
    ap.add_argument("--op", choices=["spmm", "sddmm"], default="spmm")
    ap.add_argument("--quick", action="store_true", help="a 3 x 3 x 3 corner of the synthetic grid")
    ap.add_argument("--smtx-dir", default=None, help="sweep .smtx files below this directory instead of the grid")
    ap.add_argument("--matrix-list", default=None, help="file with one benchmark per line, relative to --smtx-dir")
    ap.add_argument("--start", type=int, default=0, help="first entry of the list (or of the sorted directory) to run")
    ap.add_argument("--end", type=int, default=None, help="one past the last entry to run")
    ap.add_argument("--dimK", default=None,
                    help="comma list: dense width (SpMM) / contraction length (SDDMM) for file benchmarks, default 256 "
                         "(SpMM) or 64,128,256 (SDDMM); <= 0: the layer's own width from --batchsizes")
    ap.add_argument("--dimK-mul", type=int, default=1, help="scale every k by this factor")
    ap.add_argument("--batchsizes", default=None, help="file of `layer,k` lines for --dimK <= 0")
    ap.add_argument("--dimV", default="1,2,4,8", help="comma list of vector lengths")
    ap.add_argument("--hint", action="store_true",
                    help="SpMM through the batched entry point with the pattern's nonzero count and longest row "
                         "(workgroups sized by the real row lengths) instead of the reference-shaped entry points")
    ap.add_argument("--iters", type=int, default=100, help="launches per timed HIP-graph replay")
    ap.add_argument("--no-verify", action="store_true", help="time without checking the results first")
    ap.add_argument("--csv-dir", default=None,
                    help="also write <csv-dir>/<spmm|sddmm>/<benchmark>_<kernel>_half_sort[_<alg>]_k<k>_v<v>.csv, one "
                         "profiler-style Duration record each, as the reference's plot scripts expect them")
    args = ap.parse_args(argv)
    if args.matrix_list and not args.smtx_dir:
        raise SystemExit("--matrix-list needs --smtx-dir")

    import torch

    from . import colvec_csr as cv
    from . import ops
    from .benchmark_common import duration_csv_path, time_launches, write_duration_csv

    vs = int_list(args.dimV)
    spmm = args.op == "spmm"

    # (benchmark name, sparsity bucket or None, V -> pattern, the k values to run)
    cases = []
    if args.smtx_dir:
        table = layer_widths(args.batchsizes)
        dim_ks = int_list(args.dimK) if args.dimK else ((N_DENSE,) if spmm else (64, 128, 256))
        for name, path in file_benchmarks(args.smtx_dir, args.matrix_list, args.start, args.end):
            cases.append((name, None, (lambda V, path=path: cv.read_smtx(path, V)),
                          widths_for(name, dim_ks, args.dimK_mul, table)))
    elif spmm:
        ms, ks, ss = (MS, KS, SPARSITIES) if not args.quick else ((64, 512, 2048), (256, 1152, 4608), (0.7, 0.9, 0.98))
        widths = [k * args.dimK_mul for k in (int_list(args.dimK) if args.dimK else (N_DENSE,))]
        for M in ms:
            for K in ks:
                for s in ss:
                    def make(V, M=M, K=K, s=s):
                        return spmm_grid_pattern(M, K, s, V)
                    cases.append(("synthetic/uniform/%g/m%d_k%d" % (s, M, K), s, make, widths))
    else:
        sizes, ks, ss = (SDDMM_SIZES, SDDMM_KS, SPARSITIES) if not args.quick else \
            ((512, 2048), (64, 256), (0.7, 0.9, 0.98))
        widths = [k * args.dimK_mul for k in (int_list(args.dimK) if args.dimK else ks)]
        for M in sizes:
            for s in ss:
                def make(V, M=M, s=s):
                    return sddmm_grid_pattern(M, s, V)
                cases.append(("synthetic/uniform/%g/m%d_n%d" % (s, M, M), s, make, widths))

    def per_point(bm, dim_k, V, kernel, name, us):
        if args.csv_dir:
            write_duration_csv(duration_csv_path(args.csv_dir, bm, dim_k, V, kernel, args.op), name, us)

    rows, dense_us, failed = [], {}, 0
    for name, bucket, make, widths in cases:
        for V in vs:
            pat = make(V)
            if pat.values is None:
                pat = cv.random_values(pat, seed=V + 7)
            if pat.nnz_vec == 0:
                continue
            M, n = pat.m, pat.n
            s = bucket if bucket is not None else sparsity_bucket(name, pat.sparsity)
            prob = ops.DeviceProblem(pat, sort=True)
            for k in widths:
                if spmm:
                    # C[M, k] = A_sparse[M, n] B[n, k]
                    B_host = cv.dense_uniform(n, k, seed=11)
                    B = torch.from_numpy(B_host).cuda()
                    out = torch.empty((M, k), dtype=torch.float16, device="cuda")
                    check = lambda: verify_spmm(pat, B_host, out.cpu().numpy())
                    if (M, n, k) not in dense_us:
                        A = torch.randn((M, n), dtype=torch.float16, device="cuda")
                        dense_us[(M, n, k)] = time_launches(torch, lambda: torch.matmul(A, B, out=out), args.iters)
                    run = {kern: (lambda kern=kern: prob.spmm(B, kernel=kern, out=out, row_length_hint=args.hint))
                           for kern in ("wmma", "cuda")}
                    flops, nbytes = 2.0 * pat.nnz * k, spmm_bytes(pat, k)
                    names = {"wmma": "spmm_mfma_kernel", "cuda": "spmm_valu_kernel"}
                else:
                    # out[nnz] = (A[M, k] B[n, k]^T) sampled on the mask
                    A = torch.randn((M, k), dtype=torch.float16, device="cuda")
                    B = torch.randn((n, k), dtype=torch.float16, device="cuda")
                    out = torch.empty((pat.nnz_vec, V), dtype=torch.float16, device="cuda")
                    A_host, B_host = A.cpu().numpy(), B.cpu().numpy()
                    check = lambda: verify_sddmm(pat, A_host, B_host, out.cpu().numpy())
                    if (M, n, k) not in dense_us:
                        full = torch.empty((M, n), dtype=torch.float16, device="cuda")
                        dense_us[(M, n, k)] = time_launches(torch, lambda: torch.matmul(A, B.t(), out=full), args.iters)
                        del full
                    run = {kern: (lambda kern=kern: prob.sddmm(A, B, kernel=kern, out=out)) for kern in ("wmma", "cuda")}
                    flops, nbytes = 2.0 * pat.nnz * k, sddmm_bytes(pat, k)
                    names = {"wmma": "sddmm_mfma_kernel", "cuda": "sddmm_valu_kernel"}
                dense = dense_us[(M, n, k)]
                per_point(name, k, V, "dense", "hipblaslt_gemm_f16", dense)
                for kern in ("wmma", "cuda"):
                    verified, rel = "", float("nan")
                    if not args.no_verify:
                        out.fill_(float("nan"))
                        run[kern]()
                        torch.cuda.synchronize()
                        ok, rel = check()
                        verified = int(ok)
                        if not ok:
                            failed += 1
                            print("VERIFICATION FAILED: %s k=%d V=%d %s max relative error %.3e" % (name, k, V, kern, rel),
                                  flush=True)
                    us = time_launches(torch, run[kern], args.iters)
                    per_point(name, k, V, kern, names[kern], us)
                    rows.append({"op": args.op, "bm": name, "k": k, "M": M, "K": n if spmm else k, "N": k if spmm else n,
                                 "sparsity": round(s, 4), "V": V, "kernel": kern, "nnz_vec": pat.nnz_vec,
                                 "us": round(us, 3), "dense_us": round(dense, 3), "speedup": round(dense / us, 4),
                                 "tflops": round(flops / us * 1e-6, 3), "gbs": round(nbytes / us * 1e-3, 1),
                                 "verified": verified, "max_rel_err": "%.3e" % rel})
                print("%s M=%d n=%d k=%d s=%.2f V=%d  wmma %.2f us  cuda %.2f us  dense %.2f us" % (
                    name, M, n, k, s, V, rows[-2]["us"], rows[-1]["us"], dense), flush=True)
    if not rows:
        raise SystemExit("nothing to run")
    report(args.out, rows, "SpMM: geometric-mean speed-up over dense fp16 GEMM (hipBLASLt)" if spmm else
           "SDDMM: geometric-mean speed-up over the dense fp16 product A B^T (hipBLASLt)")
    if failed:
        print("%d point(s) failed verification" % failed, flush=True)
        return 1
    if not args.no_verify:
        print("all %d points verified" % len(rows), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

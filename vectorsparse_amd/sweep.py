"""ResNet-50-shaped SpMM sweep (and a square-mask SDDMM sweep) against dense fp16 GEMM.

    python -m vectorsparse_amd.sweep --out results.csv [--quick] [--op spmm|sddmm]

The counterpart of the reference's experiment driver (launch.py:11-36 -> job_launcher.py:38-63 ->
ncu_profile.py:80-96, then plot_spmm.py:43-58): for every (M, K, sparsity, V) of the grid it times
the MFMA path and the fine-grained path, times hipBLASLt's dense fp16 GEMM once per (M, K), and
reports speed-up = dense duration / kernel duration with the geometric mean per (V, sparsity)
bucket.  Patterns are synthetic (uniform vector placement, exactly round((1-s)K) vectors per row)
because the DLMC files are not available offline; any directory of .smtx files can be swept instead
with --smtx-dir.  Durations are device time per launch (HIP events around a HIP-graph replay).
--csv-dir also writes one duration file per (benchmark, k, v, kernel) point under the names and in the
record layout the reference's plot scripts read (file_name_server.py:6-45, :57-81), dense baseline included.
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


def geomean(xs):
    xs = [x for x in xs if x > 0]
    return math.exp(sum(math.log(x) for x in xs) / len(xs)) if xs else float("nan")


def sddmm_bytes(pat, k):
    n_ref = int(np.unique(pat.column_indices[:pat.nnz_vec]).size)
    return 2 * pat.m * k + 2 * n_ref * k + 4 * pat.nnz_vec + 4 * (pat.m_vec + 1) + 4 * pat.m_vec + 2 * pat.nnz


def sddmm_sweep(args, torch, cv, ops, time_launches):
    sizes, ks, ss = ((512, 1024, 2048, 4096), (64, 128, 256), SPARSITIES) if not args.quick else \
        ((512, 2048), (64, 256), (0.7, 0.9, 0.98))
    rows, dense_us = [], {}
    for M in sizes:
        for K in ks:
            A = torch.randn((M, K), dtype=torch.float16, device="cuda")
            B = torch.randn((M, K), dtype=torch.float16, device="cuda")
            full = torch.empty((M, M), dtype=torch.float16, device="cuda")
            dense_us[(M, K)] = time_launches(torch, lambda: torch.matmul(A, B.t(), out=full), args.iters)
            for s in ss:
                for V in VS:
                    seed = (M * 1000003 + K * 10007 + int(round(s * 100)) * 101 + V) % (2 ** 31)
                    pat = cv.uniform_pattern(M // V, M, s, seed, V)
                    prob = ops.DeviceProblem(pat, sort=True)
                    out = torch.empty((pat.nnz_vec, V), dtype=torch.float16, device="cuda")
                    flops = 2.0 * pat.nnz * K
                    bm = "synthetic/uniform/%g/m%d_n%d" % (s, M, M)
                    args.per_point(bm, K, V, "dense", "sddmm", "hipblaslt_gemm_f16", dense_us[(M, K)])
                    for kernel in ("wmma", "cuda"):
                        us = time_launches(torch, lambda: prob.sddmm(A, B, kernel=kernel, out=out), args.iters)
                        args.per_point(bm, K, V, kernel, "sddmm",
                                       "sddmm_mfma_kernel" if kernel == "wmma" else "sddmm_valu_kernel", us)
                        rows.append({"bm": "synthetic", "M": M, "K": K, "N": M, "sparsity": round(s, 4), "V": V,
                                     "kernel": kernel, "nnz_vec": pat.nnz_vec, "us": round(us, 3),
                                     "dense_us": round(dense_us[(M, K)], 3),
                                     "speedup": round(dense_us[(M, K)] / us, 4),
                                     "tflops": round(flops / us * 1e-6, 3),
                                     "gbs": round(sddmm_bytes(pat, K) / us * 1e-3, 1)})
                    print("M=N=%d K=%d s=%.2f V=%d  wmma %.2f us  cuda %.2f us  dense %.2f us" % (
                        M, K, s, V, rows[-2]["us"], rows[-1]["us"], dense_us[(M, K)]), flush=True)
    report(args.out, rows, "SDDMM: geometric-mean speed-up over the dense fp16 product A B^T (hipBLASLt)")
    return 0


def report(path, rows, title):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
        w.writeheader()
        w.writerows(rows)
    print("\n" + title + ", by vector length and sparsity")
    buckets = sorted({r["sparsity"] for r in rows})
    print("%-12s" % "kernel/V" + "".join("%9s" % ("s=%.2f" % b) for b in buckets))
    for kernel in ("wmma", "cuda"):
        for V in VS:
            line = "%-12s" % ("%s V=%d" % (kernel, V))
            for b in buckets:
                xs = [r["speedup"] for r in rows if r["kernel"] == kernel and r["V"] == V and r["sparsity"] == b]
                line += "%9.2f" % geomean(xs)
            print(line)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--out", default="spmm_sweep.csv")
    ap.add_argument("--quick", action="store_true", help="a 3 x 3 x 3 corner of the grid")
    ap.add_argument("--smtx-dir", default=None, help="sweep every .smtx under this directory instead")
    ap.add_argument("--op", choices=["spmm", "sddmm"], default="spmm",
                    help="sddmm: masks of M = N in {512, 1024, 2048, 4096} x contraction K in {64, 128, 256} "
                         "(the counterpart of the reference's SDDMM figure), dense baseline = the full A B^T")
    ap.add_argument("--hint", action="store_true",
                    help="call through the batched entry point with the pattern's nonzero count (workgroups sized "
                         "by the real row lengths) instead of the reference-shaped entry points")
    ap.add_argument("--iters", type=int, default=100, help="launches per timed HIP-graph replay")
    ap.add_argument("--csv-dir", default=None,
                    help="also write <csv-dir>/<spmm|sddmm>/<benchmark>_<kernel>_half_sort[_<alg>]_k<k>_v<v>.csv, one "
                         "profiler-style Duration record each, as the reference's plot scripts expect them")
    args = ap.parse_args(argv)

    import torch

    from . import colvec_csr as cv
    from . import ops
    from .benchmark_common import duration_csv_path, time_launches, write_duration_csv

    def per_point(bm, dim_k, V, kernel, job, name, us):
        if args.csv_dir:
            write_duration_csv(duration_csv_path(args.csv_dir, bm, dim_k, V, kernel, job), name, us)
    args.per_point = per_point

    if args.op == "sddmm":
        return sddmm_sweep(args, torch, cv, ops, time_launches)
    ms, ks, ss = (MS, KS, SPARSITIES) if not args.quick else ((64, 512, 2048), (256, 1152, 4608), (0.7, 0.9, 0.98))
    cases = []
    if args.smtx_dir:
        for path in sorted(glob.glob(os.path.join(args.smtx_dir, "**", "*.smtx"), recursive=True)):
            for V in VS:
                cases.append((path, V))
    else:
        for M in ms:
            for K in ks:
                for s in ss:
                    for V in VS:
                        cases.append(((M, K, s), V))

    dense_us = {}
    rows = []
    for spec, V in cases:
        if isinstance(spec, str):
            pat = cv.read_smtx(spec, V)
            M, K, s = pat.m, pat.n, pat.sparsity
            label = os.path.basename(spec)
            bm = os.path.relpath(spec, args.smtx_dir)
        else:
            M, K, s = spec
            seed = (M * 1000003 + K * 10007 + int(round(s * 100)) * 101 + V) % (2 ** 31)
            pat = cv.uniform_pattern(M // V, K, s, seed, V)
            label = "synthetic"
            bm = "synthetic/uniform/%g/m%d_k%d" % (s, M, K)
        pat = cv.random_values(pat, seed=V + 7)
        B = torch.from_numpy(cv.dense_uniform(K, N_DENSE, seed=11)).cuda()
        out = torch.empty((M, N_DENSE), dtype=torch.float16, device="cuda")
        if (M, K) not in dense_us:
            A = torch.randn((M, K), dtype=torch.float16, device="cuda")
            dense_us[(M, K)] = time_launches(torch, lambda: torch.matmul(A, B, out=out), args.iters)
        args.per_point(bm, N_DENSE, V, "dense", "spmm", "hipblaslt_gemm_f16", dense_us[(M, K)])
        prob = ops.DeviceProblem(pat, sort=True)
        flops = 2.0 * pat.nnz * N_DENSE
        nbytes = spmm_bytes(pat, N_DENSE)
        for kernel in ("wmma", "cuda"):
            us = time_launches(torch, lambda: prob.spmm(B, kernel=kernel, out=out, row_length_hint=args.hint), args.iters)
            args.per_point(bm, N_DENSE, V, kernel, "spmm", "spmm_mfma_kernel" if kernel == "wmma" else "spmm_valu_kernel", us)
            rows.append({"bm": label, "M": M, "K": K, "N": N_DENSE, "sparsity": round(s, 4), "V": V,
                         "kernel": kernel, "nnz_vec": pat.nnz_vec, "us": round(us, 3),
                         "dense_us": round(dense_us[(M, K)], 3), "speedup": round(dense_us[(M, K)] / us, 4),
                         "tflops": round(flops / us * 1e-6, 3), "gbs": round(nbytes / us * 1e-3, 1)})
        print("M=%d K=%d s=%.2f V=%d  wmma %.2f us  cuda %.2f us  dense %.2f us" % (
            M, K, s, V, rows[-2]["us"], rows[-1]["us"], dense_us[(M, K)]), flush=True)

    report(args.out, rows, "SpMM: geometric-mean speed-up over dense fp16 GEMM (hipBLASLt)")
    return 0


if __name__ == "__main__":
    sys.exit(main())

"""Command line of the SpMM operator, same positional arguments as the reference's
`spmm_benchmark` (spmm_benchmark.cpp:473-513):

    python -m vectorsparse_amd.spmm_benchmark [bm] [k] [v] [kernel] [sort] [function] [sparse] [mixed]

    bm       .smtx file (pattern; every nonzero becomes a v x 1 vector) or synthetic:M,K,sparsity,seed
    k        dense width (columns of B and C)
    v        vector length, 1 / 2 / 4 / 8
    kernel   0 = MFMA path (wmmaSpmm), 1 = fine-grained path (cudaSpmm); 2, 3 (Sputnik, cuSPARSE) unsupported
    sort     1 = rows dispatched longest first (SortedRowSwizzle), 0 = in order; 2 (MFMA path; not in the
             reference) = longest first with rows far longer than the rest dispatched in parts (vs_spmm_row_parts)
    function 1 = verify the result, 0 = skip
    sparse   1 = SpMM, 0 = dense fp16 GEMM baseline (hipBLASLt through torch); 2 (Blocked-ELL) unsupported
    mixed    1 = fp16 operands; 0 (fp32) unsupported, as in the reference's stubs

Operands are generated as the reference does (rhs then values from the same restarted engine).
Verification (function = 1) compares with a float64 product of the expanded matrix computed on
the host by numpy, prints the reference's verdict line and the 1e-2 relative check.
"""
import sys

import numpy as np


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 8 or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0 if argv and argv[0] in ("-h", "--help") else 2
    bm = argv[0]
    k, v, kernel, sort, func, sparse, mixed = (int(a) for a in argv[1:])
    import torch

    from . import ops, refgen
    from .benchmark_common import load_pattern, time_launches, verdict

    if not mixed:
        print("single precision is not supported (the reference's float overloads are stubs)")
        return 1
    if v not in (1, 2, 4, 8):
        print("Unsupported Vector Length!")
        return 1
    pat = load_pattern(bm, v)
    m, n = pat.m, pat.n
    print("Problem size: M: %d, N: %d, nnz: %d, K: %d" % (m, n, pat.nnz, k))

    if sparse == 0:
        lhs = refgen.make_dense_matrix(m, n)
        rhs = refgen.make_dense_matrix(n, k)
        a, b = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()
        out = torch.empty((m, k), dtype=torch.float16, device="cuda")
        print("Dense Baseline")
        us = time_launches(torch, lambda: torch.matmul(a, b, out=out))
        print("dense GEMM %dx%dx%d: %.2f us, %.2f TFLOP/s" % (m, n, k, us, 2.0 * m * n * k / us * 1e-6))
        if func:
            ref = lhs.astype(np.float64) @ rhs.astype(np.float64)
            return 0 if verdict("hipBLASLt", out.cpu().numpy(), ref) else 1
        return 0
    if sparse != 1:
        print("Blocked-ELL is a cuSPARSE baseline of the reference and is not part of this library")
        return 1
    if kernel not in (0, 1):
        print("Unsupported Kernel")
        return 1

    rhs = refgen.make_dense_matrix(n, k)
    values = refgen.make_dense_matrix(1, pat.nnz).reshape(pat.nnz_vec, v)
    pat = pat.with_values(values)
    if sort not in (0, 1, 2) or (sort == 2 and (kernel != 0 or k % 4 != 0)):
        print("Unsupported Sort")
        return 1
    prob = ops.DeviceProblem(pat, sort=bool(sort))
    b = torch.from_numpy(rhs).cuda()
    out = torch.empty((m, k), dtype=torch.float16, device="cuda")
    name = "wmma" if kernel == 0 else "cuda"
    print("Using MFMA" if kernel == 0 else "Using fine-grained VALU")
    if sort == 2:
        parts = prob.row_parts(0)[0]
        print("Rows in parts: %d slots, %d rows in up to %d parts" % (parts.n_slots, parts.n_split, parts.parts_max))
        step = lambda: prob.spmm_row_parts(b, out=out)
    else:
        step = lambda: prob.spmm(b, kernel=name, out=out)
    step()
    torch.cuda.synchronize()
    us = time_launches(torch, step)
    print("SpMM %s V=%d: %.2f us, %.2f effective TFLOP/s (2*nnz*k)" % (name, v, us, 2.0 * pat.nnz * k / us * 1e-6))
    if func:
        ref = np.zeros((m, k), dtype=np.float64)
        rhs64 = rhs.astype(np.float64)
        vals64 = pat.values.astype(np.float64)
        for i in range(pat.m_vec):
            lo, hi = int(pat.row_offsets[i]), int(pat.row_offsets[i + 1])
            if hi > lo:
                ref[i * v:(i + 1) * v] = vals64[lo:hi].T @ rhs64[pat.column_indices[lo:hi]]
        return 0 if verdict("SPMM", out.cpu().numpy(), ref) else 1
    return 0


if __name__ == "__main__":
    sys.exit(main())

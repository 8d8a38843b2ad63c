"""Command line of the SDDMM operator, same positional arguments as the reference's
`sddmm_benchmark` (sddmm_benchmark.cpp:392-435):

    python -m vectorsparse_amd.sddmm_benchmark [bm] [k] [v] [kernel] [alg] [sort] [function] [sparse] [mixed]

    bm       .smtx file (the mask pattern) or synthetic:M,N,sparsity,seed
    k        contraction length
    v        vector length, 1 / 2 / 4 / 8
    kernel   0 = MFMA path (wmmaSddmm), 1 = cross-lane path (cudaSddmm); 2, 3 unsupported
    alg      0..2 accepted (one MFMA kernel serves the reference's three schedules), 3 rejected
    sort     1 = rows dispatched longest first, 0 = in order; 2 (MFMA path, k % 8 == 0; not in the reference) =
             longest first with long rows dispatched in parts (vs_spmm_row_parts, vs_wmma_sddmm_f16_row_parts)
    function 1 = verify the result, 0 = skip
    sparse   1 = SDDMM, 0 = dense fp16 A*B^T baseline (hipBLASLt through torch)
    mixed    1 = fp16 operands; 0 unsupported

lhs and rhs are generated as the reference does (both from the same restarted engine).
"""
import sys

import numpy as np


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    if len(argv) != 9 or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0 if argv and argv[0] in ("-h", "--help") else 2
    bm = argv[0]
    k, v, kernel, alg, sort, func, sparse, mixed = (int(a) for a in argv[1:])
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
    lhs = refgen.make_dense_matrix(m, k)
    rhs = refgen.make_dense_matrix(n, k)
    a, b = torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda()

    if sparse == 0:
        out = torch.empty((m, n), dtype=torch.float16, device="cuda")
        print("Dense Baseline")
        us = time_launches(torch, lambda: torch.matmul(a, b.t(), out=out))
        print("dense GEMM %dx%dx%d: %.2f us, %.2f TFLOP/s" % (m, n, k, us, 2.0 * m * n * k / us * 1e-6))
        if func:
            ref = lhs.astype(np.float64) @ rhs.astype(np.float64).T
            return 0 if verdict("hipBLASLt", out.cpu().numpy(), ref) else 1
        return 0
    if kernel not in (0, 1):
        print("unsupported kernel")
        return 1

    prob = ops.DeviceProblem(pat, sort=bool(sort))
    out = torch.empty((pat.nnz_vec, v), dtype=torch.float16, device="cuda")
    name = "wmma" if kernel == 0 else "cuda"
    print("Using MFMA" if kernel == 0 else "Using cross-lane VALU")
    if sort not in (0, 1, 2) or (sort == 2 and (kernel != 0 or k % 8 != 0)):
        print("unsupported sort")
        return 1
    if sort == 2:
        parts = prob.row_parts(256)[0]
        print("Rows in parts: %d slots, %d rows in up to %d parts" % (parts.n_slots, parts.n_split, parts.parts_max))
        step = lambda: prob.sddmm_row_parts(a, b, out=out)
    else:
        step = lambda: prob.sddmm(a, b, kernel=name, out=out, algorithm=alg)
    step()
    torch.cuda.synchronize()
    us = time_launches(torch, step)
    print("SDDMM %s V=%d: %.2f us, %.2f effective TFLOP/s (2*nnz*k)" % (name, v, us, 2.0 * pat.nnz * k / us * 1e-6))
    if func:
        rows = np.repeat(np.arange(pat.m_vec), pat.row_lengths())
        lhs64, rhs64 = lhs.astype(np.float64), rhs.astype(np.float64)
        gathered = rhs64[pat.column_indices[:pat.nnz_vec]]
        ref = np.stack([np.einsum("jk,jk->j", lhs64[rows * v + t], gathered) for t in range(v)], axis=1)
        return 0 if verdict("SDDMM", out.cpu().numpy().reshape(-1), ref.reshape(-1)) else 1
    return 0


if __name__ == "__main__":
    sys.exit(main())

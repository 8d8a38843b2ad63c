"""The three operators on a dispatch list of row parts (SpMM, SDDMM, softmax) on seeded random patterns: vector
length, row-length family, limit, dense widths, batch on a shared pattern and launch options all vary per seed; every
output is checked against the CPU oracle through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import numpy_oracle as no
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


def _row_lengths(rng, kind, m_vec, n):
    if kind == 0:      # heavy tail
        lengths = np.minimum((rng.pareto(1.1, m_vec) + 0.05) * n * 0.1, n)
    elif kind == 1:    # a few dense rows among very short ones
        lengths = np.where(rng.random(m_vec) < 0.1, n, rng.integers(0, 20, m_vec))
    elif kind == 2:    # uniform density
        lengths = rng.binomial(n, rng.uniform(0.05, 0.9), size=m_vec)
    elif kind == 3:    # all rows dense
        lengths = np.full(m_vec, n)
    else:              # half the rows empty, the others of any length
        lengths = np.where(rng.random(m_vec) < 0.5, 0, rng.integers(1, n + 1, m_vec))
    return lengths.astype(np.int64)


@pytest.mark.parametrize("seed", range(40))
def test_three_operators_on_one_list(gpu, seed):
    rng = np.random.default_rng(20000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    m_vec = int(rng.integers(1, 160))
    n = int(rng.integers(64, 3000))
    ro, ci = cv._pattern_from_lengths(rng, m_vec, n, _row_lengths(rng, seed % 5, m_vec, n))
    pat = cv.ColVecCSR(m_vec, n, V, ro, ci).validate()
    limit = int(rng.choice([0, 1, 64, 65, 200, 512, 1000, 2304]))
    parts = ops.RowParts(m_vec, ro, limit)
    batch = int(rng.choice([1, 1, 2, 3]))
    options = {"spmm_parts_launches": int(rng.integers(0, 3))}
    if rng.random() < 0.5:
        options["spmm_waves"] = int(rng.choice([1, 2, 3, 4, 8]))
    if rng.random() < 0.5:
        options["spmm_pipe"] = int(rng.integers(1, 3))
    if rng.random() < 0.3:
        options["spmm_cols_per_lane"] = int(rng.choice([4, 8]))
    what = "seed %d V%d m_vec %d n %d nnz_vec %d limit %d batch %d %s" % (seed, V, m_vec, n, pat.nnz_vec, limit, batch,
                                                                        options)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, cid = d(parts.slots), d(pat.column_indices)

    # SpMM: per-problem values and dense operands; two calls on one workspace
    N = int(rng.choice([4, 8, 12, 40, 64, 100, 128, 200, 256, 264]))
    if batch > 1:
        N = (N + 7) // 8 * 8            # strides between problems are multiples of 16 bytes
    vals = np.stack([cv.random_values(pat, seed=seed * 7 + b).values for b in range(batch)])
    Bs = np.stack([cv.dense_uniform(n, N, seed=seed * 11 + b) for b in range(batch)])
    need = ops.spmm_row_parts_workspace_bytes(V, N, parts.n_split, parts.parts_max, batch=batch)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda") if need else None
    out = torch.full((batch, pat.m, N), 5.0, dtype=torch.float16, device="cuda")
    with _lib.thread_options(**options):
        for _ in range(2):
            ops.spmm_row_parts(V, N, n, parts, slots, pat.nnz_vec, cid, d(vals), d(Bs), out, ws)
    torch.cuda.synchronize()
    for b in range(batch):
        ref = co.spmm_host_ref_f32(m_vec, V, N, n, ro, ci, vals[b], Bs[b])
        assert_parity(out[b].cpu().numpy(), ref, "SpMM, problem %d, %s" % (b, what))

    # SDDMM on the same list
    K = int(rng.choice([8, 16, 40, 64, 96, 128, 256, 264]))
    lhs = np.stack([cv.dense_normal(pat.m, K, seed=seed * 13 + b) for b in range(batch)])
    rhs = np.stack([cv.dense_normal(n, K, seed=seed * 17 + b) for b in range(batch)])
    got = torch.full((batch, pat.nnz_vec, V), 5.0, dtype=torch.float16, device="cuda")
    ops.sddmm_row_parts(K, n, parts, slots, pat.nnz_vec, cid, d(lhs), d(rhs), got, V)
    torch.cuda.synchronize()
    for b in range(batch):
        ref = co.sddmm_host_ref_f16(m_vec, K, V, ro, ci, lhs[b], rhs[b])
        assert_parity(got[b].cpu().numpy().reshape(-1), np.asarray(ref).reshape(-1), "SDDMM, problem %d, %s" % (b, what))

    # softmax on the same list, in place
    scores = (rng.standard_normal((batch, pat.nnz_vec, V)) * 3).astype(np.float16)
    need = ops.sparse_softmax_row_parts_workspace_bytes(V, parts.n_split, parts.parts_max, batch=batch)
    sm_ws = torch.empty(need, dtype=torch.uint8, device="cuda") if need else None
    x = d(scores)
    ops.sparse_softmax_row_parts(V, parts, slots, x, scale=0.3, workspace=sm_ws)
    torch.cuda.synchronize()
    for b in range(batch):
        assert_parity(x[b].cpu().numpy(), no.sparse_softmax_ref(m_vec, V, ro, scores[b], 0.3),
                      "softmax, problem %d, %s" % (b, what))

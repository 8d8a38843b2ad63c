"""Parity on EVERY point of the two synthetic sweeps, not a sample: the 1,008 SpMM points of the ResNet-50-shaped
grid (M x K x sparsity x V, N = 256) and the 288 SDDMM points (M = N x K x sparsity x V), both kernel paths, against
the CPU oracle on the patterns the sweep driver itself times (same seeds).  The reference checks every benchmark it
launches with func = 1 (spmm_benchmark.cpp:206-225, sddmm_benchmark.cpp:279-301)."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import ops, sweep
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu

THREADS = min(co.max_threads(), 16)


@pytest.mark.parametrize("V", sweep.VS)
@pytest.mark.parametrize("M", sweep.MS)
def test_every_spmm_point_of_the_grid(gpu, M, V):
    points = 0
    for K in sweep.KS:
        B = cv.dense_uniform(K, sweep.N_DENSE, seed=11)
        Bd = torch.from_numpy(B).cuda()
        for s in sweep.SPARSITIES:
            pat = sweep.spmm_grid_pattern(M, K, s, V)
            if pat.nnz_vec == 0:
                continue
            ref = co.spmm_host_ref_f32(pat.m_vec, V, sweep.N_DENSE, K, pat.row_offsets, pat.column_indices, pat.values,
                                       B, threads=THREADS)
            prob = ops.DeviceProblem(pat, sort=True)
            for kernel in ("wmma", "cuda"):
                out = torch.full((M, sweep.N_DENSE), float("nan"), dtype=torch.float16, device="cuda")
                prob.spmm(Bd, kernel=kernel, out=out)
                assert_parity(out.cpu().numpy(), ref, "spmm M%d K%d s%g V%d %s" % (M, K, s, V, kernel))
                # what the sweep driver's own check says about the same result
                ok, rel = sweep.verify_spmm(pat, B, out.cpu().numpy())
                assert ok and rel <= 1e-2
            hinted = torch.full((M, sweep.N_DENSE), float("nan"), dtype=torch.float16, device="cuda")
            prob.spmm(Bd, out=hinted, row_length_hint=True)     # the sweep's --hint route
            assert_parity(hinted.cpu().numpy(), ref, "spmm M%d K%d s%g V%d hinted" % (M, K, s, V))
            # the schedule that stages the dense operand in LDS per block of eight vector rows (opt-in entry)
            staged = torch.full((M, sweep.N_DENSE), float("nan"), dtype=torch.float16, device="cuda")
            ops.spmm_slab(prob.m_vec, V, sweep.N_DENSE, K, prob.row_indices, prob.row_offsets, prob.column_indices,
                          prob.values, Bd, staged)
            assert_parity(staged.cpu().numpy(), ref, "spmm M%d K%d s%g V%d staged in LDS" % (M, K, s, V))
            points += 1
    assert points == len(sweep.KS) * len(sweep.SPARSITIES)


@pytest.mark.parametrize("V", sweep.VS)
@pytest.mark.parametrize("M", sweep.SDDMM_SIZES)
def test_every_sddmm_point_of_the_grid(gpu, M, V):
    points = 0
    for K in sweep.SDDMM_KS:
        A = cv.dense_normal(M, K, seed=21)
        B = cv.dense_normal(M, K, seed=22)
        Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
        for s in sweep.SPARSITIES:
            pat = sweep.sddmm_grid_pattern(M, s, V)
            ref = co.sddmm_host_ref_f32(pat.m_vec, K, V, pat.row_offsets, pat.column_indices, A, B)
            prob = ops.DeviceProblem(pat, sort=True)
            for kernel in ("wmma", "cuda"):
                out = torch.full((pat.nnz_vec, V), float("nan"), dtype=torch.float16, device="cuda")
                prob.sddmm(Ad, Bd, kernel=kernel, out=out)
                assert_parity(out.cpu().numpy().reshape(-1), ref, "sddmm M%d K%d s%g V%d %s" % (M, K, s, V, kernel))
                ok, rel = sweep.verify_sddmm(pat, A, B, out.cpu().numpy())
                assert ok and rel <= 1e-2
            points += 1
    assert points == len(sweep.SDDMM_KS) * len(sweep.SPARSITIES)

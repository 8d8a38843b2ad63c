"""Split-row SpMM (`vs_wmma_spmm_f16_ws`): the nonzero range is cut into equal runs, one per wave, and rows that
cross run boundaries are added up from fp32 partial tiles (through LDS inside a workgroup, through a workspace
across workgroups).  Same contract as the reference-shaped entry point
(tests/util.py), checked against the CPU oracle through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


def _oracle(pat, B):
    return co.spmm_host_ref_f32(pat.m_vec, pat.vec_length, B.shape[1], pat.n, pat.row_offsets,
                                pat.column_indices, pat.values, B)


def _run(pat, B, out_dtype=torch.float16, workspace="auto", piece=0, waves=0, launches=0, shared=0):
    """One call with canaries round the output and round the workspace; returns the host copy of the output."""
    prob = ops.DeviceProblem(pat)
    Bd = torch.from_numpy(B).cuda()
    k = B.shape[1]
    pad = 64
    buf = torch.full((pat.m + 2 * pad, k), 12345.0, dtype=out_dtype, device="cuda")
    out = buf[pad:pad + pat.m]
    try:
        _lib.set_option("spmm_flat_piece", piece)
        _lib.set_option("spmm_flat_waves", waves)
        _lib.set_option("spmm_flat_launches", launches)
        _lib.set_option("spmm_flat_shared", shared)
        need = ops.spmm_workspace_bytes(pat.m_vec, pat.vec_length, k, pat.n, pat.nnz_vec)
        ws_bytes = need if workspace == "auto" else int(workspace)
        guard = 4096
        ws_buf = torch.full((ws_bytes + 2 * guard,), 0x5A, dtype=torch.uint8, device="cuda")
        ws = ws_buf[guard:guard + ws_bytes] if ws_bytes else None
        if ws is not None:
            ws.zero_()   # the contract: zero before the first use; every call leaves it ready for the next
        for _ in range(2):  # the second call finds the workspace as the first left it
            out.fill_(777.0)
            ops.spmm_split_rows(pat.m_vec, pat.vec_length, k, pat.n, pat.nnz_vec, prob.row_offsets,
                                prob.column_indices, prob.values, Bd, out, ws)
        torch.cuda.synchronize()
    finally:
        _lib.set_option("spmm_flat_piece", 0)
        _lib.set_option("spmm_flat_waves", 0)
        _lib.set_option("spmm_flat_launches", 0)
        _lib.set_option("spmm_flat_shared", 0)
    host = buf.cpu().numpy()
    assert np.all(host[:pad] == 12345.0) and np.all(host[pad + pat.m:] == 12345.0), "wrote outside the output"
    wsh = ws_buf.cpu().numpy()
    assert np.all(wsh[:guard] == 0x5A) and np.all(wsh[guard + ws_bytes:] == 0x5A), "wrote outside the workspace"
    assert np.array_equal(prob.row_offsets.cpu().numpy(), pat.row_offsets)
    assert np.array_equal(prob.column_indices.cpu().numpy(), pat.column_indices)
    return host[pad:pad + pat.m]


def _from_lengths(lengths, n, V, seed):
    rng = np.random.default_rng(seed)
    lengths = np.asarray(lengths, dtype=np.int64)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    return cv.random_values(cv.ColVecCSR(len(lengths), n, V, ro, ci).validate(), seed=seed + 1)


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("piece", [0, 32, 64, 96, 512])
@pytest.mark.parametrize("waves", [0, 1, 3])
@pytest.mark.parametrize("launches", [1, 2])
@pytest.mark.parametrize("shared", [1, 2])
def test_ragged_empty_and_long_rows(gpu, V, piece, waves, launches, shared):
    # empty rows at the start, in the middle and at the end; rows of every tail length; rows that span many runs
    # and pieces; a row that starts exactly on a run boundary (the 64 in front of it ends nonzero 128)
    lengths = [0, 0, 1, 15, 16, 17, 0, 31, 33, 14, 0, 64, 65, 300, 2, 0, 128, 7, 640, 1, 0, 0]
    pat = _from_lengths(lengths, 640, V, seed=5)
    B = cv.dense_uniform(640, 192, seed=7)
    got = _run(pat, B, piece=piece, waves=waves, launches=launches, shared=shared)
    assert_parity(got, _oracle(pat, B),
                  "split rows V%d run %d waves %d launches %d shared %d" % (V, piece, waves, launches, shared))
    for i in np.nonzero(np.asarray(lengths) == 0)[0]:
        assert not got[i * V:(i + 1) * V].any(), "empty vector row %d must be written as zeros" % i


def test_all_rows_empty_and_single_row(gpu):
    pat = cv.ColVecCSR(8, 64, 8, np.zeros(9, np.int32), np.zeros(0, np.int32), np.zeros((0, 8), np.float16))
    B = cv.dense_uniform(64, 64, seed=1)
    got = _run(pat, B)
    assert got.shape == (64, 64) and not got.any()
    one = _from_lengths([2048], 2048, 8, seed=3)   # one dense row: every piece holds a segment of it
    B = cv.dense_uniform(2048, 128, seed=4)
    for waves in (1, 4, 16):
        assert_parity(_run(one, B, piece=64, waves=waves), _oracle(one, B), "single dense row, %d waves" % waves)


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("shared", [1, 2])
def test_many_short_rows_share_steps(gpu, V, shared):
    """Rows of 0 to 40 vectors, more than sixty of them empty in a row (the offsets window of a wave moves on
    several times inside one step), then long rows again: with shared steps up to 16 / V rows meet in one MFMA."""
    rng = np.random.default_rng(70 + V)
    lengths = np.concatenate([rng.integers(0, 41, 300), np.zeros(150, np.int64), [1, 0, 2, 500], np.zeros(70, np.int64),
                              rng.integers(0, 9, 200), [900, 31, 32, 33]]).astype(np.int64)
    pat = _from_lengths(lengths, 1024, V, seed=71)
    B = cv.dense_uniform(1024, 136, seed=72)
    ref = _oracle(pat, B)
    for piece, waves in ((0, 0), (32, 2), (160, 5)):
        got = _run(pat, B, piece=piece, waves=waves, shared=shared)
        assert_parity(got, ref, "short rows V%d run %d waves %d shared %d" % (V, piece, waves, shared))
        for i in np.nonzero(lengths == 0)[0]:
            assert not got[i * V:(i + 1) * V].any(), "empty vector row %d must be written as zeros" % i


@pytest.mark.parametrize("V", [2, 8])
def test_pareto_rows_with_a_dense_row(gpu, V):
    rng = np.random.default_rng(5)
    m_vec, n = 192, 2048
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 40, n).astype(np.int64)
    lengths[7] = n
    lengths[100] = 0
    pat = _from_lengths(lengths, n, V, seed=6)
    B = cv.dense_uniform(n, 256, seed=7)
    ref = _oracle(pat, B)
    a = _run(pat, B)
    assert_parity(a, ref, "pareto rows, automatic pieces")
    b = _run(pat, B)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), "two runs differ"
    c = _run(pat, B, launches=2)
    assert np.array_equal(a.view(np.uint16), c.view(np.uint16)), "one launch and two launches add in the same order"
    assert_parity(_run(pat, B, out_dtype=torch.float32), ref, "pareto rows, fp32 out")


def test_config2_and_smaller_workspaces(gpu):
    pat = cv.random_values(cv.binomial_pattern(64, 4608, 0.9, seed=1, vec_length=8), seed=101)
    B = cv.dense_uniform(4608, 256, seed=201)
    ref = _oracle(pat, B)
    need = ops.spmm_workspace_bytes(pat.m_vec, 8, 256, pat.n, pat.nnz_vec)
    assert need > 0
    for ws in ("auto", need // 2, need // 7, 16384, 0):
        assert_parity(_run(pat, B, workspace=ws), ref, "config 2, workspace %s" % ws)


def test_dense_width_edges(gpu):
    pat = _from_lengths([5, 700, 0, 40, 333, 64], 768, 8, seed=9)
    for N in (4, 8, 24, 64, 72, 136, 512, 1000):
        B = cv.dense_uniform(768, N, seed=N)
        assert_parity(_run(pat, B, piece=64, waves=2), _oracle(pat, B), "N=%d" % N)


def test_device_problem_switch_and_bad_arguments(gpu):
    pat = _from_lengths([900, 3, 3, 3, 0, 50], 1024, 4, seed=11)
    B = cv.dense_uniform(1024, 64, seed=12)
    prob = ops.DeviceProblem(pat, sort=True)
    out = prob.spmm(torch.from_numpy(B).cuda(), split_rows=True)
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy(), _oracle(pat, B), "DeviceProblem(split_rows=True)")
    # split_rows=None: a dense row among short ones is dispatched in parts (its list and their workspace appear),
    # uniform rows are not; both give the oracle's result
    lone = _from_lengths([2048] + [40] * 255, 2048, 8, seed=13)
    Bl = cv.dense_uniform(2048, 128, seed=14)
    p_lone = ops.DeviceProblem(lone)
    got = p_lone.spmm(torch.from_numpy(Bl).cuda(), split_rows=None)
    torch.cuda.synchronize()
    assert p_lone.row_parts(0)[0].n_split == 1 and p_lone.row_parts(0)[2] is not None
    assert_parity(got.cpu().numpy(), _oracle(lone, Bl), "split_rows=None, one dense row")
    even = cv.random_values(cv.uniform_pattern(256, 2048, 0.9, seed=15, vec_length=8), 16)
    p_even = ops.DeviceProblem(even)
    got = p_even.spmm(torch.from_numpy(Bl).cuda(), split_rows=None)
    torch.cuda.synchronize()
    assert p_even.row_parts(0)[0].n_split == 0 and p_even.row_parts(0)[2] is None and p_even._workspace is None
    assert_parity(got.cpu().numpy(), _oracle(even, Bl), "split_rows=None, uniform rows")
    L = _lib.lib()
    args = [pat.m_vec, 4, 64, 1024, pat.nnz_vec, 0, prob.row_offsets.data_ptr(), prob.column_indices.data_ptr(),
            prob.values.data_ptr(), torch.from_numpy(B).cuda().data_ptr(), out.data_ptr()]
    assert L.vs_wmma_spmm_f16_ws(*args, 0, -1, 0) == 1            # negative workspace size
    assert L.vs_wmma_spmm_f16_ws(*args, 0, 4096, 0) == 1          # size without a buffer
    assert L.vs_wmma_spmm_f16_ws(*args, out.data_ptr() + 4, 4096, 0) == 1   # misaligned workspace
    bad = list(args)
    bad[4] = -1
    assert L.vs_wmma_spmm_f16_ws(*bad, 0, 0, 0) == 1              # negative nonzero count


def test_one_workspace_for_problems_of_different_shapes(gpu):
    """The arrival counters sit in an area that depends on the workspace's size alone: a call on a larger problem
    must not find an earlier call's partial tiles where it looks for its counters (nor the other way round)."""
    L = _lib.lib()
    shapes = ((64, 1024, 8, 128, 30, 1000), (768, 4608, 8, 256, 31, 4608), (32, 512, 4, 64, 32, 500),
              (1500, 2048, 1, 192, 33, 2048), (768, 4608, 8, 256, 34, 3000))
    ws_bytes = 24 << 20
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device="cuda")   # zeroed once, before the first use
    for (m_vec, n, V, N, seed, longest) in shapes:
        rng = np.random.default_rng(seed)
        lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 60, n).astype(np.int64)
        lengths[m_vec // 3] = longest
        pat = _from_lengths(lengths, n, V, seed=seed)
        B = cv.dense_uniform(n, N, seed=seed + 1)
        prob = ops.DeviceProblem(pat)
        out = torch.full((pat.m, N), 55.0, dtype=torch.float16, device="cuda")
        st = L.vs_wmma_spmm_f16_ws(m_vec, V, N, n, pat.nnz_vec, 0, prob.row_offsets.data_ptr(),
                                   prob.column_indices.data_ptr(), prob.values.data_ptr(),
                                   torch.from_numpy(B).cuda().data_ptr(), out.data_ptr(), ws.data_ptr(), ws_bytes, 0)
        assert st == 0, L.vs_status_string(st)
        torch.cuda.synchronize()
        assert_parity(out.cpu().numpy(), _oracle(pat, B), "shared workspace, %d rows V%d N%d" % (m_vec, V, N))

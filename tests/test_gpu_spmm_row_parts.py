"""SpMM with long rows dispatched in parts (`vs_spmm_row_parts` + `vs_wmma_spmm_f16_row_parts`): the list names
parts of rows, each served by a workgroup of its own; the parts of a split row meet as fp32 partial tiles in a
workspace and the workgroup that arrives last adds them up.  Same contract as the reference-shaped entry point
(tests/util.py), checked against the CPU oracle through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity, retired_variants_built

pytestmark = pytest.mark.gpu


def _oracle(pat, B):
    return co.spmm_host_ref_f32(pat.m_vec, pat.vec_length, B.shape[1], pat.n, pat.row_offsets,
                                pat.column_indices, pat.values, B)


def _from_lengths(lengths, n, V, seed):
    rng = np.random.default_rng(seed)
    lengths = np.asarray(lengths, dtype=np.int64)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    return cv.random_values(cv.ColVecCSR(len(lengths), n, V, ro, ci).validate(), seed=seed + 1)


def _run(pat, B, limit=0, calls=2, options=None):
    """`calls` calls in a row on one workspace, canaries round the output and the workspace; the host copy of the
    output and the dispatch list."""
    parts = ops.RowParts(pat.m_vec, pat.row_offsets, limit)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, ci, vals, Bd = d(parts.slots), d(pat.column_indices), d(pat.values), d(B)
    k = B.shape[1]
    pad = 64
    buf = torch.full((pat.m + 2 * pad, k), 12345.0, dtype=torch.float16, device="cuda")
    out = buf[pad:pad + pat.m]
    need = ops.spmm_row_parts_workspace_bytes(pat.vec_length, k, parts.n_split, parts.parts_max)
    assert (need > 0) == (parts.n_split > 0)
    guard = 4096
    ws_buf = torch.full((need + 2 * guard,), 0x5A, dtype=torch.uint8, device="cuda")
    ws = ws_buf[guard:guard + need] if need else None
    if ws is not None:
        ws.zero_()   # the contract: zero before the first use; every call leaves it ready for the next
    with _lib.thread_options(**(options or {})):
        for _ in range(calls):
            out.fill_(777.0)
            ops.spmm_row_parts(pat.vec_length, k, pat.n, parts, slots, pat.nnz_vec, ci, vals, Bd, out, ws)
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert np.all(host[:pad] == 12345.0) and np.all(host[pad + pat.m:] == 12345.0), "wrote outside the output"
    wsh = ws_buf.cpu().numpy()
    assert np.all(wsh[:guard] == 0x5A) and np.all(wsh[guard + need:] == 0x5A), "wrote outside the workspace"
    if need:
        counters = wsh[guard:guard + need // 128 // 256 * 256]
        assert not counters.any(), "the arrival counters must be back at zero"
    assert np.array_equal(ci.cpu().numpy(), pat.column_indices)
    assert np.array_equal(slots.cpu().numpy(), parts.slots)
    return host[pad:pad + pat.m], parts


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("limit", [64, 128, 320, 0])
@pytest.mark.parametrize("N", [64, 136, 256])
@pytest.mark.parametrize("launches", [1, 2])
def test_ragged_empty_and_long_rows(gpu, V, limit, N, launches):
    # empty rows at the start, in the middle and at the end; rows of every tail length; rows just under, at and
    # over the limits; rows of many parts
    lengths = [0, 0, 1, 15, 16, 17, 0, 31, 33, 63, 64, 65, 127, 128, 129, 300, 2, 0, 320, 321, 640, 1, 1024, 0, 0]
    pat = _from_lengths(lengths, 1024, V, seed=5)
    B = cv.dense_uniform(1024, N, seed=7)
    got, parts = _run(pat, B, limit=limit, options={"spmm_parts_launches": launches})
    assert parts.n_split > 0 or limit == 0   # (the default limit is beyond these rows)
    assert_parity(got, _oracle(pat, B), "row parts V%d limit %d N%d, %d launches" % (V, limit, N, launches))
    for i in np.nonzero(np.asarray(lengths) == 0)[0]:
        assert not got[i * V:(i + 1) * V].any(), "empty vector row %d must be written as zeros" % i


@pytest.mark.parametrize("V", [2, 8])
def test_pareto_rows_with_dense_rows_on_every_launch_shape(gpu, V):
    rng = np.random.default_rng(5)
    m_vec, n = 300, 4608
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 80, n).astype(np.int64)
    lengths[7] = n
    lengths[150] = n
    lengths[100] = 0
    pat = _from_lengths(lengths, n, V, seed=6)
    B = cv.dense_uniform(n, 256, seed=7)
    ref = _oracle(pat, B)
    a, parts = _run(pat, B)
    assert parts.parts_max == 4 and parts.longest_part_vec == 1152
    assert_parity(a, ref, "pareto rows, default limit")
    b, _ = _run(pat, B)
    assert np.array_equal(a.view(np.uint16), b.view(np.uint16)), "two runs differ"
    one, _ = _run(pat, B, options={"spmm_parts_launches": 1})
    two, _ = _run(pat, B, options={"spmm_parts_launches": 2})
    assert np.array_equal(one.view(np.uint16), two.view(np.uint16)), "one launch and two launches add in the same order"
    # one block per wave, several blocks per wave one after the other and pipelined, both tile widths, one wave
    for opts in ({"spmm_pipe": 1}, {"spmm_pipe": 2}, {"spmm_waves": 1, "spmm_pipe": 2}, {"spmm_waves": 2},
                 {"spmm_cols_per_lane": 4}, {"spmm_cols_per_lane": 8, "spmm_waves": 3},
                 {"spmm_blocks_per_wave": 2, "spmm_pipe": 2}, {"spmm_steps": 1},
                 {"spmm_steps": 4 if retired_variants_built() else 2},
                 {"spmm_parts_launches": 1, "spmm_waves": 1}, {"spmm_parts_launches": 2, "spmm_waves": 1}):
        for limit in (0, 512):
            got, _ = _run(pat, B, limit=limit, calls=1, options=opts)
            assert_parity(got, ref, "pareto rows, limit %d, %s" % (limit, opts))


def test_no_row_split_and_all_rows_empty(gpu):
    pat = cv.random_values(cv.uniform_pattern(64, 512, 0.9, seed=3, vec_length=8), 4)
    B = cv.dense_uniform(512, 128, seed=5)
    got, parts = _run(pat, B)
    assert parts.n_split == 0 and parts.parts_max == 0 and parts.n_slots == 64
    assert_parity(got, _oracle(pat, B), "no row over the limit")
    empty = cv.ColVecCSR(8, 64, 8, np.zeros(9, np.int32), np.zeros(0, np.int32), np.zeros((0, 8), np.float16))
    got, parts = _run(empty, cv.dense_uniform(64, 64, seed=1))
    assert parts.n_slots == 8 and not got.any()


def test_dense_width_edges_and_rejections(gpu):
    pat = _from_lengths([5, 700, 0, 40, 333, 64], 768, 8, seed=9)
    for N in (4, 8, 24, 72, 512, 1000):
        B = cv.dense_uniform(768, N, seed=N)
        got, _ = _run(pat, B, limit=128)
        assert_parity(got, _oracle(pat, B), "N=%d" % N)
    L = _lib.lib()
    parts = ops.RowParts(pat.m_vec, pat.row_offsets, 128)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, ci, vals = d(parts.slots), d(pat.column_indices), d(pat.values)
    B = d(cv.dense_uniform(768, 64, seed=1))
    out = torch.full((pat.m, 64), 9.0, dtype=torch.float16, device="cuda")
    need = ops.spmm_row_parts_workspace_bytes(8, 64, parts.n_split, parts.parts_max)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    args = lambda k, ws_bytes: (1, 8, k, 768, parts.n_slots, slots.data_ptr(), parts.n_split, parts.parts_max, pat.nnz_vec,
                                parts.longest_part_vec, ci.data_ptr(), vals.data_ptr(), 0, B.data_ptr(), 0, out.data_ptr(), 0,
                                ws.data_ptr(), ws_bytes, 0)
    assert L.vs_wmma_spmm_f16_row_parts(*args(62, need)) == 801       # dense width not a multiple of 4
    assert L.vs_wmma_spmm_f16_row_parts(*args(64, need - 16)) == 801  # workspace too small
    assert L.vs_wmma_spmm_f16_row_parts(*args(64, -1)) == 1
    bad = list(args(64, need))
    bad[5] = slots.data_ptr() + 4
    assert L.vs_wmma_spmm_f16_row_parts(*bad) == 1                    # misaligned list
    torch.cuda.synchronize()
    assert bool((out == 9.0).all()), "a rejected call must not launch anything"


def test_one_workspace_for_problems_of_different_shapes(gpu):
    L = _lib.lib()
    shapes = ((64, 1024, 8, 128, 30, 1000), (512, 4608, 8, 256, 31, 4608), (32, 512, 4, 64, 32, 500),
              (700, 2048, 1, 192, 33, 2048), (512, 4608, 8, 256, 34, 3000))
    ws_bytes = 24 << 20
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device="cuda")   # zeroed once, before the first use
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    for (m_vec, n, V, N, seed, longest) in shapes:
        rng = np.random.default_rng(seed)
        lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 60, n).astype(np.int64)
        lengths[m_vec // 3] = longest
        pat = _from_lengths(lengths, n, V, seed=seed)
        B = cv.dense_uniform(n, N, seed=seed + 1)
        parts = ops.RowParts(m_vec, pat.row_offsets, 256)
        assert ops.spmm_row_parts_workspace_bytes(V, N, parts.n_split, parts.parts_max) <= ws_bytes
        out = torch.full((pat.m, N), 55.0, dtype=torch.float16, device="cuda")
        ops.spmm_row_parts(V, N, n, parts, d(parts.slots), pat.nnz_vec, d(pat.column_indices), d(pat.values), d(B), out, ws)
        torch.cuda.synchronize()
        assert_parity(out.cpu().numpy(), _oracle(pat, B), "shared workspace, %d rows V%d N%d" % (m_vec, V, N))


def test_device_problem_entry(gpu):
    pat = _from_lengths([2048] + [40] * 255, 2048, 8, seed=13)
    B = cv.dense_uniform(2048, 128, seed=14)
    prob = ops.DeviceProblem(pat)
    Bd = torch.from_numpy(B).cuda()
    out = prob.spmm_row_parts(Bd)
    out2 = prob.spmm_row_parts(Bd, limit_vec=1024)
    torch.cuda.synchronize()
    ref = _oracle(pat, B)
    assert_parity(out.cpu().numpy(), ref, "DeviceProblem.spmm_row_parts")
    assert_parity(out2.cpu().numpy(), ref, "DeviceProblem.spmm_row_parts(limit_vec=1024)")


@pytest.mark.parametrize("seed", range(40))
def test_random_patterns_limits_and_options(gpu, seed):
    """Random row-length distributions, vector lengths, dense widths, limits and launch shapes against the oracle."""
    rng = np.random.default_rng(7000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    m_vec = int(rng.integers(1, 120))
    n = int(rng.integers(64, 3000))
    kind = seed % 4
    if kind == 0:      # heavy tail
        lengths = np.minimum((rng.pareto(1.1, m_vec) + 0.05) * n * 0.1, n)
    elif kind == 1:    # a few dense rows among short and empty ones
        lengths = np.where(rng.random(m_vec) < 0.1, n, rng.integers(0, 20, m_vec))
    elif kind == 2:    # uniform density
        lengths = rng.binomial(n, rng.uniform(0.05, 0.9), size=m_vec)
    else:              # every row dense
        lengths = np.full(m_vec, n)
    pat = _from_lengths(lengths.astype(np.int64), n, V, seed=seed)
    N = int(rng.choice([4, 8, 12, 40, 64, 100, 128, 200, 256, 264, 388]))
    B = cv.dense_uniform(n, N, seed=seed + 1)
    limit = int(rng.choice([0, 1, 64, 65, 200, 512, 1000]))
    opts = {"spmm_parts_launches": int(rng.integers(0, 3))}
    if rng.random() < 0.5:
        opts["spmm_waves"] = int(rng.choice([1, 2, 3, 4, 8]))
    if rng.random() < 0.5:
        opts["spmm_pipe"] = int(rng.integers(1, 3))
    if rng.random() < 0.3:
        opts["spmm_cols_per_lane"] = int(rng.choice([4, 8]))
    if rng.random() < 0.3:
        opts["spmm_blocks_per_wave"] = int(rng.choice([1, 2, 4]))
    what = "seed %d V%d m_vec%d n%d N%d nnz_vec%d limit %d %s" % (seed, V, m_vec, n, N, pat.nnz_vec, limit, opts)
    print(what, flush=True)
    got, parts = _run(pat, B, limit=limit, options=opts)
    assert_parity(got, _oracle(pat, B), what)
    for i in np.nonzero(np.diff(pat.row_offsets) == 0)[0]:
        assert not got[i * V:(i + 1) * V].any(), "empty vector row %d must be written as zeros" % i


def test_hip_graph_replays_equal_eager(gpu):
    """The entry point is capturable (no allocation, no memset, no synchronisation inside) and every replay finds the
    arrival counters as the one before left them: replays with fresh operands in between equal the eager result."""
    rng = np.random.default_rng(3)
    lengths = np.minimum((rng.pareto(1.5, 400) + 0.3) * 100, 3000).astype(np.int64)
    pat = _from_lengths(lengths, 3000, 8, seed=4)
    prob = ops.DeviceProblem(pat)
    assert prob.row_parts(0)[0].n_split > 0
    g = torch.Generator(device="cuda").manual_seed(5)
    Bd = torch.randn((3000, 128), device="cuda", generator=g).half()
    out = torch.empty((pat.m, 128), dtype=torch.float16, device="cuda")
    for launches in (1, 2):
        with _lib.thread_options(spmm_parts_launches=launches):
            prob.spmm_row_parts(Bd, out=out)
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                prob.spmm_row_parts(Bd, out=out)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                prob.spmm_row_parts(Bd, out=out)
            for rep in range(4):
                Bd.copy_(torch.randn(Bd.shape, device="cuda", generator=g).half())   # new operand, same buffer
                prob.spmm_row_parts(Bd, out=out)
                torch.cuda.synchronize()
                want = out.clone()
                out.zero_()
                torch.cuda.synchronize()
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(out, want), "replay %d, %d launch(es)" % (rep, launches)
    assert_parity(out.cpu().numpy(), _oracle(pat, Bd.cpu().numpy()), "rows in parts under a HIP graph")


@pytest.mark.parametrize("V", [2, 8])
@pytest.mark.parametrize("launches", [1, 2])
def test_batch_on_a_shared_pattern(gpu, V, launches):
    """Five problems on one pattern and one list: per-problem values and dense operands, then a shared dense
    operand; each agrees with the oracle and with the single call on its operands."""
    rng = np.random.default_rng(21)
    lengths = np.minimum((rng.pareto(1.4, 90) + 0.2) * 60, 1500).astype(np.int64)
    lengths[3] = 1500
    base = _from_lengths(lengths, 1500, V, seed=22)
    batch, N = 5, 136
    vals = np.stack([cv.random_values(base, seed=30 + b).values for b in range(batch)])
    Bs = np.stack([cv.dense_uniform(1500, N, seed=40 + b) for b in range(batch)])
    parts = ops.RowParts(base.m_vec, base.row_offsets, 128)
    assert parts.n_split > 0
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, ci, vd, Bd = d(parts.slots), d(base.column_indices), d(vals), d(Bs)
    need = ops.spmm_row_parts_workspace_bytes(V, N, parts.n_split, parts.parts_max, batch=batch)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    with _lib.thread_options(spmm_parts_launches=launches):
        out = torch.full((batch, base.m, N), 3.0, dtype=torch.float16, device="cuda")
        for _ in range(2):
            ops.spmm_row_parts(V, N, 1500, parts, slots, base.nnz_vec, ci, vd, Bd, out, ws)
        shared = torch.full((batch, base.m, N), 3.0, dtype=torch.float16, device="cuda")
        ops.spmm_row_parts(V, N, 1500, parts, slots, base.nnz_vec, ci, vd, Bd[0], shared, ws)
        torch.cuda.synchronize()
        for b in range(batch):
            pat = base.with_values(vals[b])
            assert_parity(out[b].cpu().numpy(), _oracle(pat, Bs[b]), "batched, problem %d" % b)
            assert_parity(shared[b].cpu().numpy(), _oracle(pat, Bs[0]), "batched, shared dense operand, problem %d" % b)
            single = torch.empty((base.m, N), dtype=torch.float16, device="cuda")
            ws1 = torch.zeros(need, dtype=torch.uint8, device="cuda")
            ops.spmm_row_parts(V, N, 1500, parts, slots, base.nnz_vec, ci, vd[b], Bd[b], single, ws1)
            torch.cuda.synchronize()
            # (not bit for bit: how a row's blocks are shared among waves follows the size of the launch)
            assert_parity(out[b].cpu().numpy(), single.float().cpu().numpy(), "batched against single, problem %d" % b)
    assert not ws.cpu().numpy()[:need // 5 // 256 * 256].any(), "the arrival counters must be back at zero"


def test_batch_of_one_ignores_the_leading_stride(gpu):
    """[1, ...] operands whose leading stride is no multiple of 16 bytes (n * k odd multiples of 4 halves): a batch of
    one passes no per-problem stride, so the alignment rule for strides does not apply; all three operators."""
    V, n, N = 4, 333, 12
    lengths = [333, 5, 0, 200, 17, 333, 1]
    pat = _from_lengths(lengths, n, V, seed=61)
    B = cv.dense_uniform(n, N, seed=62)
    parts = ops.RowParts(pat.m_vec, pat.row_offsets, 64)
    assert parts.n_split > 0 and (n * N) % 8 != 0
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, ci = d(parts.slots), d(pat.column_indices)
    ws = torch.zeros(ops.spmm_row_parts_workspace_bytes(V, N, parts.n_split, parts.parts_max), dtype=torch.uint8,
                     device="cuda")
    out = torch.empty((1, pat.m, N), dtype=torch.float16, device="cuda")
    ops.spmm_row_parts(V, N, n, parts, slots, pat.nnz_vec, ci, d(pat.values[None]), d(B[None]), out, ws)
    torch.cuda.synchronize()
    assert_parity(out[0].cpu().numpy(), _oracle(pat, B), "batch of one, [1, n, k] operands")

    scores = d(pat.values[None]).clone()
    sm_ws = torch.empty(max(8, ops.sparse_softmax_row_parts_workspace_bytes(V, parts.n_split, parts.parts_max)),
                        dtype=torch.uint8, device="cuda")
    ops.sparse_softmax_row_parts(V, parts, slots, scores, scale=0.5, workspace=sm_ws)
    torch.cuda.synchronize()
    from oracle import numpy_oracle as no
    assert_parity(scores[0].cpu().numpy(), no.sparse_softmax_ref(pat.m_vec, V, pat.row_offsets, pat.values, 0.5),
                  "softmax, batch of one")


def test_more_long_rows_than_split_rows_can_be_numbered(gpu):
    """33000 rows of 128 vectors at a limit of 64: 32767 rows run as two halves, the others whole, in one list and
    one launch; one and two launches agree bit for bit and with the oracle."""
    V, m_vec, n, N = 1, 33000, 256, 8
    pat = _from_lengths(np.full(m_vec, 128), n, V, seed=71)
    B = cv.dense_uniform(n, N, seed=72)
    ref = _oracle(pat, B)
    one, parts = _run(pat, B, limit=64, options={"spmm_parts_launches": 1})
    assert parts.n_split == 32767 and parts.n_slots == m_vec + 32767
    assert_parity(one, ref, "32767 split rows and 233 whole ones")
    two, _ = _run(pat, B, limit=64, options={"spmm_parts_launches": 2})
    assert np.array_equal(one, two)

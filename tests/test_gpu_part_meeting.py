"""The meeting of partial tiles across workgroups (rows in parts; the split-row schedule of the entry point that
allocates nothing) under load: one captured graph holding both operators is replayed 500 times while a second stream
keeps the memory system busy with large copies; every replay must give the bits of the first, and the arrival counters
of the caller-owned workspace must be back at zero.  The loop stops at the first mismatch."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu

REPLAYS = 500


def test_replays_under_a_competing_stream_keep_their_bits(gpu):
    L = _lib.lib()
    rng = np.random.default_rng(7)
    m_vec, n, N, V = 512, 4608, 256, 8
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 150, n).astype(np.int64)
    lengths[5] = n          # a dense row: many parts, many pieces
    ro, ci = cv._pattern_from_lengths(rng, m_vec, n, lengths)
    pat = cv.random_values(cv.ColVecCSR(m_vec, n, V, ro, ci).validate(), seed=8)
    B = cv.dense_uniform(n, N, seed=9)
    prob = ops.DeviceProblem(pat, sort=True)
    Bd = torch.from_numpy(B).cuda()
    out_parts = torch.empty((pat.m, N), dtype=torch.float16, device="cuda")
    out_noalloc = torch.empty((pat.m, N), dtype=torch.float16, device="cuda")
    assert L.vs_wmma_spmm_noalloc_scratch_bytes() > 0      # (the symbol lookup, outside the capture)

    def both(stream):
        with _lib.thread_options(spmm_parts_launches=1):   # the parts meet inside the launch
            prob.spmm_row_parts(Bd, out=out_parts, stream=stream, limit_vec=512)
        st = L.vs_wmma_spmm_f16_noalloc(m_vec, V, N, n, pat.nnz_vec, 0, prob.row_offsets.data_ptr(),
                                        prob.column_indices.data_ptr(), prob.values.data_ptr(), Bd.data_ptr(),
                                        out_noalloc.data_ptr(), stream.cuda_stream)
        assert st == 0, L.vs_status_string(st)

    work = torch.cuda.Stream()
    with torch.cuda.stream(work):
        both(work)                                          # eager: allocates the object's workspace, warms up
    work.synchronize()
    parts, _, workspace, _ = prob.row_parts(512)
    assert parts.n_split > 10 and workspace is not None
    ref = co.spmm_host_ref_f32(m_vec, V, N, n, pat.row_offsets, pat.column_indices, pat.values, B)
    assert_parity(out_parts.cpu().numpy(), ref, "rows in parts")
    assert_parity(out_noalloc.cpu().numpy(), ref, "no-alloc split rows")

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=work):
        both(work)
    first_parts = first_noalloc = None
    noise = torch.cuda.Stream()
    big_a = torch.empty(64 << 20, dtype=torch.float32, device="cuda")   # 256 MiB each: past the Infinity Cache
    big_b = torch.empty_like(big_a)
    for replay in range(REPLAYS):
        with torch.cuda.stream(noise):
            big_b.copy_(big_a, non_blocking=True)
            big_a.copy_(big_b, non_blocking=True)
        with torch.cuda.stream(work):
            out_parts.fill_(-1.0)
            out_noalloc.fill_(-1.0)
            graph.replay()
        work.synchronize()
        if replay == 0:
            first_parts, first_noalloc = out_parts.clone(), out_noalloc.clone()
            assert_parity(first_parts.cpu().numpy(), ref, "rows in parts, first replay")
            assert_parity(first_noalloc.cpu().numpy(), ref, "no-alloc split rows, first replay")
            continue
        assert torch.equal(out_parts, first_parts), "rows in parts: replay %d differs from the first" % replay
        assert torch.equal(out_noalloc, first_noalloc), "no-alloc split rows: replay %d differs from the first" % replay
    noise.synchronize()
    # the counters' area of the workspace (a fifth of it, whatever the problem) is back at zero
    counter_bytes = (workspace.numel() // 5 + 255) // 256 * 256
    assert not bool(workspace[:counter_bytes].any()), "an arrival counter was left behind"

"""`vs_wmma_spmm_f16_noalloc`: the split-row SpMM with its workspace in a static device array of the library.
Through the C ABI, against `vs_wmma_spmm_f16_ws` with a caller workspace of the same size (bit for bit) and
against the CPU oracle; calls in a row on problems of different shapes - a smaller one, then larger ones with more
arrival counters than any call before - so that whatever a call left in the array must not leak into the next."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


def _problem(m_vec, n, V, N, seed, longest):
    rng = np.random.default_rng(seed)
    lengths = np.minimum((rng.pareto(1.5, m_vec) + 0.3) * 60, n).astype(np.int64)
    lengths[m_vec // 3] = longest      # a row that spans many pieces
    lengths[m_vec // 2] = 0
    ro, ci = cv._pattern_from_lengths(rng, m_vec, n, lengths)
    pat = cv.random_values(cv.ColVecCSR(m_vec, n, V, ro, ci).validate(), seed=seed + 1)
    return pat, cv.dense_uniform(n, N, seed=seed + 2)


def _device(pat, B):
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return d(pat.row_offsets), d(pat.column_indices), d(pat.values), d(B)


def test_two_calls_in_a_row_match_the_workspace_entry_point(gpu):
    L = _lib.lib()
    scratch = L.vs_wmma_spmm_noalloc_scratch_bytes()
    assert scratch == 16 << 20
    workspace = torch.zeros(scratch, dtype=torch.uint8, device="cuda")
    # the first problem splits many rows across pieces; the second is smaller in every dimension; the third and
    # fourth have more pieces and other tile shapes than any before them (their arrival counters lie where an
    # earlier call's would have put partial tiles, if the layout followed the problem instead of the array)
    for (m_vec, n, V, N, seed, longest) in ((512, 4096, 8, 256, 1, 4096), (96, 1024, 8, 128, 2, 1000),
                                            (1024, 4608, 8, 256, 5, 4608), (2048, 2048, 2, 64, 6, 2048)):
        pat, B = _problem(m_vec, n, V, N, seed, longest)
        ro, ci, vals, Bd = _device(pat, B)
        assert L.vs_wmma_spmm_workspace_bytes(m_vec, V, N, n, pat.nnz_vec) > 0, "the case must use the scratch"
        pad = 64
        buf = torch.full((pat.m + 2 * pad, N), 4321.0, dtype=torch.float16, device="cuda")
        got = buf[pad:pad + pat.m]
        want = torch.full((pat.m, N), -1.0, dtype=torch.float16, device="cuda")
        st = L.vs_wmma_spmm_f16_noalloc(m_vec, V, N, n, pat.nnz_vec, 0, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                        Bd.data_ptr(), got.data_ptr(), 0)
        assert st == 0, L.vs_status_string(st)
        st = L.vs_wmma_spmm_f16_ws(m_vec, V, N, n, pat.nnz_vec, 0, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                   Bd.data_ptr(), want.data_ptr(), workspace.data_ptr(), scratch, 0)
        assert st == 0, L.vs_status_string(st)
        torch.cuda.synchronize()
        host = buf.cpu().numpy()
        assert np.all(host[:pad] == 4321.0) and np.all(host[pad + pat.m:] == 4321.0), "wrote outside the output"
        assert np.array_equal(host[pad:pad + pat.m].view(np.uint16), want.cpu().numpy().view(np.uint16)), \
            "static scratch and caller workspace give different bits"
        ref = co.spmm_host_ref_f32(m_vec, V, N, n, pat.row_offsets, pat.column_indices, pat.values, B)
        assert_parity(host[pad:pad + pat.m], ref, "no-alloc entry point, %d rows" % m_vec)
        assert np.array_equal(ro.cpu().numpy(), pat.row_offsets) and np.array_equal(ci.cpu().numpy(), pat.column_indices)


def test_sizes_beyond_the_scratch_are_rejected(gpu):
    L = _lib.lib()
    pat, B = _problem(16, 256, 8, 4224, 3, 200)      # 8 * 4224 > 32768
    ro, ci, vals, Bd = _device(pat, B)
    out = torch.full((pat.m, 4224), 9.0, dtype=torch.float16, device="cuda")
    st = L.vs_wmma_spmm_f16_noalloc(16, 8, 4224, 256, pat.nnz_vec, 0, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                    Bd.data_ptr(), out.data_ptr(), 0)
    assert st == 801 and b"limit" in L.vs_status_string(st)
    torch.cuda.synchronize()
    assert bool((out == 9.0).all()), "a rejected call must not launch anything"
    # at the limit it runs
    pat, B = _problem(16, 256, 8, 4096, 4, 200)
    ro, ci, vals, Bd = _device(pat, B)
    out = torch.empty((pat.m, 4096), dtype=torch.float16, device="cuda")
    st = L.vs_wmma_spmm_f16_noalloc(16, 8, 4096, 256, pat.nnz_vec, 0, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                    Bd.data_ptr(), out.data_ptr(), 0)
    assert st == 0
    torch.cuda.synchronize()
    ref = co.spmm_host_ref_f32(16, 8, 4096, 256, pat.row_offsets, pat.column_indices, pat.values, B)
    assert_parity(out.cpu().numpy(), ref, "no-alloc entry point at its size limit")


def test_captured_into_a_graph_and_replayed(gpu):
    """The call under HIP graph capture (the callers it exists for): the symbol lookup is made before the capture
    by asking for the scratch size; every replay - with eager calls of the same entry point on other shapes and
    synchronisations in between - gives the bits of the eager call."""
    L = _lib.lib()
    assert L.vs_wmma_spmm_noalloc_scratch_bytes() == 16 << 20   # resolves this device's array outside the capture
    pat, B = _problem(256, 2048, 8, 128, 11, 2048)
    ro, ci, vals, Bd = _device(pat, B)
    other, oB = _problem(64, 1024, 4, 64, 12, 1024)
    oro, oci, ovals, oBd = _device(other, oB)
    oout = torch.empty((other.m, 64), dtype=torch.float16, device="cuda")
    eager = torch.empty((pat.m, 128), dtype=torch.float16, device="cuda")
    st = L.vs_wmma_spmm_f16_noalloc(256, 8, 128, 2048, pat.nnz_vec, 0, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                    Bd.data_ptr(), eager.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    want = eager.cpu().numpy().view(np.uint16)
    out = torch.empty_like(eager)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        st = L.vs_wmma_spmm_f16_noalloc(256, 8, 128, 2048, pat.nnz_vec, 0, ro.data_ptr(), ci.data_ptr(), vals.data_ptr(),
                                        Bd.data_ptr(), out.data_ptr(), side.cuda_stream)
    assert st == 0
    for replay in range(6):
        out.fill_(-3.0)
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint16), want), "replay %d differs from the eager call" % replay
        st = L.vs_wmma_spmm_f16_noalloc(64, 4, 64, 1024, other.nnz_vec, 0, oro.data_ptr(), oci.data_ptr(),
                                        ovals.data_ptr(), oBd.data_ptr(), oout.data_ptr(),
                                        torch.cuda.current_stream().cuda_stream)
        assert st == 0
        torch.cuda.synchronize()
    ref = co.spmm_host_ref_f32(256, 8, 128, 2048, pat.row_offsets, pat.column_indices, pat.values, B)
    assert_parity(out.cpu().numpy(), ref, "no-alloc entry point, replayed")


def test_counters_recover_from_an_inconsistent_call_and_reset(gpu):
    """A call whose nonzeros_vec is smaller than row_offsets[m_vec] computes (and counts) only the parts that exist,
    so the arrival counters are back at zero for the next call; vs_wmma_spmm_noalloc_reset clears them in any case."""
    L = _lib.lib()
    pat, B = _problem(256, 4096, 8, 256, 21, 4096)
    ro, ci, vals, Bd = _device(pat, B)
    out = torch.empty((pat.m, 256), dtype=torch.float16, device="cuda")
    args = (ro.data_ptr(), ci.data_ptr(), vals.data_ptr(), Bd.data_ptr(), out.data_ptr(), 0)
    ref = co.spmm_host_ref_f32(256, 8, 256, 4096, pat.row_offsets, pat.column_indices, pat.values, B)
    # cut inside the long row that spans many pieces (results of this call are undefined; only its side effects count)
    cut = int(pat.row_offsets[256 // 3] + 1500)
    assert cut < pat.nnz_vec
    assert L.vs_wmma_spmm_f16_noalloc(256, 8, 256, 4096, cut, 0, *args) == 0
    torch.cuda.synchronize()
    assert L.vs_wmma_spmm_f16_noalloc(256, 8, 256, 4096, pat.nnz_vec, 0, *args) == 0
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy(), ref, "the call after an inconsistent one")
    assert L.vs_wmma_spmm_noalloc_reset(0) == 0
    out.fill_(0)
    assert L.vs_wmma_spmm_f16_noalloc(256, 8, 256, 4096, pat.nnz_vec, 0, *args) == 0
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy(), ref, "the call after a reset")

"""SDDMM driven by a dispatch list of row parts (`vs_spmm_row_parts` + `vs_wmma_sddmm_f16_row_parts`): rows far
longer than the rest are served as several slots.  Same contract as the reference-shaped entry point (tests/util.py),
checked against the CPU oracle through the C ABI; the operator has no sum across parts, so the bits equal those of
the row kernel."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from vectorsparse_amd import _lib, ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


def _mask(lengths, n, V, seed):
    rng = np.random.default_rng(seed)
    lengths = np.asarray(lengths, dtype=np.int64)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    return cv.ColVecCSR(len(lengths), n, V, ro, ci).validate()


def _oracle(mask, A, B):
    return co.sddmm_host_ref_f16(mask.m_vec, A.shape[1], mask.vec_length, mask.row_offsets, mask.column_indices, A, B)


def _run(mask, A, B, limit):
    parts = ops.RowParts(mask.m_vec, mask.row_offsets, limit)
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, ci, Ad, Bd = d(parts.slots), d(mask.column_indices), d(A), d(B)
    pad = 64
    buf = torch.full((mask.nnz_vec + 2 * pad, mask.vec_length), 4321.0, dtype=torch.float16, device="cuda")
    out = buf[pad:pad + mask.nnz_vec]
    ops.sddmm_row_parts(A.shape[1], mask.n, parts, slots, mask.nnz_vec, ci, Ad, Bd, out, mask.vec_length)
    torch.cuda.synchronize()
    host = buf.cpu().numpy()
    assert np.all(host[:pad] == 4321.0) and np.all(host[pad + mask.nnz_vec:] == 4321.0), "wrote outside the output"
    assert np.array_equal(ci.cpu().numpy(), mask.column_indices) and np.array_equal(slots.cpu().numpy(), parts.slots)
    return host[pad:pad + mask.nnz_vec], parts


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("K", [8, 32, 64, 72, 128, 256, 320])
@pytest.mark.parametrize("limit", [64, 200, 0])
def test_ragged_empty_and_long_rows(gpu, V, K, limit):
    lengths = [0, 0, 1, 15, 16, 17, 0, 31, 33, 63, 64, 65, 127, 128, 129, 300, 2, 0, 320, 321, 640, 1, 1500, 0, 0]
    mask = _mask(lengths, 1536, V, seed=5)
    A = cv.dense_normal(mask.m, K, seed=6)
    B = cv.dense_normal(1536, K, seed=7)
    got, parts = _run(mask, A, B, limit)
    assert parts.n_split > 0
    assert_parity(got.reshape(-1), np.asarray(_oracle(mask, A, B)).reshape(-1), "V%d K%d limit %d" % (V, K, limit))


@pytest.mark.parametrize("seed", range(30))
def test_random_masks_equal_the_row_kernel_bit_for_bit(gpu, seed):
    rng = np.random.default_rng(9000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    m_vec = int(rng.integers(1, 150))
    n = int(rng.integers(64, 3000))
    if seed % 3 == 0:
        lengths = np.minimum((rng.pareto(1.1, m_vec) + 0.05) * n * 0.1, n)
    elif seed % 3 == 1:
        lengths = np.where(rng.random(m_vec) < 0.1, n, rng.integers(0, 20, m_vec))
    else:
        lengths = rng.binomial(n, rng.uniform(0.05, 0.9), size=m_vec)
    mask = _mask(lengths.astype(np.int64), n, V, seed=seed)
    K = int(rng.choice([8, 16, 40, 64, 96, 128, 200, 256, 264, 512]))
    A = cv.dense_normal(mask.m, K, seed=seed + 1)
    B = cv.dense_normal(n, K, seed=seed + 2)
    limit = int(rng.choice([0, 1, 64, 65, 200, 512, 1000]))
    what = "seed %d V%d m_vec%d n%d K%d nnz_vec%d limit %d" % (seed, V, m_vec, n, K, mask.nnz_vec, limit)
    print(what, flush=True)
    got, _ = _run(mask, A, B, limit)
    assert_parity(got.reshape(-1), np.asarray(_oracle(mask, A, B)).reshape(-1), what)
    prob = ops.DeviceProblem(mask, sort=True)
    plain = prob.sddmm(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), algorithm=1)
    torch.cuda.synchronize()
    assert np.array_equal(got.view(np.uint16), plain.cpu().numpy().view(np.uint16)), "differs from the row kernel"


def test_device_problem_entry_and_rejections(gpu):
    mask = _mask([2048] + [40] * 255, 2048, 8, seed=13)
    A = cv.dense_normal(mask.m, 64, seed=1)
    B = cv.dense_normal(2048, 64, seed=2)
    prob = ops.DeviceProblem(mask)
    Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    out = prob.sddmm_row_parts(Ad, Bd)
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy().reshape(-1), np.asarray(_oracle(mask, A, B)).reshape(-1), "DeviceProblem.sddmm_row_parts")
    L = _lib.lib()
    parts, slots = prob.row_parts(512)[:2]
    out.fill_(9.0)
    args = lambda k, sl: (1, k, 2048, parts.n_slots, sl, mask.nnz_vec, prob.column_indices.data_ptr(), Ad.data_ptr(), 0,
                          Bd.data_ptr(), 0, out.data_ptr(), 0, 8, 0)
    assert L.vs_wmma_sddmm_f16_row_parts(*args(60, slots.data_ptr())) == 801      # k not a multiple of 8
    assert L.vs_wmma_sddmm_f16_row_parts(*args(64, slots.data_ptr() + 4)) == 1    # misaligned list
    assert L.vs_wmma_sddmm_f16_row_parts(*args(64, 0)) == 1
    torch.cuda.synchronize()
    assert bool((out == 9.0).all()), "a rejected call must not launch anything"


def test_batch_on_a_shared_mask(gpu):
    rng = np.random.default_rng(31)
    lengths = np.minimum((rng.pareto(1.4, 120) + 0.2) * 60, 2000).astype(np.int64)
    lengths[5] = 2000
    mask = _mask(lengths, 2000, 4, seed=32)
    batch, K = 6, 64
    As = np.stack([cv.dense_normal(mask.m, K, seed=50 + b) for b in range(batch)])
    Bs = np.stack([cv.dense_normal(2000, K, seed=60 + b) for b in range(batch)])
    parts = ops.RowParts(mask.m_vec, mask.row_offsets, 256)
    assert parts.n_split > 0
    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    slots, ci, Ad, Bd = d(parts.slots), d(mask.column_indices), d(As), d(Bs)
    out = torch.full((batch, mask.nnz_vec, 4), 3.0, dtype=torch.float16, device="cuda")
    ops.sddmm_row_parts(K, 2000, parts, slots, mask.nnz_vec, ci, Ad, Bd, out, 4)
    torch.cuda.synchronize()
    for b in range(batch):
        assert_parity(out[b].cpu().numpy().reshape(-1), np.asarray(_oracle(mask, As[b], Bs[b])).reshape(-1),
                      "batched SDDMM, problem %d" % b)

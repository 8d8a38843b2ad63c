"""Batched entry points, sparse softmax and the fixed-mask attention layer on the GPU."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import numpy_oracle as no
from vectorsparse_amd import ops
from vectorsparse_amd import colvec_csr as cv
from util import assert_parity

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("V", [1, 2, 4, 8])
def test_sparse_softmax_parity(gpu, V):
    # ragged rows incl. empty ones, a row longer than the register-cached limit (512 vectors)
    lengths = np.array([0, 1, 3, 64, 65, 200, 513, 700, 0, 17], dtype=np.int64)
    rng = np.random.default_rng(V)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), 1024, lengths)
    pat = cv.random_values(cv.ColVecCSR(len(lengths), 1024, V, ro, ci), seed=V + 1, scale=3.0)
    prob = ops.DeviceProblem(pat, sort=True)
    scale = 0.125
    out = ops.sparse_softmax(pat.m_vec, V, prob.row_indices, prob.row_offsets, prob.values, scale=scale)
    torch.cuda.synchronize()
    ref = no.sparse_softmax_ref(pat.m_vec, V, pat.row_offsets, pat.values, scale)
    assert_parity(out.cpu().numpy(), ref, "softmax V%d" % V)
    # in place
    vals = prob.values.clone()
    ops.sparse_softmax(pat.m_vec, V, prob.row_indices, prob.row_offsets, vals, vals, scale=scale)
    torch.cuda.synchronize()
    assert np.array_equal(vals.cpu().numpy(), out.cpu().numpy())


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_batched_equals_unbatched(gpu, kernel):
    V, heads, K, N = 8, 5, 64, 64
    pat = cv.binomial_pattern(24, 192, 0.8, seed=2, vec_length=V)
    prob = ops.DeviceProblem(pat)
    g = torch.Generator(device="cuda").manual_seed(0)
    lhs = torch.randn((heads, pat.m, K), device="cuda", generator=g).half()
    rhs = torch.randn((heads, 192, K), device="cuda", generator=g).half()
    dense = torch.rand((heads, 192, N), device="cuda", generator=g).half()
    scores = torch.empty((heads, pat.nnz_vec, V), dtype=torch.float16, device="cuda")
    ops.sddmm_batched(pat.m_vec, K, 192, pat.nnz_vec, prob.row_indices, prob.row_offsets, prob.column_indices,
                      lhs, rhs, scores, V, kernel=kernel)
    out = torch.empty((heads, pat.m, N), dtype=torch.float16, device="cuda")
    ops.spmm_batched(pat.m_vec, V, N, 192, prob.row_indices, prob.row_offsets, prob.column_indices, scores, dense,
                     out, kernel=kernel)
    torch.cuda.synchronize()
    for h in range(heads):
        one = prob.sddmm(lhs[h], rhs[h], kernel=kernel)
        assert torch.equal(one, scores[h]), "head %d sddmm" % h
        prob.values = scores[h]
        assert torch.equal(prob.spmm(dense[h], kernel=kernel), out[h]), "head %d spmm" % h
    # a shared (stride 0) dense operand
    shared = torch.empty_like(out)
    ops.spmm_batched(pat.m_vec, V, N, 192, prob.row_indices, prob.row_offsets, prob.column_indices, scores,
                     dense[0], shared, kernel=kernel)
    torch.cuda.synchronize()
    prob.values = scores[3]
    assert torch.equal(prob.spmm(dense[0], kernel=kernel), shared[3])


@pytest.mark.parametrize("kernel", ["wmma", "cuda"])
def test_attention_layer_vs_dense_masked_attention(gpu, kernel):
    # config-5 structure at a size the float64 brute force finishes quickly: band + strided column mask
    V, heads, seq, d = 8, 3, 512, 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=64, stride=64)
    layer = ops.SparseAttention(mask)
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((heads, seq, d)).astype(np.float16) for _ in range(3))
    out = layer.forward(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(),
                        kernel=kernel)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    dense_mask = np.zeros((seq, seq), dtype=bool)
    for i in range(mask.m_vec):
        cols = mask.column_indices[mask.row_offsets[i]:mask.row_offsets[i + 1]]
        dense_mask[i * V:(i + 1) * V, cols] = True
    for h in range(heads):
        s = q[h].astype(np.float64) @ k[h].astype(np.float64).T / np.sqrt(d)
        s[~dense_mask] = -np.inf
        p = np.exp(s - s.max(axis=1, keepdims=True))
        p /= p.sum(axis=1, keepdims=True)
        ref = p @ v[h].astype(np.float64)
        # End to end against an unrounded float64 layer: the chain rounds to fp16 three times (scores,
        # probabilities, output), so the per-element 1e-2 criterion of a single operator does not apply
        # to near-zero outputs; the bound here is max |error| <= 1e-2 * rms(ref).  The per-operator
        # criterion is checked step by step in test_attention_steps_match_the_oracle_chain.
        rms = float(np.sqrt(np.mean(ref * ref)))
        err = float(np.max(np.abs(got[h].astype(np.float64) - ref))) / rms
        assert err <= 1e-2, "attention head %d %s: max |err| / rms = %.3e" % (h, kernel, err)


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("N", [64, 256])
def test_softmax_fused_into_spmm(gpu, V, N):
    # ragged rows incl. empty ones and rows long enough for several waves; scores with a wide range
    lengths = np.array([0, 1, 31, 32, 33, 64, 200, 513, 0, 17, 90, 300], dtype=np.int64)
    rng = np.random.default_rng(V + N)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), 640, lengths)
    pat = cv.random_values(cv.ColVecCSR(len(lengths), 640, V, ro, ci), seed=V, scale=4.0)
    W = cv.dense_uniform(640, N, seed=9)
    scale = 0.3
    prob = ops.DeviceProblem(pat, sort=True)
    out = torch.full((pat.m, N), 7.0, dtype=torch.float16, device="cuda")
    ops.spmm_softmax_batched(pat.m_vec, V, N, 640, prob.row_indices, prob.row_offsets, prob.column_indices,
                             prob.values, torch.from_numpy(W).cuda(), out, scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy().astype(np.float64)
    # (1) against the exact float64 definition softmax(scale*x) @ W.  The probabilities enter the MFMA as
    # fp16 (as they do when the separate softmax kernel stores them), so outputs that cancel to nearly
    # zero carry that rounding; the bound for the fused operator is max |err| <= 1e-2 * rms(ref) per row.
    probs = no.sparse_softmax_ref(pat.m_vec, V, pat.row_offsets, pat.values, scale)
    # (2) against the same definition with the exponentials rounded to fp16 where the kernel rounds them
    # (before the normalisation): here the per-element 1e-2 criterion of a single operator applies.
    x = pat.values.astype(np.float64) * scale
    exact = np.zeros((pat.m, N))
    rounded = np.zeros((pat.m, N))
    for i in range(pat.m_vec):
        lo, hi = int(ro[i]), int(ro[i + 1])
        if hi > lo:
            rows = W[ci[lo:hi]].astype(np.float64)
            exact[i * V:(i + 1) * V] = probs[lo:hi].T @ rows
            e = np.exp(x[lo:hi] - x[lo:hi].max(axis=0, keepdims=True))
            rounded[i * V:(i + 1) * V] = (e.astype(np.float16).astype(np.float64).T @ rows) / e.sum(axis=0)[:, None]
    assert_parity(got, rounded, "softmax+spmm V%d N%d" % (V, N))
    rms = np.sqrt(np.mean(exact * exact, axis=1, keepdims=True))
    nonempty = rms[:, 0] > 0
    assert float(np.max(np.abs(got - exact)[nonempty] / rms[nonempty])) <= 1e-2
    for i in np.nonzero(lengths == 0)[0]:
        assert not out[i * V:(i + 1) * V].any()


def test_fused_and_unfused_layers_agree(gpu):
    V, heads, seq, d = 8, 16, 1024, 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=128, stride=128)
    layer = ops.SparseAttention(mask)
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.randn((heads, seq, d), device="cuda", generator=g).half() for _ in range(3))
    a = layer.forward(q, k, v, fused=True).float().cpu().numpy()
    b = layer.forward(q, k, v, fused=False).float().cpu().numpy()
    rms = float(np.sqrt(np.mean(b * b)))
    assert float(np.max(np.abs(a - b))) <= 1e-2 * rms
    # the default: one launch where blocks of rows share their columns, two launches where they do not
    assert layer.union_rows(d, d, heads) == 128 // V
    assert torch.equal(layer.forward(q, k, v), layer.forward(q, k, v, fused="layer"))
    scattered = ops.SparseAttention(cv.uniform_pattern(seq // V, seq, 0.9, seed=2, vec_length=V))
    assert scattered.union_rows(d, d, heads) == 1
    assert torch.equal(scattered.forward(q, k, v), scattered.forward(q, k, v, fused=True))
    # few heads: a launch of few workgroups is as long as its longest workgroup, and the two launches win
    assert layer.union_rows(d, d, 2) == 1
    assert torch.equal(layer.forward(q[:2], k[:2], v[:2]), layer.forward(q[:2], k[:2], v[:2], fused=True))


def test_attention_steps_match_the_oracle_chain(gpu):
    # the same layer step by step against the three oracles (exact intermediate layout)
    V, seq, d = 8, 256, 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=32, stride=32)
    prob = ops.DeviceProblem(mask)
    rng = np.random.default_rng(7)
    q, k, v = (rng.standard_normal((seq, d)).astype(np.float16) for _ in range(3))
    scores = prob.sddmm(torch.from_numpy(q).cuda(), torch.from_numpy(k).cuda())
    torch.cuda.synchronize()
    s_host = scores.cpu().numpy()
    assert_parity(s_host.reshape(-1),
                  co.sddmm_host_ref_f32(mask.m_vec, d, V, mask.row_offsets, mask.column_indices, q, k), "scores")
    probs = ops.sparse_softmax(mask.m_vec, V, prob.row_indices, prob.row_offsets, scores, scale=0.125)
    torch.cuda.synchronize()
    p_host = probs.cpu().numpy()
    assert_parity(p_host, no.sparse_softmax_ref(mask.m_vec, V, mask.row_offsets, s_host, 0.125), "probs")
    prob.values = probs
    out = prob.spmm(torch.from_numpy(v).cuda())
    torch.cuda.synchronize()
    assert_parity(out.cpu().numpy(),
                  co.spmm_host_ref_f32(mask.m_vec, V, d, seq, mask.row_offsets, mask.column_indices, p_host, v),
                  "context")


def _dense_attention(mask, q, k, v, scale):
    V = mask.vec_length
    allowed = np.zeros((mask.m, mask.n), dtype=bool)
    for i in range(mask.m_vec):
        cols = mask.column_indices[mask.row_offsets[i]:mask.row_offsets[i + 1]]
        allowed[i * V:(i + 1) * V, cols] = True
    out = np.zeros((q.shape[0], mask.m, v.shape[2]))
    for h in range(q.shape[0]):
        s = q[h].astype(np.float64) @ k[h].astype(np.float64).T * scale
        s[~allowed] = -np.inf
        with np.errstate(invalid="ignore"):
            p = np.exp(s - np.where(allowed.any(axis=1, keepdims=True), s.max(axis=1, keepdims=True), 0.0))
        p[~allowed] = 0.0
        denom = p.sum(axis=1, keepdims=True)
        p = np.divide(p, denom, out=np.zeros_like(p), where=denom > 0)
        out[h] = p @ v[h].astype(np.float64)
    return out


OBSERVED = {"loose": 0.0, "strict": 0.0}


def _check_layer(got, ref, what, kind="chain"):
    # End-to-end bounds for a chain with fp16 operands in both MFMA stages, fp16 probabilities and an fp16 result.
    # loose: |err| / max(|ref|, rms(ref)) - relative for the large outputs, absolute at the scale of a typical
    # output for those near zero; strict: the per-operator metric of tests/util.py, |err| / max(|ref|, 1e-2 rms),
    # which for a chain is dominated by the outputs that cancel to near zero.  Both are printed; the limits (LIMITS
    # below) are about twice the largest values observed over this file's cases on MI355X.
    ref = np.asarray(ref, dtype=np.float64)
    got = got.astype(np.float64)
    rms = float(np.sqrt(np.mean(ref * ref)))
    loose = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), rms)))
    strict = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-2 * rms)))
    OBSERVED["loose"] = max(OBSERVED["loose"], loose)
    OBSERVED["strict"] = max(OBSERVED["strict"], strict)
    print("attention parity %-60s loose %.3e  strict %.3e" % (what, loose, strict))
    assert np.all(np.isfinite(got)), what
    loose_limit, strict_limit = LIMITS[kind]
    assert loose <= loose_limit, "%s: max |err| / max(|ref|, rms) = %.3e > %.1e" % (what, loose, loose_limit)
    assert strict <= strict_limit, "%s: max |err| / max(|ref|, 1e-2 rms) = %.3e > %.2f" % (what, strict, strict_limit)


# Largest values observed over this file's cases on MI355X -> limit (about twice the observation):
#   single-launch kernels (per-row, union, streamed; scores and probabilities stay on the chip):
#       loose 1.4e-3, strict 8.1e-2  ->  3e-3, 0.17
#   chains with fp16 scores / probabilities in memory (SDDMM -> softmax -> SpMM, softmax-fused SpMM, and
#   whatever `forward` picks): loose 7.0e-3, strict 0.33  ->  1e-2 (the contract's figure), 0.7
LIMITS = {"single": (3e-3, 0.17), "chain": (1e-2, 0.7)}


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("dims", [(64, 64), (32, 128), (128, 40), (72, 64)], ids=lambda d: "dqk%d_dv%d" % d)
def test_single_launch_attention(gpu, V, dims):
    d_qk, d_v = dims
    heads = 3
    lengths = np.array([0, 1, 15, 16, 17, 31, 32, 33, 64, 130, 300, 5, 0, 48, 7, 100], dtype=np.int64)
    rng = np.random.default_rng(V * 7 + d_qk)
    n = 384
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), n, lengths)
    mask = cv.ColVecCSR(len(lengths), n, V, ro, ci).validate()
    prob = ops.DeviceProblem(mask, sort=True)
    q = rng.standard_normal((heads, mask.m, d_qk)).astype(np.float16)
    k = rng.standard_normal((heads, n, d_qk)).astype(np.float16)
    v = rng.standard_normal((heads, n, d_v)).astype(np.float16)
    scale = 1.0 / np.sqrt(d_qk)
    ref = _dense_attention(mask, q, k, v, scale)
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    try:
        # (chunk, waves, rows per workgroup): one chunk / several chunks per long row; rows = 1 is the
        # one-row-per-workgroup kernel, anything else the union-gather kernel (LDS copy or global fallback)
        for chunk, waves, rows in ((0, 0, 1), (64, 3, 1), (32, 8, 1), (96, 1, 0), (0, 0, 8), (64, 0, 3), (32, 0, 5), (0, 0, 16), (0, 0, 128)):
            _lib_set("attention_chunk", chunk)
            _lib_set("attention_waves", waves)
            pad = torch.full((heads, mask.m + 16, d_v), 3.0, dtype=torch.float16, device="cuda")
            out = pad[:, 8:8 + mask.m]
            ops.sparse_attention(mask.m_vec, V, n, prob.row_indices, prob.row_offsets, prob.column_indices,
                                 qd, kd, vd, out=out, scale=scale, rows_per_workgroup=rows)
            torch.cuda.synchronize()
            host = pad.cpu().numpy()
            assert np.all(host[:, :8] == 3.0) and np.all(host[:, 8 + mask.m:] == 3.0), "wrote outside the output"
            _check_layer(host[:, 8:8 + mask.m], ref,
                         "V%d dqk%d dv%d chunk%d waves%d rows%d" % (V, d_qk, d_v, chunk, waves, rows), kind="single")
            for i in np.nonzero(lengths == 0)[0]:
                assert not host[:, 8 + i * V:8 + (i + 1) * V].any(), "an empty row must produce zeros"
    finally:
        _lib_set("attention_chunk", 0)
        _lib_set("attention_waves", 0)


@pytest.mark.parametrize("V", [2, 8])
def test_union_gather_on_structured_and_random_masks(gpu, V):
    heads, seq, d = 2, 1024, 64
    rng = np.random.default_rng(V)
    q, k, v = (rng.standard_normal((heads, seq, d)).astype(np.float16) for _ in range(3))
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    masks = {
        "band": cv.band_strided_pattern(seq, V, band_half_width=64, stride=128),     # union fits LDS
        "random": cv.uniform_pattern(seq // V, seq, 0.7, seed=3, vec_length=V),      # union too large: fallback
    }
    for name, mask in masks.items():
        prob = ops.DeviceProblem(mask)
        ref = _dense_attention(mask, q, k, v, 0.125)
        for rows in (1, 2, 4, 8, 16, 64, 128):
            out = ops.sparse_attention(mask.m_vec, V, seq, prob.row_indices, prob.row_offsets,
                                       prob.column_indices, qd, kd, vd, scale=0.125, rows_per_workgroup=rows)
            again = ops.sparse_attention(mask.m_vec, V, seq, prob.row_indices, prob.row_offsets,
                                         prob.column_indices, qd, kd, vd, scale=0.125, rows_per_workgroup=rows)
            torch.cuda.synchronize()
            _check_layer(out.cpu().numpy(), ref, "%s mask V%d rows%d" % (name, V, rows), kind="single")
            assert torch.equal(out, again)      # deterministic
        if name == "band":
            assert ops.SparseAttention(mask).union_rows(d, d) == 128 // V


def _with_empty_rows(mask, first, last):
    """The same pattern with vector rows [first, last) emptied: whole workgroups without a single column."""
    lengths = np.diff(mask.row_offsets).copy()
    keep = np.ones(mask.nnz_vec, dtype=bool)
    keep[mask.row_offsets[first]:mask.row_offsets[last]] = False
    lengths[first:last] = 0
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    return cv.ColVecCSR(mask.m_vec, mask.n, mask.vec_length, offsets, mask.column_indices[keep].copy())


def _capacity(V, n, d_qk, d_v, rows, with_plan):
    """Distinct columns a workgroup takes without (0) or with (1) a plan."""
    from vectorsparse_amd import _lib
    return _lib.lib().vs_sparse_attention_union_capacity(V, n, d_qk, d_v, rows, with_plan, None)


def _unions(mask, rows):
    """Distinct columns of every block of `rows` consecutive vector rows."""
    ro, ci = mask.row_offsets, mask.column_indices
    return [int(np.unique(ci[ro[f]:ro[min(f + rows, mask.m_vec)]]).size) for f in range(0, mask.m_vec, rows)]


@pytest.mark.parametrize("V,seq,half_width,stride,rows", [(4, 4096, 176, 32, 8), (1, 2048, 128, 16, 128)])
def test_plan_raises_the_union_capacity(gpu, V, seq, half_width, stride, rows):
    """Blocks whose distinct columns fit a workgroup's LDS only when the column bitmap and the column list
    stay out of it: dense tile with a plan, per-row path without, both equal to dense masked attention."""
    d = 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=half_width, stride=stride)
    built, held = _capacity(V, seq, d, d, rows, 0), _capacity(V, seq, d, d, rows, 1)
    unions = _unions(mask, rows)
    assert built < max(unions) <= held and min(unions) <= built, (built, held, min(unions), max(unions))
    rng = np.random.default_rng(70 + V)
    q, k, v = (rng.standard_normal((1, seq, d)).astype(np.float16) for _ in range(3))
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    ref = _dense_attention(mask, q, k, v, 0.125)
    layer = ops.SparseAttention(mask)
    assert layer.union_rows(d, d) >= rows                 # the host-side choice counts on the plan
    prob = layer.prob
    args = (mask.m_vec, V, seq, prob.row_indices, prob.row_offsets, prob.column_indices, qd, kd, vd)
    plan = ops.sparse_attention_plan(mask.m_vec, V, seq, d, d, rows, prob.row_offsets, prob.column_indices)
    planned = ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=rows, plan=plan)
    rebuilt = ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=rows)
    out = layer.forward(qd, kd, vd, scale=0.125)
    torch.cuda.synchronize()
    _check_layer(planned.cpu().numpy(), ref, "V%d planned" % V, kind="single")
    _check_layer(rebuilt.cpu().numpy(), ref, "V%d rebuilt" % V, kind="single")
    _check_layer(out.cpu().numpy(), ref, "V%d layer" % V)
    assert not torch.equal(planned, rebuilt)              # different summation orders: the paths did differ


@pytest.mark.parametrize("V,seq,half_width,stride,dims", [
    (8, 4096, 300, 64, (64, 64)),      # unions of about 700 columns: six sub-rounds of 128
    (8, 4096, 900, 128, (64, 64)),     # about 1900 columns: fifteen sub-rounds
    (2, 2048, 400, 0, (32, 128)),      # plain band, wide V rows (one workgroup per CU)
    (1, 2048, 400, 256, (64, 64)),     # 128 vector rows per workgroup
])
def test_planned_launch_streams_large_unions(gpu, V, seq, half_width, stride, dims):
    """Unions of more columns than fit in LDS at once: with a plan, eight waves stream them through LDS with
    a running maximum and sums; rows whose columns all fall into a late sub-round, rows empty in some
    sub-round, a negative and a zero scale go through the same rescaling."""
    d_qk, d_v = dims
    mask = cv.band_strided_pattern(seq, V, band_half_width=half_width, stride=stride or seq)
    mask = _with_empty_rows(mask, 3, 5)
    rows = 128 // V
    unions = _unions(mask, rows)
    assert 512 < max(unions) <= _capacity(V, seq, d_qk, d_v, rows, 1) == 2048
    rng = np.random.default_rng(90 + V)
    q = rng.standard_normal((2, seq, d_qk)).astype(np.float16)
    k = rng.standard_normal((2, seq, d_qk)).astype(np.float16)
    v = rng.standard_normal((2, seq, d_v)).astype(np.float16)
    # make the maximum of many rows sit in a late sub-round: large keys at the top end of the sequence
    k[:, seq - seq // 8:, :] *= 3.0
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    prob = ops.DeviceProblem(mask)
    args = (mask.m_vec, V, seq, prob.row_indices, prob.row_offsets, prob.column_indices, qd, kd, vd)
    plan = ops.sparse_attention_plan(mask.m_vec, V, seq, d_qk, d_v, rows, prob.row_offsets, prob.column_indices)
    for scale in (0.125, -0.125, 0.0):
        ref = _dense_attention(mask, q, k, v, scale)
        planned = ops.sparse_attention(*args, scale=scale, rows_per_workgroup=rows, plan=plan)
        again = ops.sparse_attention(*args, scale=scale, rows_per_workgroup=rows, plan=plan)
        torch.cuda.synchronize()
        _check_layer(planned.cpu().numpy(), ref, "V%d scale %g streamed" % (V, scale), kind="single")
        assert torch.equal(planned, again)
    layer = ops.SparseAttention(mask)
    assert layer.union_rows(d_qk, d_v, 16) == rows        # the host-side choice counts on the streamed kernel
    out = layer.forward(*(x.repeat(8, 1, 1) for x in (qd, kd, vd)), scale=0.125)     # sixteen heads
    torch.cuda.synchronize()
    _check_layer(out[:2].cpu().numpy(), _dense_attention(mask, q, k, v, 0.125), "V%d layer streamed" % V)
    assert torch.equal(out[:2], out[14:])


@pytest.mark.parametrize("V", [1, 8])
def test_planned_launch_equals_unplanned(gpu, V):
    """Workgroups of fewer than eight waves: the plan holds exactly what the kernel would rebuild, same bits
    out.  Eight waves stream the union when they have a plan (another order of summation): both meet the
    layer bound.  A plan made for another launch shape is ignored safely (per-row path)."""
    heads, seq, d = 2, 1024, 64
    rng = np.random.default_rng(40 + V)
    q, k, v = (rng.standard_normal((heads, seq, d)).astype(np.float16) for _ in range(3))
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    masks = {
        "band": cv.band_strided_pattern(seq, V, band_half_width=64, stride=128),
        "random": cv.uniform_pattern(seq // V, seq, 0.7, seed=3, vec_length=V),   # every union too large
        "ragged": cv.binomial_pattern(seq // V, seq, 0.97, seed=4, vec_length=V),  # some fit, some do not
        "hollow": _with_empty_rows(cv.band_strided_pattern(seq, V, band_half_width=32, stride=256), 16 // V, 9 * (16 // V)),
    }
    for name, mask in masks.items():
        prob = ops.DeviceProblem(mask)
        ref = _dense_attention(mask, q, k, v, 0.125)
        for rows in (16 // V, 4 * (16 // V), 128 // V):
            args = (mask.m_vec, V, seq, prob.row_indices, prob.row_offsets, prob.column_indices, qd, kd, vd)
            plain = ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=rows)
            plan = ops.sparse_attention_plan(mask.m_vec, V, seq, d, d, rows, prob.row_offsets, prob.column_indices)
            planned = ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=rows, plan=plan)
            torch.cuda.synchronize()
            _check_layer(planned.cpu().numpy(), ref, "%s V%d rows%d planned" % (name, V, rows), kind="single")
            # a planned launch holds more columns per workgroup: same bits unless some union fits only then
            built, held = _capacity(V, seq, d, d, rows, 0), _capacity(V, seq, d, d, rows, 1)
            streamed = rows == 128 // V
            if not streamed and not any(built < u <= held for u in _unions(mask, rows)):
                assert torch.equal(plain, planned), "%s V%d rows%d" % (name, V, rows)
            else:
                _check_layer(plain.cpu().numpy(), ref, "%s V%d rows%d rebuilt" % (name, V, rows), kind="single")
        # a negative scale (sign handled inside the kernel) through the same paths
        neg = ops.sparse_attention(*args, scale=-0.125, rows_per_workgroup=128 // V, plan=plan)
        torch.cuda.synchronize()
        _check_layer(neg.cpu().numpy(), _dense_attention(mask, q, k, v, -0.125), "%s V%d negative scale" % (name, V), kind="single")
        # a plan made for another launch shape: rejected on the host when it is too small for this shape (the
        # kernels read it at this shape's offsets before they can tell), detected in the kernel and ignored when
        # it is large enough
        from vectorsparse_amd import _lib
        other = ops.sparse_attention_plan(mask.m_vec, V, seq, d, d, 16 // V, prob.row_offsets, prob.column_indices)
        need = _lib.lib().vs_sparse_attention_plan_bytes(mask.m_vec, V, seq, d, d, 128 // V)
        if other.numel() < need:
            with pytest.raises(_lib.VSparseError):
                ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=128 // V, plan=other)
            other = torch.cat([other, torch.zeros(need - other.numel(), dtype=torch.uint8, device="cuda")])
        tiny = torch.zeros(64, dtype=torch.uint8, device="cuda")
        with pytest.raises(_lib.VSparseError):
            ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=128 // V, plan=tiny)
        out = ops.sparse_attention(*args, scale=0.125, rows_per_workgroup=128 // V, plan=other)
        torch.cuda.synchronize()
        _check_layer(out.cpu().numpy(), ref, "%s V%d foreign plan" % (name, V), kind="single")


def _lib_set(name, value):
    from vectorsparse_amd import _lib
    _lib.set_option(name, value)


def test_single_launch_layer_matches_three_launch_layer(gpu):
    V, heads, seq, d = 8, 4, 1024, 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=128, stride=128)
    layer = ops.SparseAttention(mask)
    g = torch.Generator(device="cuda").manual_seed(2)
    q, k, v = (torch.randn((heads, seq, d), device="cuda", generator=g).half() for _ in range(3))
    a = layer.forward(q, k, v, fused="layer").float().cpu().numpy()
    b = layer.forward(q, k, v, fused=False).float().cpu().numpy()
    rms = float(np.sqrt(np.mean(b * b)))
    assert float(np.max(np.abs(a - b))) <= 1e-2 * rms
    again = layer.forward(q, k, v, fused="layer").float().cpu().numpy()
    assert np.array_equal(a, again)       # deterministic


def test_single_launch_attention_rejects_unsupported_shapes(gpu):
    from vectorsparse_amd import _lib
    mask = cv.uniform_pattern(4, 64, 0.5, seed=1, vec_length=8)
    prob = ops.DeviceProblem(mask)
    q = torch.zeros((1, 32, 256), dtype=torch.float16, device="cuda")
    k = torch.zeros((1, 64, 256), dtype=torch.float16, device="cuda")
    v = torch.zeros((1, 64, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(_lib.VSparseError):     # d_qk > 128: use the three-operator chain
        ops.sparse_attention(4, 8, 64, prob.row_indices, prob.row_offsets, prob.column_indices, q, k, v)


def test_union_kernel_on_awkward_shapes(gpu):
    """Seeded random shapes around the kernel's granularities: n not a multiple of 32 (bitmap words), fewer
    rows than a workgroup takes, head widths that leave MFMA slices partly empty, a column in the last
    position, with and without a plan."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        V = int(rng.choice([1, 2, 4, 8]))
        n = int(rng.choice([1, 7, 31, 32, 33, 100, 257, 500]))
        m_vec = int(rng.choice([1, 3, 16 // V, 16 // V + 1, 37]))
        d_qk = int(rng.choice([8, 24, 40, 64, 104, 128]))
        d_v = int(rng.choice([8, 16, 48, 64, 72, 128]))
        rows = int(rng.choice([2, 3, 16 // V, 5 * (16 // V), 128]))
        heads = int(rng.choice([1, 3]))
        lengths = rng.integers(0, min(n, 60) + 1, m_vec)
        ro, ci = cv._pattern_from_lengths(rng, m_vec, n, lengths)
        if ro[m_vec] > ro[m_vec - 1]:
            ci[-1] = n - 1        # columns of a row ascend, so its last one can be moved to the mask's last column
        mask = cv.ColVecCSR(m_vec, n, V, ro, ci)
        mask.validate()
        q = rng.standard_normal((heads, mask.m, d_qk)).astype(np.float16)
        k = rng.standard_normal((heads, n, d_qk)).astype(np.float16)
        v = rng.standard_normal((heads, n, d_v)).astype(np.float16)
        scale = 1.0 / np.sqrt(d_qk)
        ref = _dense_attention(mask, q, k, v, scale)
        prob = ops.DeviceProblem(mask)
        qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
        what = "case %d: V%d n%d m_vec%d dqk%d dv%d rows%d heads%d" % (case, V, n, m_vec, d_qk, d_v, rows, heads)
        print(what, flush=True)
        args = (mask.m_vec, V, n, prob.row_indices, prob.row_offsets, prob.column_indices, qd, kd, vd)
        pad = torch.full((heads, mask.m + 16, d_v), 5.0, dtype=torch.float16, device="cuda")
        ops.sparse_attention(*args, out=pad[:, 8:8 + mask.m], scale=scale, rows_per_workgroup=rows)
        plan = ops.sparse_attention_plan(mask.m_vec, V, n, d_qk, d_v, rows, prob.row_offsets, prob.column_indices)
        planned = ops.sparse_attention(*args, scale=scale, rows_per_workgroup=rows, plan=plan)
        torch.cuda.synchronize()
        host = pad.cpu().numpy()
        assert np.all(host[:, :8] == 5.0) and np.all(host[:, 8 + mask.m:] == 5.0), what + ": wrote outside the output"
        if np.sqrt(np.mean(ref * ref)) > 0:
            _check_layer(host[:, 8:8 + mask.m], ref, what, kind="single")
            _check_layer(planned.cpu().numpy(), ref, what + " planned", kind="single")
        else:
            assert not host[:, 8:8 + mask.m].any() and not planned.cpu().numpy().any(), what


def test_config5_full_size(gpu):
    """The benchmark set's attention layer at its real size (16 heads x 4096 x 64, V = 8, band 257 + every 128th column) through
    the path the benchmark takes (plan + union kernel) and through the per-row kernel, against a float64
    dense masked attention computed head by head."""
    V, heads, seq, d = 8, 16, 4096, 64
    mask = cv.band_strided_pattern(seq, V, band_half_width=128, stride=128)
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal((heads, seq, d)).astype(np.float16) for _ in range(3))
    allowed = np.zeros((seq, seq), dtype=bool)
    for i in range(mask.m_vec):
        allowed[i * V:(i + 1) * V, mask.column_indices[mask.row_offsets[i]:mask.row_offsets[i + 1]]] = True
    ref = np.empty((heads, seq, d))
    for h in range(heads):
        s = (q[h].astype(np.float64) @ k[h].astype(np.float64).T) * 0.125
        s[~allowed] = -np.inf
        p = np.exp(s - s.max(axis=1, keepdims=True))
        ref[h] = (p / p.sum(axis=1, keepdims=True)) @ v[h].astype(np.float64)
    layer = ops.SparseAttention(mask)
    assert layer.union_rows(d, d) == 16
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    out = layer.forward(qd, kd, vd)                       # plan + union kernel
    prob = layer.prob
    per_row = ops.sparse_attention(mask.m_vec, V, seq, prob.row_indices, prob.row_offsets, prob.column_indices,
                                   qd, kd, vd, scale=0.125)
    chain = layer.forward(qd, kd, vd, fused=False)        # SDDMM -> softmax -> SpMM, three launches
    torch.cuda.synchronize()
    _check_layer(out.cpu().numpy(), ref, "config 5, union kernel with plan", kind="single")
    _check_layer(per_row.cpu().numpy(), ref, "config 5, per-row kernel", kind="single")
    _check_layer(chain.cpu().numpy(), ref, "config 5, three operators")


def _random_mask(rng, seq, V, kind):
    m_vec = seq // V
    if kind == "band":
        return cv.band_strided_pattern(seq, V, band_half_width=int(rng.integers(8, 200)),
                                       stride=int(rng.choice([16, 64, 128, seq])))
    if kind == "blocks":
        block = int(rng.choice([32, 64, 256]))
        shared = np.sort(rng.choice(seq, int(rng.integers(0, 64)), replace=False))
        rows = [np.union1d(np.arange((r * V) // block * block, min(seq, ((r * V) // block + 1) * block)), shared)
                for r in range(m_vec)]
    else:  # ragged: anything from empty rows to nearly full ones
        rows = [np.sort(rng.choice(seq, int(rng.integers(0, seq if r % 7 == 0 else 40)), replace=False))
                for r in range(m_vec)]
    offsets = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int32)
    return cv.ColVecCSR(m_vec, seq, V, offsets, np.concatenate(rows).astype(np.int32)).validate()


@pytest.mark.parametrize("seed", range(12))
def test_attention_random_cases(gpu, seed):
    """Seeded mixes of vector length, sequence length, head widths, mask family and workgroup size through
    every attention path, against dense masked attention."""
    rng = np.random.default_rng(1000 + seed)
    V = int(rng.choice([1, 2, 4, 8]))
    seq = int(rng.choice([128, 200, 512, 1000])) // V * V
    d_qk = int(rng.choice([8, 32, 64, 72, 128]))
    d_v = int(rng.choice([8, 40, 64, 128]))
    heads = int(rng.integers(1, 4))
    mask = _random_mask(rng, seq, V, ["band", "blocks", "ragged"][seed % 3])
    q = rng.standard_normal((heads, seq, d_qk)).astype(np.float16)
    k = rng.standard_normal((heads, seq, d_qk)).astype(np.float16)
    v = rng.standard_normal((heads, seq, d_v)).astype(np.float16)
    scale = float(rng.choice([0.05, 0.125, -0.1]))
    ref = _dense_attention(mask, q, k, v, scale)
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    prob = ops.DeviceProblem(mask, sort=bool(seed % 2))
    args = (mask.m_vec, V, seq, prob.row_indices, prob.row_offsets, prob.column_indices, qd, kd, vd)
    what = "seed %d V%d seq %d d %d/%d" % (seed, V, seq, d_qk, d_v)
    out = ops.sparse_attention(*args, scale=scale)
    torch.cuda.synchronize()
    _check_layer(out.cpu().numpy(), ref, what + " per row", kind="single")
    for rows in (16 // V, 128 // V):
        if rows < 2:
            continue
        out = ops.sparse_attention(*args, scale=scale, rows_per_workgroup=rows)
        torch.cuda.synchronize()
        _check_layer(out.cpu().numpy(), ref, what + " rows %d rebuilt" % rows, kind="single")
        if _capacity(V, seq, d_qk, d_v, rows, 1) > 0:
            plan = ops.sparse_attention_plan(mask.m_vec, V, seq, d_qk, d_v, rows, prob.row_offsets,
                                             prob.column_indices)
            out = ops.sparse_attention(*args, scale=scale, rows_per_workgroup=rows, plan=plan)
            torch.cuda.synchronize()
            _check_layer(out.cpu().numpy(), ref, what + " rows %d planned" % rows, kind="single")
    layer = ops.SparseAttention(mask)
    for fused in (None, True, False) + (("parts",) if d_qk % 8 == 0 and d_v % 4 == 0 else ()):
        out = layer.forward(qd, kd, vd, scale=scale, fused=fused)
        torch.cuda.synchronize()
        _check_layer(out.cpu().numpy(), ref, what + " layer fused=%s" % fused)


def test_streamed_kernel_falls_back_on_oversized_unions(gpu):
    """Blocks of rows whose union exceeds what a plan lists (scattered columns over a long sequence): the
    streamed kernel's workgroups take the per-row path; a mask that mixes such blocks with banded ones runs
    both paths in one launch."""
    V, seq, d = 8, 4096, 64
    scattered = cv.uniform_pattern(seq // V, seq, 0.9, seed=11, vec_length=V)
    band = cv.band_strided_pattern(seq, V, band_half_width=64, stride=128)
    # first half of the rows banded, second half scattered
    half = band.m_vec // 2
    lengths = np.concatenate([np.diff(band.row_offsets)[:half], np.diff(scattered.row_offsets)[half:]])
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    columns = np.concatenate([band.column_indices[:band.row_offsets[half]],
                              scattered.column_indices[scattered.row_offsets[half]:]])
    mixed = cv.ColVecCSR(band.m_vec, seq, V, offsets, columns).validate()
    rng = np.random.default_rng(12)
    q, k, v = (rng.standard_normal((1, seq, d)).astype(np.float16) for _ in range(3))
    qd, kd, vd = (torch.from_numpy(x).cuda() for x in (q, k, v))
    for name, mask in (("scattered", scattered), ("mixed", mixed)):
        unions = _unions(mask, 16)
        assert max(unions) > _capacity(V, seq, d, d, 16, 1)
        assert (min(unions) <= 512) == (name == "mixed")
        prob = ops.DeviceProblem(mask)
        plan = ops.sparse_attention_plan(mask.m_vec, V, seq, d, d, 16, prob.row_offsets, prob.column_indices)
        out = ops.sparse_attention(mask.m_vec, V, seq, prob.row_indices, prob.row_offsets, prob.column_indices,
                                   qd, kd, vd, scale=0.125, rows_per_workgroup=16, plan=plan)
        torch.cuda.synchronize()
        _check_layer(out.cpu().numpy(), _dense_attention(mask, q, k, v, 0.125), name, kind="single")


@pytest.mark.parametrize("V", [1, 2, 4, 8])
@pytest.mark.parametrize("limit", [64, 200, 0])
def test_sparse_softmax_over_rows_in_parts(gpu, V, limit):
    """The softmax driven by a dispatch list of row parts: rows of every length incl. empty ones and rows of many
    parts, a batch of three, in place and out of place, against the float64 definition and the row kernel."""
    rng = np.random.default_rng(40 + V)
    lengths = np.array([0, 1, 63, 64, 65, 200, 0, 513, 1500, 31, 3000, 2, 0, 640], dtype=np.int64)
    ro, ci = cv._pattern_from_lengths(rng, len(lengths), 3000, lengths)
    pat = cv.ColVecCSR(len(lengths), 3000, V, ro, ci)
    batch = 3
    scores = (rng.standard_normal((batch, pat.nnz_vec, V)) * 3).astype(np.float16)
    scale = 0.37
    parts = ops.RowParts(pat.m_vec, pat.row_offsets, limit)
    assert parts.n_split > 0
    slots = torch.from_numpy(parts.slots).cuda()
    need = ops.sparse_softmax_row_parts_workspace_bytes(V, parts.n_split, parts.parts_max, batch=batch)
    ws = torch.full((need + 64,), 0x5A, dtype=torch.uint8, device="cuda")   # (no need to clear it)
    x = torch.from_numpy(scores).cuda()
    out = torch.full_like(x, 7.0)
    ops.sparse_softmax_row_parts(V, parts, slots, x, out, scale=scale, workspace=ws[:need])
    inplace = x.clone()
    ops.sparse_softmax_row_parts(V, parts, slots, inplace, scale=scale, workspace=ws[:need])
    prob = ops.DeviceProblem(pat)
    plain = ops.sparse_softmax(pat.m_vec, V, prob.row_indices, prob.row_offsets, x.clone(), scale=scale)
    torch.cuda.synchronize()
    assert torch.equal(out, inplace), "in place and out of place differ"
    assert bool((ws[need:] == 0x5A).all()), "wrote outside the workspace"
    for b in range(batch):
        ref = no.sparse_softmax_ref(pat.m_vec, V, pat.row_offsets, scores[b], scale)
        assert_parity(out[b].cpu().numpy(), ref, "softmax over rows in parts V%d limit %d problem %d" % (V, limit, b))
        assert_parity(out[b].cpu().numpy(), plain[b].float().cpu().numpy(), "against the row kernel")
    # one vector row of the whole: every scalar row sums to one
    sums = out[0].float().cpu().numpy()[ro[10]:ro[11]].sum(axis=0)
    assert np.allclose(sums, 1.0, atol=2e-2)


def test_attention_with_global_tokens_takes_rows_in_parts(gpu):
    """A band mask with global tokens (a few rows that attend to everything, a few columns everybody attends to): the
    layer picks the three operators on the dispatch list of row parts; same contract as the other routes."""
    seq, V, heads, d = 2048, 8, 3, 64
    rows = []
    for i in range(seq // V):
        c = i * V + V // 2
        rows.append(np.arange(seq) if i < 2 else np.union1d(np.arange(max(0, c - 24), min(seq, c + 24)), np.arange(16)))
    ro = np.concatenate([[0], np.cumsum([len(r) for r in rows])]).astype(np.int32)
    mask = cv.ColVecCSR(seq // V, seq, V, ro, np.concatenate(rows).astype(np.int32))
    layer = ops.SparseAttention(mask)
    assert layer.prob.row_parts(0)[0].n_split == 2
    g = torch.Generator(device="cuda").manual_seed(8)
    q, k, v = (torch.randn((heads, seq, d), device="cuda", generator=g).half() for _ in range(3))
    got = layer.forward(q, k, v)                       # automatic: the parts chain
    forced = layer.forward(q, k, v, fused="parts")
    chain = layer.forward(q, k, v, fused=False)        # the three operators on whole rows
    torch.cuda.synchronize()
    assert torch.equal(got, forced)
    ref = _dense_attention(mask, q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), 1.0 / 8.0)
    _check_layer(got.cpu().numpy(), ref, "rows in parts, global tokens")
    _check_layer(chain.cpu().numpy(), ref, "whole rows, global tokens")
    # against the chain on whole rows: the same arithmetic up to the order of the fp32 sums
    diff = (got.float() - chain.float()).abs().max().item()
    assert diff < 2e-2 * max(1.0, chain.float().abs().max().item()), diff

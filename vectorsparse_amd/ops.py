"""Host-side mirror of the reference's operator API over the C ABI.

The four device operators keep the reference's names, argument order and
dimension letters (include/wmma_spmm.cuh:15-21, include/cuda_spmm.cuh:15-21,
include/wmma_sddmm.cuh:17-24, include/cuda_sddmm.cuh:16-23).  Arguments are
torch tensors on the GPU (used only as owners of device memory) or raw device
addresses; the output dtype of ``output_matrix`` / ``output_values`` (fp16 or
fp32) picks the overload, as C++ overload resolution does in the reference.
Every call is asynchronous on ``stream`` (default: torch's current stream).
"""
import ctypes

import numpy as np
import torch

from . import _lib


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


# torch's raw-handle getter when this torch has it: torch.cuda.current_stream() builds a Stream object per call
# (2.8 us on the host against 0.1 us, measured; an eager SpMM launch is 3.8 us of GPU time)
_raw_current_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(stream):
    if stream is None:
        if _raw_current_stream is not None:
            return _raw_current_stream(torch.cuda.current_device())
        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, torch.cuda.Stream):
        return stream.cuda_stream
    return int(stream)


def _expect(t, dtype, name):
    """Type / placement / layout check of a tensor argument; returns its device address (raw addresses pass)."""
    if t is None or type(t) is int:
        return t
    if t.dtype is not dtype:
        raise TypeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_cuda:
        raise ValueError("%s must live in device memory" % name)
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    return t.data_ptr()


def _spmm(entry, m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
          output_matrix, stream):
    f32 = isinstance(output_matrix, torch.Tensor) and output_matrix.dtype is torch.float32
    fn = getattr(_lib.lib(), entry + "_f32out" if f32 else entry)
    st = fn(m_vec, vec_length, k, n, _expect(row_indices, torch.int32, "row_indices"),
            _expect(row_offsets, torch.int32, "row_offsets"), _expect(column_indices, torch.int32, "column_indices"),
            _expect(values, torch.float16, "values"), _expect(rhs_matrix, torch.float16, "rhs_matrix"),
            _expect(output_matrix, torch.float32 if f32 else torch.float16, "output_matrix"), _stream(stream))
    if st:
        _lib.check(st, entry)
    return output_matrix


def _sddmm(entry, m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
           output_values, vec_length, stream, algorithm=None):
    f32 = isinstance(output_values, torch.Tensor) and output_values.dtype is torch.float32
    fn = getattr(_lib.lib(), entry + "_f32out" if f32 else entry)
    args = [m_vec, k, n, nonzeros_vec, _expect(row_indices, torch.int32, "row_indices"),
            _expect(row_offsets, torch.int32, "row_offsets"), _expect(col_indices, torch.int32, "col_indices"),
            _expect(lhs_matrix, torch.float16, "lhs_matrix"), _expect(rhs_matrix, torch.float16, "rhs_matrix"),
            _expect(output_values, torch.float32 if f32 else torch.float16, "output_values"), vec_length,
            _stream(stream)]
    if algorithm is not None:
        args.append(algorithm)
    st = fn(*args)
    if st:
        _lib.check(st, entry)
    return output_values


class spmm:
    """Namespace ``spmm`` of the reference: C[m x k] = A[m x n] (column-vector CSR) * B[n x k]."""

    @staticmethod
    def wmmaSpmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                 output_matrix, stream=None):
        """MFMA path (reference: tensor-core path, src/wmma_spmm.cu:400-409)."""
        return _spmm("vs_wmma_spmm_f16", m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                     values, rhs_matrix, output_matrix, stream)

    @staticmethod
    def cudaSpmm(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                 output_matrix, stream=None):
        """Fine-grained packed-fp16 VALU path (reference: src/cuda_spmm.cu:316-325)."""
        return _spmm("vs_cuda_spmm_f16", m_vec, vec_length, k, n, row_indices, row_offsets, column_indices,
                     values, rhs_matrix, output_matrix, stream)


def spmm_launch_shape(m_vec, vec_length, k, n, batch=1, nonzeros_vec=-1, longest_row_vec=-1, long_rows=-1):
    """The launch shape `wmmaSpmm` (hints negative) or `spmm_batched` (hints as passed there) would choose, under the
    calling thread's options, as a dict; touches no device."""
    import ctypes
    shape = (ctypes.c_int * 8)()
    _lib.check(_lib.lib().vs_wmma_spmm_launch_shape(batch, m_vec, vec_length, k, n, nonzeros_vec, longest_row_vec,
                                                    long_rows, ctypes.cast(shape, ctypes.c_void_p)),
               "vs_wmma_spmm_launch_shape")
    names = ("cols_per_lane", "steps_in_flight", "waves", "blocks_per_wave", "team_slots", "ragged", "dma", "pipelined")
    return dict(zip(names, (int(x) for x in shape)))


def spmm_workspace_bytes(m_vec, vec_length, k, n, nonzeros_vec):
    """Preferred workspace size of `spmm_split_rows` for this problem (0: no row can be split)."""
    return int(_lib.lib().vs_wmma_spmm_workspace_bytes(m_vec, vec_length, k, n, nonzeros_vec))


def spmm_split_rows(m_vec, vec_length, k, n, nonzeros_vec, row_offsets, column_indices, values, rhs_matrix,
                    output_matrix, workspace=None, stream=None, row_indices=None):
    """wmmaSpmm on the schedule that splits the nonzero range instead of the rows (skewed row lengths).

    workspace: a device tensor (any dtype), zero-filled before its first use (it starts with arrival counters
    that every call leaves at zero), for the partial tiles of rows that cross workgroups; or None (one workgroup
    then takes everything).  Returns output_matrix.
    """
    f32 = output_matrix.dtype is torch.float32
    entry = "vs_wmma_spmm_f16_f32out_ws" if f32 else "vs_wmma_spmm_f16_ws"
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    st = getattr(_lib.lib(), entry)(
        m_vec, vec_length, k, n, nonzeros_vec, _expect(row_indices, torch.int32, "row_indices"),
        _expect(row_offsets, torch.int32, "row_offsets"), _expect(column_indices, torch.int32, "column_indices"),
        _expect(values, torch.float16, "values"), _expect(rhs_matrix, torch.float16, "rhs_matrix"),
        _expect(output_matrix, torch.float32 if f32 else torch.float16, "output_matrix"), _ptr(workspace), ws_bytes,
        _stream(stream))
    if st:
        _lib.check(st, entry)
    return output_matrix


def spmm_slab_workspace_bytes(m_vec, vec_length, k, n):
    """Workspace `spmm_slab` needs for this shape under the current "spmm_slab_parts" option (0: none)."""
    return int(_lib.lib().vs_wmma_spmm_slab_workspace_bytes(m_vec, vec_length, k, n))


def spmm_slab(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix, output_matrix,
              workspace=None, stream=None):
    """wmmaSpmm on the schedule that stages the dense operand in LDS once per block of eight vector rows
    (`vs_wmma_spmm_f16_slab`; k % 8 == 0, fp16 output).  workspace: a device tensor of at least
    `spmm_slab_workspace_bytes(...)` bytes, or None to allocate one for the call.  Returns output_matrix."""
    need = spmm_slab_workspace_bytes(m_vec, vec_length, k, n)
    if workspace is None and need > 0:
        workspace = torch.empty(need, dtype=torch.uint8, device=output_matrix.device)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    st = _lib.lib().vs_wmma_spmm_f16_slab(
        m_vec, vec_length, k, n, _expect(row_indices, torch.int32, "row_indices"),
        _expect(row_offsets, torch.int32, "row_offsets"), _expect(column_indices, torch.int32, "column_indices"),
        _expect(values, torch.float16, "values"), _expect(rhs_matrix, torch.float16, "rhs_matrix"),
        _expect(output_matrix, torch.float16, "output_matrix"), _ptr(workspace), ws_bytes, _stream(stream))
    if st:
        _lib.check(st, "vs_wmma_spmm_f16_slab")
    return output_matrix


class sddmm:
    """Namespace ``sddmm`` of the reference: D = (A[m x k] * B[n x k]^T) sampled on a column-vector CSR mask."""

    @staticmethod
    def wmmaSddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                  output_values, vec_length, stream=None, algorithm=1):
        """MFMA path (reference: src/wmma_sddmm.cu:3190-3202)."""
        return _sddmm("vs_wmma_sddmm_f16", m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                      lhs_matrix, rhs_matrix, output_values, vec_length, stream, algorithm)

    @staticmethod
    def cudaSddmm(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                  output_values, vec_length, stream=None):
        """Cross-lane dot-product path (reference: src/cuda_sddmm.cu:1295-1331)."""
        return _sddmm("vs_cuda_sddmm_f16", m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices,
                      lhs_matrix, rhs_matrix, output_values, vec_length, stream)


def _stride(t, batch):
    """Element stride between consecutive problems of a [batch, ...] tensor (0 when shared)."""
    if batch == 1 or t.dim() < 3:
        return 0
    return t.stride(0)


def spmm_batched(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, values, rhs_matrix,
                 output_matrix, kernel="wmma", stream=None, nonzeros_vec=-1, longest_row_vec=-1, long_rows=-1):
    """`batch` SpMMs sharing one pattern in one launch.

    values: [batch, nnz_vec, V] (or [nnz_vec, V] shared), rhs_matrix: [batch, n, k] (or [n, k] shared),
    output_matrix: [batch, m, k], all fp16 and contiguous in their trailing dimensions.
    long_rows >= 0 (MFMA path): row_indices orders the rows by length, longest first, and its first long_rows
    entries are the rows of more than LONG_ROW_VECTORS nonzero vectors (vs_wmma_spmm_f16_batched_sorted).
    """
    batch = output_matrix.shape[0]
    for t, nm in ((values, "values"), (rhs_matrix, "rhs_matrix"), (output_matrix, "output_matrix")):
        _expect_batched(t, torch.float16, nm)
    entry = "vs_wmma_spmm_f16_batched" if kernel == "wmma" else "vs_cuda_spmm_f16_batched"
    hints = [int(nonzeros_vec), int(longest_row_vec)]
    if kernel == "wmma" and long_rows >= 0:
        entry = "vs_wmma_spmm_f16_batched_sorted"
        hints.append(int(long_rows))
    st = getattr(_lib.lib(), entry)(batch, m_vec, vec_length, k, n, *hints,
                                    _ptr(row_indices), _ptr(row_offsets), _ptr(column_indices), _ptr(values), _stride(values, batch), _ptr(rhs_matrix),
                                    _stride(rhs_matrix, batch), _ptr(output_matrix), _stride(output_matrix, batch),
                                    _stream(stream))
    _lib.check(st, entry)
    return output_matrix


def spmm_softmax_batched(m_vec, vec_length, k, n, row_indices, row_offsets, column_indices, scores, rhs_matrix,
                         output_matrix, scale=1.0, stream=None, nonzeros_vec=-1, longest_row_vec=-1):
    """out[b] = softmax_row(scale * scores[b]) @ rhs_matrix[b] in one launch (softmax fused into SpMM)."""
    if output_matrix.dim() == 2:
        output_matrix = output_matrix.unsqueeze(0)
    batch = output_matrix.shape[0]
    for t, nm in ((scores, "scores"), (rhs_matrix, "rhs_matrix"), (output_matrix, "output_matrix")):
        _expect_batched(t, torch.float16, nm)
    st = _lib.lib().vs_wmma_spmm_softmax_f16_batched(
        batch, m_vec, vec_length, k, n, int(nonzeros_vec), int(longest_row_vec), _ptr(row_indices), _ptr(row_offsets),
        _ptr(column_indices), _ptr(scores),
        _stride(scores, batch), _ptr(rhs_matrix), _stride(rhs_matrix, batch), _ptr(output_matrix),
        _stride(output_matrix, batch), float(scale), _stream(stream))
    _lib.check(st, "vs_wmma_spmm_softmax_f16_batched")
    return output_matrix


def sparse_attention(m_vec, vec_length, n, row_indices, row_offsets, col_indices, q, k, v, out=None, scale=None,
                     stream=None, rows_per_workgroup=0, plan=None):
    """Single-launch fixed-mask attention: out = softmax(scale * mask(q k^T)) v.

    q: [heads, m, d_qk], k: [heads, n, d_qk], v: [heads, n, d_v] (or 2-D for one head), fp16.
    rows_per_workgroup: 0 / 1 = one vector row per workgroup; >= 2 = union-gather kernel for masks whose
    neighbouring rows share columns, optionally (and much faster) with a plan from `sparse_attention_plan`.
    """
    if q.dim() == 2:
        q, k, v = q.unsqueeze(0), k.unsqueeze(0), v.unsqueeze(0)
        if out is not None:
            out = out.unsqueeze(0)
    heads, m, d_qk = q.shape
    d_v = v.shape[2]
    if scale is None:
        scale = 1.0 / float(d_qk) ** 0.5
    if out is None:
        out = torch.empty((heads, m, d_v), dtype=torch.float16, device=q.device)
    for t, nm in ((q, "q"), (k, "k"), (v, "v"), (out, "out")):
        _expect_batched(t, torch.float16, nm)
    st = _lib.lib().vs_sparse_attention_f16(heads, m_vec, vec_length, n, d_qk, d_v, _ptr(row_indices),
                                            _ptr(row_offsets), _ptr(col_indices), _ptr(q), _stride(q, heads),
                                            _ptr(k), _stride(k, heads), _ptr(v), _stride(v, heads), _ptr(out),
                                            _stride(out, heads), float(scale), int(rows_per_workgroup),
                                            _ptr(plan), 0 if plan is None else plan.numel() * plan.element_size(),
                                            _stream(stream))
    _lib.check(st, "vs_sparse_attention_f16")
    return out


def sddmm_batched(m_vec, k, n, nonzeros_vec, row_indices, row_offsets, col_indices, lhs_matrix, rhs_matrix,
                  output_values, vec_length, kernel="wmma", stream=None, algorithm=1):
    """`batch` SDDMMs sharing one mask in one launch.

    lhs_matrix: [batch, m, k], rhs_matrix: [batch, n, k], output_values: [batch, nnz_vec, V], fp16.
    """
    batch = output_values.shape[0]
    for t, nm in ((lhs_matrix, "lhs_matrix"), (rhs_matrix, "rhs_matrix"), (output_values, "output_values")):
        _expect_batched(t, torch.float16, nm)
    args = [batch, m_vec, k, n, nonzeros_vec, _ptr(row_indices), _ptr(row_offsets), _ptr(col_indices),
            _ptr(lhs_matrix), _stride(lhs_matrix, batch), _ptr(rhs_matrix), _stride(rhs_matrix, batch),
            _ptr(output_values), _stride(output_values, batch), vec_length, _stream(stream)]
    if kernel == "wmma":
        entry = "vs_wmma_sddmm_f16_batched"
        args.append(algorithm)
    else:
        entry = "vs_cuda_sddmm_f16_batched"
    _lib.check(getattr(_lib.lib(), entry)(*args), entry)
    return output_values


def sparse_softmax(m_vec, vec_length, row_indices, row_offsets, values_in, values_out=None, scale=1.0,
                   stream=None):
    """Row-wise softmax(scale * x) over each scalar row's nonzeros, [nnz_vec, V] or [batch, nnz_vec, V]."""
    if values_out is None:
        values_out = torch.empty_like(values_in)
    _expect_batched(values_in, torch.float16, "values_in")
    _expect_batched(values_out, torch.float16, "values_out")
    batch = values_in.shape[0] if values_in.dim() == 3 else 1
    st = _lib.lib().vs_sparse_softmax_f16(batch, m_vec, vec_length, _ptr(row_indices), _ptr(row_offsets),
                                          _ptr(values_in), _stride(values_in, batch), _ptr(values_out),
                                          _stride(values_out, batch), float(scale), _stream(stream))
    _lib.check(st, "vs_sparse_softmax_f16")
    return values_out


def _expect_batched(t, dtype, name):
    if t.dtype != dtype:
        raise TypeError("%s must be %s, got %s" % (name, dtype, t.dtype))
    if not t.is_cuda:
        raise ValueError("%s must live in device memory" % name)
    inner = t[0] if t.dim() == 3 else t
    if not inner.is_contiguous():
        raise ValueError("%s must be contiguous in its trailing dimensions" % name)


def sparse_attention_plan(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup, row_offsets, col_indices, stream=None):
    """Analyse a fixed mask once for the union-gather kernel: returns the plan (a device byte tensor) that
    `sparse_attention(..., rows_per_workgroup=..., plan=...)` reads instead of rebuilding it per launch."""
    size = _lib.lib().vs_sparse_attention_plan_bytes(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup)
    if size <= 0:
        raise _lib.VSparseError("vs_sparse_attention_plan_bytes: shape not supported by the union kernel")
    plan = torch.empty(size, dtype=torch.uint8, device=row_offsets.device)
    st = _lib.lib().vs_sparse_attention_plan(m_vec, vec_length, n, d_qk, d_v, rows_per_workgroup, _ptr(row_offsets),
                                             _ptr(col_indices), _ptr(plan), size, _stream(stream))
    _lib.check(st, "vs_sparse_attention_plan")
    return plan


class SparseAttention:
    """One fixed-mask sparse attention layer: SDDMM (QK^T on the mask) -> row softmax -> SpMM (P V).

    The mask is a column-vector CSR pattern over [seq, seq] shared by all heads.  `forward` runs the layer as
    one launch (scores and probabilities never leave the chip), as two (SDDMM, then the SpMM with the softmax
    folded in) or as the three operators, one batched launch each, chained on one stream with no host
    synchronisation and no re-layout (the SDDMM output layout is the SpMM value layout); by default it
    picks the faster of the first two for the mask, the head widths and the head count.
    """

    def __init__(self, mask, device="cuda", sort=True):
        self.prob = DeviceProblem(mask, sort=sort, device=device)
        self.mask = mask
        self._plans = {}
        self._rows = {}

    def _parts_route_fits(self, d_v, heads):
        """The SpMM of the three-operator route on row parts takes less than 2 GiB of partial tiles (the limit of
        vs_wmma_spmm_f16_row_parts); larger masks or more heads take the other routes."""
        parts = self.prob.row_parts(512)[0]
        return spmm_row_parts_workspace_bytes(self.prob.vec_length, d_v, parts.n_split, parts.parts_max,
                                              batch=heads) < 2 ** 31

    def union_rows(self, d_qk, d_v, heads=16):
        """Rows per workgroup for the single-launch kernel with these head widths and head count (cached)."""
        key = (int(d_qk), int(d_v), int(heads))
        if key not in self._rows:
            self._rows[key] = self._union_rows(self.mask, *key)
        return self._rows[key]

    def plan(self, d_qk, d_v, heads=16):
        """Device plan of the union kernel for these head widths (built on first use), or None."""
        rows = self.union_rows(d_qk, d_v, heads)
        if rows < 2:
            return None
        key = (int(d_qk), int(d_v), rows)
        if key not in self._plans:
            p = self.prob
            self._plans[key] = sparse_attention_plan(p.m_vec, p.vec_length, p.n, key[0], key[1], rows,
                                                     p.row_offsets, p.column_indices)
        return self._plans[key]

    # Cost model of the row choice below, in us per layer, fitted on MI355X (2..64 heads x 1024..16384 rows, band,
    # band + strided and uniform random masks of 8..960 nonzero vectors per row).  A streamed workgroup (128
    # scalar rows) alone on its CU takes 3.5 + 0.0235 * (union columns), two sharing a CU 7 + 0.04 * columns
    # each; heads wider than 64 run one workgroup per CU at 6 + 0.037 * columns.  SDDMM followed by the
    # softmax-fused SpMM takes 6 us plus, per 16 heads, a per vector row and b per nonzero vector (ns, by vector
    # length; 1.3 a and 1.7 b for the wider heads).
    _TWO_LAUNCH_NS = {8: (19.5, 0.35), 4: (15.6, 0.29), 2: (13.2, 0.25), 1: (12.0, 0.22)}

    @staticmethod
    def _union_rows(mask, d_qk, d_v, heads=16):
        """Vector rows per workgroup for the single-launch kernel: workgroups of eight waves (128 scalar rows,
        which stream the union of their columns through LDS) when every block's distinct columns stay within
        the library's capacity for this shape and the cost model above puts the launch below the two-launch
        path, else 1 (the two launches, any mask).

        The streamed kernel pays per union column, the two launches per nonzero: measured (us per layer, 16
        heads x 4096, d = 64) a +-4 band takes 12.5 against 18.6 (V = 8) and 12.7 against 63.7 (V = 1), a
        uniform random mask at 99.8 % sparsity 10.8 against 17.8, at 99.5 % 20.8 against 19.3, at 98 % 54.8
        against 31.3 (V = 8).  A launch of few workgroups is bound by the longest of them (2 heads x 2048,
        V = 1, 98 % random: 47.9 us streamed against 10.6 us), hence the head count.  Smaller workgroups (the
        kernel that holds the union at once) were slower than eight waves on every mask where both apply
        (+-4 .. +-64 bands: four waves 17.6 .. 27.1 us, eight waves 12.5 .. 15.3 us), so they are left to
        callers that ask for them."""
        ro, ci = mask.row_offsets, mask.column_indices
        if mask.m_vec == 0 or mask.nnz_vec == 0:
            return 1
        used = ctypes.c_int(0)
        want = 128 // mask.vec_length
        cap = _lib.lib().vs_sparse_attention_union_capacity(mask.vec_length, mask.n, d_qk, d_v, want, 1,
                                                            ctypes.addressof(used))
        rows = used.value
        if cap <= 0 or rows != want:
            return 1
        unions = [np.unique(ci[ro[first]:ro[min(first + rows, mask.m_vec)]]).size
                  for first in range(0, mask.m_vec, rows)]
        longest = max(unions)
        if longest > cap:
            return 1
        wide = d_qk > 64 or d_v > 64
        if wide:
            alone = 6.0 + 0.037 * longest
            busy = sum(6.0 + 0.037 * u for u in unions) * heads / 256.0
        else:
            alone = 3.5 + 0.0235 * longest
            busy = sum(7.0 + 0.04 * u for u in unions) * heads / 512.0
        per_row, per_nonzero = SparseAttention._TWO_LAUNCH_NS[mask.vec_length]
        if wide:
            per_row, per_nonzero = 1.3 * per_row, 1.7 * per_nonzero
        two_launches = 6.0 + (per_row * mask.m_vec + per_nonzero * mask.nnz_vec) * (heads / 16.0) * 1e-3
        return rows if max(alone, busy) <= two_launches else 1

    def forward(self, q, k, v, scale=None, kernel="wmma", stream=None, scores=None, out=None, fused=None):
        """q, k, v: fp16 [heads, seq, d] on the device.  Returns fp16 [heads, seq, d].

        fused: "parts" runs the three operators on the dispatch list of row parts (masks with rows far longer than
        the rest, e.g. global tokens); "layer" runs the whole layer in one launch with scores and probabilities kept in LDS; True
        folds only the softmax into the SpMM launch (two launches, raw scores go through memory); False runs
        the three operators one after the other.  Default on the MFMA path: "layer" when the cost model of
        `_union_rows` puts the streamed union kernel ahead (banded, blocky, strided and very sparse masks: 1.5-15x
        faster than the alternatives), else True - on masks without shared columns the single launch gathers
        K / V rows per row and is 10-60 % slower than the two launches (16 heads x 4096, uniform random masks,
        90-98 % sparse, V = 1..8).
        """
        p = self.prob
        heads, seq, d = q.shape
        if scale is None:
            scale = 1.0 / float(d) ** 0.5
        if scores is None:
            scores = torch.empty((heads, p.nnz_vec, p.vec_length), dtype=torch.float16, device=q.device)
        if out is None:
            out = torch.empty((heads, seq, v.shape[2]), dtype=torch.float16, device=q.device)
        if fused is None:
            if kernel != "wmma":
                fused = False
            elif (d % 8 == 0 and v.shape[2] % 4 == 0 and p.n * v.shape[2] < 2 ** 31 and p.row_parts(0)[0].n_split > 0
                  and self._parts_route_fits(v.shape[2], heads)):
                # rows far longer than the rest - global tokens: the three operators on the dispatch list of row
                # parts (16 heads x 4096, d = 64, a +-32..128 band with 64-256 global tokens: 72-119 us against
                # 145-160 us in one launch and 280-295 us for SDDMM + softmax-fused SpMM on whole rows)
                fused = "parts"
            else:
                fused = "layer" if self.union_rows(q.shape[2], v.shape[2], heads) >= 2 else True
        if fused == "parts":
            p.sddmm_row_parts(q, k, out=scores, stream=stream)
            p.softmax_row_parts(scores, scale=scale, stream=stream)
            return p.spmm_row_parts(v, out=out, stream=stream, limit_vec=512, values=scores)
        if fused == "layer":
            return sparse_attention(p.m_vec, p.vec_length, p.n, p.row_indices, p.row_offsets, p.column_indices,
                                    q, k, v, out=out, scale=scale, stream=stream,
                                    rows_per_workgroup=self.union_rows(q.shape[2], v.shape[2], heads),
                                    plan=self.plan(q.shape[2], v.shape[2], heads))
        sddmm_batched(p.m_vec, d, p.n, p.nnz_vec, p.row_indices, p.row_offsets, p.column_indices, q, k, scores,
                      p.vec_length, kernel=kernel, stream=stream)
        if fused:
            return spmm_softmax_batched(p.m_vec, p.vec_length, v.shape[2], p.n, p.row_indices, p.row_offsets,
                                        p.column_indices, scores, v, out, scale, stream=stream,
                                        nonzeros_vec=p.nnz_vec, longest_row_vec=p.longest_row_vec)
        sparse_softmax(p.m_vec, p.vec_length, p.row_indices, p.row_offsets, scores, scores, scale, stream=stream)
        spmm_batched(p.m_vec, p.vec_length, v.shape[2], p.n, p.row_indices, p.row_offsets, p.column_indices,
                     scores, v, out, kernel=kernel, stream=stream, nonzeros_vec=p.nnz_vec,
                     longest_row_vec=p.longest_row_vec)
        return out


def IdentityRowSwizzle(rows):
    """include/bm_test_utils.h:196-198 through the C ABI (host arrays)."""
    out = np.empty(rows, dtype=np.int32)
    _lib.lib().vs_identity_row_swizzle(rows, out.ctypes.data)
    return out


def SortedRowSwizzle(rows, row_offsets):
    """include/bm_test_utils.h:200-215 through the C ABI (host arrays)."""
    ro = np.ascontiguousarray(row_offsets, dtype=np.int32)
    out = np.empty(rows, dtype=np.int32)
    _lib.lib().vs_sorted_row_swizzle(rows, ro.ctypes.data, out.ctypes.data)
    return out


class RowParts:
    """The dispatch list of `vs_spmm_row_parts` for a pattern: rows of more than `limit_vec` nonzero vectors (0 =
    the library's default) cut into parts that get a workgroup each, everything ordered longest first.  Host arrays in,
    host array out (`slots`, int32 [n_slots][4]); `n_split`, `parts_max`, `longest_part_vec` as the C function
    returns them."""

    def __init__(self, m_vec, row_offsets, limit_vec=0):
        import ctypes
        ro = np.ascontiguousarray(row_offsets, dtype=np.int32)
        step = 1152 if limit_vec <= 0 else (limit_vec + 63) // 64 * 64   # (the default limit is 1152 at least)
        room = m_vec + 2 * (int(ro[m_vec] if m_vec > 0 else 0) // step) + 64
        counts = [ctypes.c_int(0) for _ in range(4)]
        for attempt in range(2):
            slots = np.empty((room, 4), dtype=np.int32)
            st = _lib.lib().vs_spmm_row_parts(m_vec, ro.ctypes.data, limit_vec, slots.ctypes.data, room,
                                              *[ctypes.addressof(c) for c in counts])
            if st == 801 and attempt == 0 and counts[0].value + counts[1].value > room:
                room = counts[0].value + counts[1].value   # (the counts say what the list needs)
                continue
            break
        if st:
            _lib.check(st, "vs_spmm_row_parts")
        self.n_slots, self.n_split, self.parts_max, self.longest_part_vec = (c.value for c in counts)
        self.slots = np.ascontiguousarray(slots[:self.n_slots + self.n_split])  # (one entry per split row behind the list)


def spmm_row_parts_workspace_bytes(vec_length, k, n_split, parts_max, batch=1):
    return int(_lib.lib().vs_wmma_spmm_row_parts_workspace_bytes(batch, vec_length, k, n_split, parts_max))


def spmm_row_parts(vec_length, k, n, parts, slots, nonzeros_vec, column_indices, values, rhs_matrix, output_matrix,
                   workspace=None, stream=None):
    """wmmaSpmm driven by a dispatch list of row parts (`parts`: a RowParts, `slots`: its list as a device int32
    tensor).  workspace: a device tensor of at least spmm_row_parts_workspace_bytes(...) bytes, zero-filled before
    its first use, or None when no row is split.  A leading batch dimension on output_matrix ([batch, m, k]) runs
    that many problems on the shared pattern; values / rhs_matrix with the same leading dimension are per problem,
    without it shared.  Returns output_matrix."""
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    batch = output_matrix.shape[0] if output_matrix.dim() == 3 else 1
    per_problem = lambda t, dims: _stride(t, batch)
    st = _lib.lib().vs_wmma_spmm_f16_row_parts(
        batch, vec_length, k, n, parts.n_slots, _expect(slots, torch.int32, "slots"), parts.n_split, parts.parts_max,
        nonzeros_vec, parts.longest_part_vec, _expect(column_indices, torch.int32, "column_indices"),
        _expect(values, torch.float16, "values"), per_problem(values, 2),
        _expect(rhs_matrix, torch.float16, "rhs_matrix"), per_problem(rhs_matrix, 2),
        _expect(output_matrix, torch.float16, "output_matrix"), per_problem(output_matrix, 2), _ptr(workspace), ws_bytes,
        _stream(stream))
    if st:
        _lib.check(st, "vs_wmma_spmm_f16_row_parts")
    return output_matrix


def sddmm_row_parts(k, n, parts, slots, nonzeros_vec, col_indices, lhs_matrix, rhs_matrix, output_values, vec_length,
                    stream=None):
    """wmmaSddmm driven by a dispatch list of row parts (`parts`: a RowParts, `slots`: its list as a device int32
    tensor).  A leading batch dimension on output_values ([batch, nnz_vec, V]) runs that many problems on the shared
    mask; lhs_matrix / rhs_matrix with the same leading dimension are per problem, without it shared.  Returns
    output_values."""
    batch = output_values.shape[0] if output_values.dim() == 3 else 1
    per_problem = lambda t, dims: _stride(t, batch)
    st = _lib.lib().vs_wmma_sddmm_f16_row_parts(
        batch, k, n, parts.n_slots, _expect(slots, torch.int32, "slots"), nonzeros_vec,
        _expect(col_indices, torch.int32, "col_indices"), _expect(lhs_matrix, torch.float16, "lhs_matrix"),
        per_problem(lhs_matrix, 2), _expect(rhs_matrix, torch.float16, "rhs_matrix"), per_problem(rhs_matrix, 2),
        _expect(output_values, torch.float16, "output_values"), per_problem(output_values, 2), vec_length, _stream(stream))
    if st:
        _lib.check(st, "vs_wmma_sddmm_f16_row_parts")
    return output_values


def sparse_softmax_row_parts(vec_length, parts, slots, values_in, values_out=None, scale=1.0, workspace=None,
                             stream=None):
    """Row-wise softmax of scale * values driven by a dispatch list of row parts (`parts`: a RowParts, `slots`: its
    list as a device int32 tensor); values [nnz_vec, V] or [batch, nnz_vec, V].  workspace: a device tensor of at
    least sparse_softmax_row_parts_workspace_bytes(...) bytes (None when no row is split).  Returns values_out
    (values_in when None: in place)."""
    if values_out is None:
        values_out = values_in
    batch = values_in.shape[0] if values_in.dim() == 3 else 1
    stride = lambda t: _stride(t, batch)
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    st = _lib.lib().vs_sparse_softmax_f16_row_parts(
        batch, vec_length, parts.n_slots, _expect(slots, torch.int32, "slots"), parts.n_split, parts.parts_max,
        _expect(values_in, torch.float16, "values_in"), stride(values_in),
        _expect(values_out, torch.float16, "values_out"), stride(values_out), float(scale), _ptr(workspace), ws_bytes,
        _stream(stream))
    if st:
        _lib.check(st, "vs_sparse_softmax_f16_row_parts")
    return values_out


def sparse_softmax_row_parts_workspace_bytes(vec_length, n_split, parts_max, batch=1):
    return int(_lib.lib().vs_sparse_softmax_row_parts_workspace_bytes(batch, vec_length, n_split, parts_max))


LONG_ROW_VECTORS = 512  # rows beyond this are "long" for vs_wmma_spmm_f16_batched_sorted (eight 64-vector blocks)


def split_rows_pays(m_vec, nonzeros_vec, longest_row_vec):
    """Whether the split-row SpMM schedule is expected to beat the row-per-workgroup one with row-length hints.
    Measured at N = 256, V = 8, rows of up to 4608 vectors, 64 to 2048 vector rows: a row of 25 or more mean lengths
    (one dense row among rows of a hundred) holds its workgroups for 11.1-12.0 us on up to 1024 rows where the split
    schedule needs 9.8-11.4 us; on 2048 rows the hinted schedule is ahead (12.5 against 14.9 us), as it is on milder
    skew (Pareto or log-normal lengths, longest row 6 to 18 mean lengths: 1024 Pareto rows 13.4 against 16.9 us) and
    on uniform or binomial lengths (by 1.6 to 2 times).  (Rows in parts, DeviceProblem.spmm_row_parts, are ahead
    of both on all of these; the rule is for callers that have a workspace but no dispatch list.)"""
    if m_vec <= 0 or m_vec > 1024 or nonzeros_vec < 8192:
        return False
    return longest_row_vec * m_vec >= 25.0 * nonzeros_vec


class DeviceProblem:
    """Device-resident operands of one SpMM / SDDMM problem (caller-owned buffers, as in BmFN)."""

    def __init__(self, pattern, sort=False, device="cuda"):
        self.pattern = pattern
        self.m_vec = pattern.m_vec
        self.vec_length = pattern.vec_length
        self.n = pattern.n
        self.nnz_vec = pattern.nnz_vec
        lengths = np.diff(pattern.row_offsets)
        self.longest_row_vec = int(lengths.max()) if lengths.size else 0
        # with the sorted swizzle the long rows are the first entries of row_indices
        self.long_rows = int(np.count_nonzero(lengths > LONG_ROW_VECTORS)) if sort else -1
        # a few rows far longer than the rest: schedules that give every row the same number of waves stall on them
        self.skewed = bool(pattern.nnz_vec >= 65536 and lengths.max() >= 8 * max(1.0, lengths.mean()))
        swz = SortedRowSwizzle(pattern.m_vec, pattern.row_offsets) if sort else IdentityRowSwizzle(pattern.m_vec)
        self.row_indices = torch.from_numpy(swz).to(device)
        self.row_offsets = torch.from_numpy(np.ascontiguousarray(pattern.row_offsets)).to(device)
        self.column_indices = torch.from_numpy(np.ascontiguousarray(pattern.column_indices)).to(device)
        self._workspace = None  # partial tiles of the split-row SpMM, allocated on first use
        self._parts = {}        # limit -> (RowParts, its list on the device, workspace), made on first use
        self.values = None
        if pattern.values is not None:
            self.values = torch.from_numpy(np.ascontiguousarray(pattern.values)).to(device)

    def row_parts(self, limit_vec=0):
        """The pattern's dispatch list of row parts (see RowParts) on the device, made once per limit."""
        if limit_vec not in self._parts:
            parts = RowParts(self.m_vec, self.pattern.row_offsets, limit_vec)
            slots = torch.from_numpy(parts.slots).to(self.column_indices.device)
            self._parts[limit_vec] = [parts, slots, None, None]   # (+ SpMM workspace, softmax workspace: on first use)
        return self._parts[limit_vec]

    def spmm_row_parts(self, rhs_matrix, out=None, stream=None, limit_vec=0, values=None):
        """SpMM (MFMA path, fp16 output) with long rows dispatched as several parts; the list and the workspace
        for the parts' partial tiles belong to this object.  values: the pattern's own by default; [batch, nnz_vec, V]
        (with rhs_matrix [batch, n, k] or [n, k]) runs a batch on the shared pattern."""
        values = self.values if values is None else values
        k = rhs_matrix.shape[-1]
        batch = values.shape[0] if values.dim() == 3 else 1
        if out is None:
            shape = (self.m_vec * self.vec_length, k) if values.dim() == 2 else (batch, self.m_vec * self.vec_length, k)
            out = torch.empty(shape, dtype=torch.float16, device=rhs_matrix.device)
        entry = self.row_parts(limit_vec)
        parts, slots = entry[0], entry[1]
        need = spmm_row_parts_workspace_bytes(self.vec_length, k, parts.n_split, parts.parts_max, batch=batch)
        if need and (entry[2] is None or entry[2].numel() < need):
            entry[2] = torch.zeros(need, dtype=torch.uint8, device=rhs_matrix.device)
        return spmm_row_parts(self.vec_length, k, self.n, parts, slots, self.nnz_vec, self.column_indices, values,
                              rhs_matrix, out, entry[2] if need else None, stream)

    def softmax_row_parts(self, values_in, values_out=None, scale=1.0, stream=None, limit_vec=512):
        """Row-wise softmax of scale * values ([nnz_vec, V] or [batch, nnz_vec, V]) with long rows normalised by
        several waves (in place by default)."""
        entry = self.row_parts(limit_vec)
        parts, slots = entry[0], entry[1]
        batch = values_in.shape[0] if values_in.dim() == 3 else 1
        need = sparse_softmax_row_parts_workspace_bytes(self.vec_length, parts.n_split, parts.parts_max, batch=batch)
        if need and (entry[3] is None or entry[3].numel() < need):
            entry[3] = torch.empty(need, dtype=torch.uint8, device=values_in.device)
        return sparse_softmax_row_parts(self.vec_length, parts, slots, values_in, values_out, scale,
                                        entry[3] if need else None, stream)

    def spmm(self, rhs_matrix, kernel="wmma", out_dtype=torch.float16, out=None, stream=None, row_length_hint=False,
             split_rows=False):
        """SpMM through the reference-shaped entry points; with row_length_hint (fp16 output only) through the
        batched entry point with batch = 1, which also takes the pattern's nonzero count and longest row and
        sizes its workgroups by the real row lengths instead of by n; with split_rows (MFMA path) on the
        schedule that cuts the nonzero range into equal pieces, with a workspace this object owns.
        split_rows=None chooses from the row lengths: rows in parts (spmm_row_parts) where the pattern has rows
        long enough to be split, else the row-length hints."""
        k = rhs_matrix.shape[1]
        if out is None:
            out = torch.empty((self.m_vec * self.vec_length, k), dtype=out_dtype, device=rhs_matrix.device)
        if split_rows is None:
            # rows in parts wherever the dispatch list splits a row (measured ahead of both other schedules on
            # Pareto lengths and on a dense row among short ones, 64 to 2048 rows; within 4 % on log-normal lengths),
            # else the row-length hints
            if kernel == "wmma" and k % 4 == 0 and out.dtype == torch.float16 and self.n * k < 2 ** 31:
                parts = self.row_parts(0)[0]
                # (the entry point addresses the partial tiles with 32-bit offsets: less than 2 GiB of them)
                if parts.n_split > 0 and spmm_row_parts_workspace_bytes(self.vec_length, k, parts.n_split,
                                                                        parts.parts_max) < 2 ** 31:
                    return self.spmm_row_parts(rhs_matrix, out=out, stream=stream)
            split_rows = False
            row_length_hint = True
        if split_rows and kernel == "wmma":
            need = spmm_workspace_bytes(self.m_vec, self.vec_length, k, self.n, self.nnz_vec)
            if self._workspace is None or self._workspace.numel() < need:
                self._workspace = torch.zeros(max(need, 16), dtype=torch.uint8, device=rhs_matrix.device)
            return spmm_split_rows(self.m_vec, self.vec_length, k, self.n, self.nnz_vec, self.row_offsets,
                                   self.column_indices, self.values, rhs_matrix, out, self._workspace, stream)
        if row_length_hint and out.dtype == torch.float16:
            spmm_batched(self.m_vec, self.vec_length, k, self.n, self.row_indices, self.row_offsets,
                         self.column_indices, self.values, rhs_matrix, out.unsqueeze(0), kernel=kernel, stream=stream,
                         nonzeros_vec=self.nnz_vec, longest_row_vec=self.longest_row_vec, long_rows=self.long_rows)
            return out
        fn = spmm.wmmaSpmm if kernel == "wmma" else spmm.cudaSpmm
        return fn(self.m_vec, self.vec_length, k, self.n, self.row_indices, self.row_offsets,
                  self.column_indices, self.values, rhs_matrix, out, stream)

    def sddmm_row_parts(self, lhs_matrix, rhs_matrix, out=None, stream=None, limit_vec=256):
        """SDDMM (MFMA path, fp16 output, k % 8 == 0) with long rows of the mask dispatched as several parts.  The
        parts have nothing to add up, so the limit is low (measured at K = 64..256 on 256 to 2048 rows of Pareto
        lengths and on a dense row among short ones: 128 to 512 vectors within 5 % of each other, 1152 20-70 % behind)."""
        k = lhs_matrix.shape[-1]   # (operands [rows, k], or [batch, rows, k] for a batch on the shared mask)
        if out is None:
            lead = (lhs_matrix.shape[0],) if lhs_matrix.dim() == 3 else ()
            out = torch.empty(lead + (self.nnz_vec, self.vec_length), dtype=torch.float16, device=lhs_matrix.device)
        parts, slots = self.row_parts(limit_vec)[:2]
        return sddmm_row_parts(k, self.n, parts, slots, self.nnz_vec, self.column_indices, lhs_matrix, rhs_matrix, out,
                               self.vec_length, stream)

    def sddmm(self, lhs_matrix, rhs_matrix, kernel="wmma", out_dtype=torch.float16, out=None, stream=None,
              algorithm=None):
        """SDDMM on the mask.  algorithm (MFMA path): 1 = a wave per (row, slot), 2 = waves split the nonzero
        range (robust to skewed row lengths), 0 = the library's choice between 1 and the fine-grained kernel (small
        masks of short vectors); None picks 2 for large, heavily skewed masks, else 0."""
        k = lhs_matrix.shape[1]
        if out is None:
            out = torch.empty((self.nnz_vec, self.vec_length), dtype=out_dtype, device=lhs_matrix.device)
        if algorithm is None:
            # skewed masks: rows in parts (ahead of the nonzero-range schedule by 25-30 % at K = 64..256, and of the
            # row kernel by 2.7-3.4 times, on Pareto lengths), where the entry point takes the shape
            if self.skewed and kernel == "wmma" and k % 8 == 0 and k > 0 and out.dtype == torch.float16:
                return self.sddmm_row_parts(lhs_matrix, rhs_matrix, out=out, stream=stream)
            algorithm = 2 if (self.skewed and k <= 256) else 0
        if kernel == "wmma":
            return sddmm.wmmaSddmm(self.m_vec, k, self.n, self.nnz_vec, self.row_indices, self.row_offsets,
                                   self.column_indices, lhs_matrix, rhs_matrix, out, self.vec_length, stream,
                                   algorithm)
        return sddmm.cudaSddmm(self.m_vec, k, self.n, self.nnz_vec, self.row_indices, self.row_offsets,
                               self.column_indices, lhs_matrix, rhs_matrix, out, self.vec_length, stream)

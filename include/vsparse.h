/*
 * vsparse — C ABI of the MI355X (gfx950) column-vector-sparse SpMM / SDDMM library.
 *
 * Every entry point is `extern "C"`, takes plain ints and raw pointers, and
 * mirrors one function of the reference's operator API (cited per function,
 * paths relative to the reference tree).  Dimension letters are the
 * reference's, not BLAS's:
 *
 *   SpMM   C[m x k] = A[m x n] * B[n x k]      m = m_vec * vec_length, A sparse
 *   SDDMM  D[nnz]   = (A[m x k] * B[n x k]^T) sampled at the mask's nonzeros
 *
 * Sparse operands are column-vector CSR: `row_offsets[m_vec + 1]`,
 * `column_indices[nnz_vec]`, and `values[nnz_vec * vec_length]` fp16 where
 * values[j * vec_length + v] is the element in scalar row i*vec_length + v,
 * column column_indices[j], of vector row i.  Dense operands are row-major
 * fp16; fp16 is IEEE binary16, passed as `void *`.
 *
 * Conventions shared by all device entry points
 *   - all array pointers are DEVICE pointers owned by the caller; nothing is
 *     retained after return; no allocation inside the library; no workspace
 *     except where an entry point takes one as an argument;
 *   - the output is fully overwritten (alpha = 1, beta = 0), including the
 *     rows of empty vector rows, and nothing outside it is written;
 *   - the launch is asynchronous on `stream` (a hipStream_t; NULL = default
 *     stream); the functions are re-entrant;
 *   - the return value is 0 on success, otherwise a hipError_t-valued int:
 *     1 (hipErrorInvalidValue) for null pointers, negative sizes,
 *     misaligned operands or unsupported vec_length / algorithm;
 *     801 (hipErrorNotSupported) for shapes the selected path cannot take;
 *     any other value is the launch error reported by the runtime.
 *     On a non-zero return no kernel was launched.
 *   - `row_indices[m_vec]` is the row swizzle: work item t processes vector
 *     row row_indices[t].  It must be a permutation of 0..m_vec-1.
 *   - `row_offsets` is ascending from 0 and row_offsets[m_vec] = nnz_vec must not
 *     exceed 2^31 - 65536: the kernels step past a row's end in 32-bit arithmetic
 *     before they clamp the position.  Column indices lie in [0, n); they need not
 *     be sorted within a row (vs_sparse_attention_f16 takes a row's columns as a set:
 *     distinct within the row).  None of this is checked: the arrays are in device
 *     memory, which the entry points do not read on the host.
 */
#ifndef VSPARSE_H
#define VSPARSE_H

#ifdef __cplusplus
extern "C" {
#endif

#define VS_SUCCESS 0
#define VS_ERROR_INVALID_VALUE 1
#define VS_ERROR_NOT_SUPPORTED 801

/* Library version, major * 10000 + minor * 100 + patch. */
int vs_version(void);

/* Short text for a status returned by the functions below. */
const char *vs_status_string(int status);

/*
 * Replaces spmm::wmmaSpmm(half in, half out) — include/wmma_spmm.cuh:15-21,
 * src/wmma_spmm.cu:400-409.  fp16 MFMA with fp32 accumulate.
 * vec_length in {2, 4, 8} as in the reference (1 is accepted as well).
 * Requirements: `values` aligned to 2*vec_length bytes, `rhs_matrix` and
 * `output_matrix` aligned to 16 bytes.  Any k >= 1 (the reference assumes
 * k % 64 == 0 and reads / writes past the operands otherwise, src/wmma_spmm.cu:362);
 * k % 4 != 0 takes a slower kernel that moves the dense operands half by half.
 */
int vs_wmma_spmm_f16(int m_vec, int vec_length, int k, int n,
                     const int *row_indices, const int *row_offsets,
                     const int *column_indices, const void *values,
                     const void *rhs_matrix, void *output_matrix, void *stream);

/* fp32-output overload of the same operator — include/wmma_spmm.cuh:7-13, src/wmma_spmm.cu:388-397. */
int vs_wmma_spmm_f16_f32out(int m_vec, int vec_length, int k, int n,
                            const int *row_indices, const int *row_offsets,
                            const int *column_indices, const void *values,
                            const void *rhs_matrix, float *output_matrix, void *stream);

/*
 * The same operator (spmm::wmmaSpmm, include/wmma_spmm.cuh:15-21 and :7-13) on a schedule that balances
 * skewed row lengths across the whole chip, which the reference's SortedRowSwizzle
 * (include/bm_test_utils.h:200-215) only approximates by reordering whole rows: the nonzero range is cut
 * into equal runs, one wave per (run, column tile) and eight runs per workgroup; a row that crosses run
 * boundaries is computed in segments whose fp32 partial tiles are added in ascending order - inside a
 * workgroup through LDS, across workgroups through `workspace` by whichever wave brings a row's last part (one
 * launch, nobody waits, no atomics on the output; deterministic; the result does not depend on row_indices, which may be null and is ignored).
 * nonzeros_vec must equal row_offsets[m_vec] (the host cannot read it from device memory).
 * workspace: device memory, 16-byte aligned, workspace_bytes long, owned by the caller, ZERO-FILLED before its
 * first use: it starts with arrival counters that every call finds at zero and leaves at zero (so no call
 * spends a launch on clearing them); the rest is undefined before and after.  The counters' area (1/128 of the
 * workspace) depends on workspace_bytes alone, so one workspace serves problems of different shapes one after
 * the other as long as it is always passed with the same size.  Not shared between calls that may
 * overlap.  (Option "spmm_flat_launches" = 2 adds the parts in a second launch instead and uses no counters.)  vs_wmma_spmm_workspace_bytes() returns the
 * size that lets the library pick its preferred run length (0 when one workgroup takes everything); a smaller
 * workspace - even none - is accepted and makes the runs longer (fewer waves, same results up to the
 * order of the fp32 summation).  Requires k % 4 == 0 (else 801); alignment as vs_wmma_spmm_f16.  Faster than vs_wmma_spmm_f16 when
 * a few rows hold a large share of the nonzeros; slower on uniform rows.
 */
long long vs_wmma_spmm_workspace_bytes(int m_vec, int vec_length, int k, int n, int nonzeros_vec);
int vs_wmma_spmm_f16_ws(int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                        const int *row_indices, const int *row_offsets,
                        const int *column_indices, const void *values,
                        const void *rhs_matrix, void *output_matrix,
                        void *workspace, long long workspace_bytes, void *stream);
int vs_wmma_spmm_f16_f32out_ws(int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                               const int *row_indices, const int *row_offsets,
                               const int *column_indices, const void *values,
                               const void *rhs_matrix, float *output_matrix,
                               void *workspace, long long workspace_bytes, void *stream);

/*
 * vs_wmma_spmm_f16_ws without the workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the partial tiles go to a
 * static device array of vs_wmma_spmm_noalloc_scratch_bytes() = 16 MiB that the library holds on every GPU it
 * runs on until the process ends.  The call allocates and frees nothing.  It has no counterpart in the
 * reference.  Same results, bit for bit, as vs_wmma_spmm_f16_ws with a workspace of that size.
 * Size limit: vec_length * (k rounded up to a multiple of 128) <= 32768 (the array must hold the partial tiles
 * of some sixty pieces beside its counters); beyond it the call returns 801 (hipErrorNotSupported) and launches nothing.
 * Every call on a GPU shares that GPU's array: calls that may overlap on one GPU (different streams, different
 * threads) race on it and must be serialised by the caller.  Nothing in the array has to be cleared between
 * calls, whatever their shapes: it starts zeroed, the arrival counters have a fixed area of their own that every
 * call leaves at zero (also a call whose nonzeros_vec is smaller than row_offsets[m_vec]: parts past nonzeros_vec are
 * neither computed nor counted), and every partial tile that is read was written by the same call.  Only calls that
 * overlapped on one GPU, or a launch that was aborted, can leave a counter behind; vs_wmma_spmm_noalloc_reset puts
 * the counters back to zero (a small kernel on `stream`, no allocation; not needed otherwise).
 * Under HIP graph capture: the address of the current GPU's array is looked up once per device, on the first call of
 * vs_wmma_spmm_noalloc_scratch_bytes() or of the entry point on that device - make that call before the capture
 * begins (the lookup is a runtime call, not a stream operation).
 */
long long vs_wmma_spmm_noalloc_scratch_bytes(void);
int vs_wmma_spmm_noalloc_reset(void *stream);
int vs_wmma_spmm_f16_noalloc(int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                             const int *row_indices, const int *row_offsets,
                             const int *column_indices, const void *values,
                             const void *rhs_matrix, void *output_matrix, void *stream);

/*
 * The same operator (spmm::wmmaSpmm, include/wmma_spmm.cuh:15-21; the tile loop of src/wmma_spmm.cu:77-90, whose
 * dense tile loader src/spmm_utils/dense_tile.h:255-259 fetches every nonzero's rhs row from memory) on a schedule that
 * stages the dense operand in LDS once per block of eight vector rows: a workgroup walks its part of the contraction in
 * windows of 128 rhs rows, loaded dense and coalesced, and every wave picks its own row's nonzeros out of the resident
 * windows.  A block of rows is spread over several parts of the contraction (so that the launch fills the chip); the
 * parts leave fp32 tiles in `workspace` and a second launch adds them in ascending order (deterministic).
 * workspace: device memory, 16-byte aligned, at least vs_wmma_spmm_slab_workspace_bytes(...) bytes (0 when the
 * rows alone fill the chip); its contents are undefined before and after, nothing has to be cleared.  Requires
 * k % 8 == 0 and n * k < 2^31, else 801.  Columns need not be sorted (sorted columns are what it is fast on).
 * Measured slower than vs_wmma_spmm_f16 on every shape of the ResNet-shaped sweep (2048 x 4608 x 256, V = 8: 31 us
 * against 15.6 us at 50 % sparsity, 28 against 5.3 us at 90 %), so no other entry point chooses it; it exists as the
 * measured form of the LDS-staged tile loop.  Option "spmm_slab_parts" (1..64, 0 = automatic) sets the number of parts
 * for the calls that follow - pass the same value to both functions.
 */
long long vs_wmma_spmm_slab_workspace_bytes(int m_vec, int vec_length, int k, int n);
int vs_wmma_spmm_f16_slab(int m_vec, int vec_length, int k, int n,
                          const int *row_indices, const int *row_offsets,
                          const int *column_indices, const void *values,
                          const void *rhs_matrix, void *output_matrix,
                          void *workspace, long long workspace_bytes, void *stream);

/*
 * Replaces spmm::cudaSpmm(half in, half out) — include/cuda_spmm.cuh:15-21,
 * src/cuda_spmm.cu:316-325.  Fine-grained path on the fp16 vector ALU
 * (mixed-precision FMA: exact fp16 x fp16 products, fp32 accumulate).  The
 * reference rounds each product to fp16 (src/spmm_utils/compute_utils.h:45);
 * that rounding is deliberately not reproduced because it alone breaks the
 * 1e-2 relative-error contract against the host loop.
 * vec_length in {1, 2, 4, 8}.  Same alignment rules; any k >= 1 (k % 8 != 0 takes a
 * slower kernel that moves the dense operands half by half).
 * Against vs_wmma_spmm_f16 on the same problems (one MI355X, k = 256, geometric means over 42 shapes per sparsity):
 * at vec_length 1 level with it - 3 % behind at 80 %, 1 % at 90 %, 2 % ahead at 95 %, 8 % ahead at 98 % - because
 * every nonzero of such a pattern brings in its own row of the dense operand and both kernels then run at the rate
 * the L2s deliver gathered rows (2048 x 4608 at 90 %: 20.2 against 20.1 us, 24 TB/s); at vec_length 2, 4, 8 it is
 * 7-15 %, 15-26 % and 24-40 % behind, since the vector ALU multiplies every value of a vector separately where an
 * MFMA tile takes up to sixteen rows for the price of one.
 */
int vs_cuda_spmm_f16(int m_vec, int vec_length, int k, int n,
                     const int *row_indices, const int *row_offsets,
                     const int *column_indices, const void *values,
                     const void *rhs_matrix, void *output_matrix, void *stream);

/* fp32-output overload — include/cuda_spmm.cuh:7-13, src/cuda_spmm.cu:304-313. */
int vs_cuda_spmm_f16_f32out(int m_vec, int vec_length, int k, int n,
                            const int *row_indices, const int *row_offsets,
                            const int *column_indices, const void *values,
                            const void *rhs_matrix, float *output_matrix, void *stream);

/*
 * Replaces sddmm::wmmaSddmm(half in, half out) — include/wmma_sddmm.cuh:17-24,
 * src/wmma_sddmm.cu:3190-3202.  fp16 MFMA, fp32 accumulate, one rounding to
 * fp16 on store.  vec_length in {2, 4, 8} (1 accepted).  `algorithm` selects
 * among the reference's four Volta register/shuffle schedules (0..3); they
 * compute the same function, and so do the two schedules here, bit for bit:
 * 1 = a wave owns (vector row, slot) and walks that row's nonzeros, rows
 * taken in row_indices order (best for rows of similar length); 2 = the waves
 * split the nonzero range itself, whatever rows it crosses (k <= 256; row
 * lengths may be arbitrarily skewed, row_indices is not used; slower on short
 * rows and small problems).  0 = automatic: schedule 1, except that masks of few
 * nonzeros with vec_length <= 4 - which fill a quarter of a matrix-core tile or
 * less - run on the fine-grained kernel of vs_cuda_sddmm_f16 (same function
 * within the fp32-accumulation tolerance, not the same bits).
 * 3 (the reference's timing-only hardware
 * simulation, whose results are wrong by design) is rejected with
 * hipErrorInvalidValue.
 * Any k >= 0; the whole of k is contracted (the reference drops k % 64).  k % 8 != 0
 * runs on the scalar-load variant of the fine-grained kernel of vs_cuda_sddmm_f16,
 * whatever the algorithm.  lhs_matrix / rhs_matrix aligned to 16 bytes when
 * k % 8 == 0 (2 bytes otherwise), output_values to 2*vec_length bytes.
 */
int vs_wmma_sddmm_f16(int m_vec, int k, int n, int nonzeros_vec,
                      const int *row_indices, const int *row_offsets,
                      const int *col_indices, const void *lhs_matrix,
                      const void *rhs_matrix, void *output_values,
                      int vec_length, void *stream, int algorithm);

/* fp32-output overload — include/wmma_sddmm.cuh:8-15, src/wmma_sddmm.cu:3175-3187. */
int vs_wmma_sddmm_f16_f32out(int m_vec, int k, int n, int nonzeros_vec,
                             const int *row_indices, const int *row_offsets,
                             const int *col_indices, const void *lhs_matrix,
                             const void *rhs_matrix, float *output_values,
                             int vec_length, void *stream, int algorithm);

/*
 * Replaces sddmm::cudaSddmm(half in, half out) — include/cuda_sddmm.cuh:16-23,
 * src/cuda_sddmm.cu:1295-1331.  Per-lane slices of the contraction with a
 * cross-lane (DPP / ds_swizzle) reduction; packed-fp16 dot products with
 * exact products and fp32 sums (the reference's fp16 rounding of each product,
 * src/cuda_sddmm.cu:382, is deliberately not reproduced).  vec_length in {1, 2, 4, 8}; any k >= 1
 * (k % 8 != 0 takes a slower scalar-load kernel).
 */
int vs_cuda_sddmm_f16(int m_vec, int k, int n, int nonzeros_vec,
                      const int *row_indices, const int *row_offsets,
                      const int *col_indices, const void *lhs_matrix,
                      const void *rhs_matrix, void *output_values,
                      int vec_length, void *stream);

/* fp32-output overload — include/cuda_sddmm.cuh:7-14, src/cuda_sddmm.cu:1281-1293. */
int vs_cuda_sddmm_f16_f32out(int m_vec, int k, int n, int nonzeros_vec,
                             const int *row_indices, const int *row_offsets,
                             const int *col_indices, const void *lhs_matrix,
                             const void *rhs_matrix, float *output_values,
                             int vec_length, void *stream);

/*
 * Batched forms: `batch` independent problems that share one sparsity pattern
 * (row_indices, row_offsets, column indices) in a single launch; problem b uses
 * each operand pointer advanced by b * its stride (strides in ELEMENTS; a stride
 * of 0 shares the operand).  batch <= 65535.  Everything else is as in the
 * unbatched entry points.  No counterpart in the reference, which launches one
 * problem per process; they exist because sparse attention runs one mask over
 * many heads (the reference only links an external sparse-transformer repository,
 * README.md:76).
 * nonzeros_vec, longest_row_vec of the SpMM forms: the number of nonzero vectors
 * of the pattern (row_offsets[m_vec]) and of its longest vector row when the caller
 * knows them, negative otherwise.  They only size the workgroups (the unbatched SpMM
 * entry points keep the reference's argument list, which does not carry them, and
 * size them by n instead): by the longest row while the launch leaves room on the
 * chip, by the mean row length once it fills it, and - when the longest row is more
 * than four times the mean - with enough waves per row that the longest one does not
 * outlast the rest of the launch.  Results do not depend on them beyond the order of
 * the fp32 summation.
 */
int vs_wmma_spmm_f16_batched(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                             int longest_row_vec, const int *row_indices, const int *row_offsets,
                             const int *column_indices,
                             const void *values, long long stride_values,
                             const void *rhs_matrix, long long stride_rhs,
                             void *output_matrix, long long stride_output, void *stream);
/*
 * vs_wmma_spmm_f16_batched for rows ordered by length, longest first (vs_sorted_row_swizzle): `long_rows` is
 * the number of leading entries of row_indices whose rows hold more than 512 nonzero vectors (negative: not
 * known, then this is vs_wmma_spmm_f16_batched).  On launches that fill the chip only those rows are shared
 * by the waves of a workgroup; every other row is served by a single wave, so that no wave is launched
 * without work - where the unsorted entry points hand every row the waves that only the long ones need.
 * A pure launch-shape hint like the other two: a wrong count, or an order that is not by length, costs
 * time (a long row behind the count is served by one wave), never correctness.  No counterpart in the
 * reference, whose sorted order only reorders the dispatch of whole rows (include/bm_test_utils.h:200-215).
 */
int vs_wmma_spmm_f16_batched_sorted(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                                    int longest_row_vec, int long_rows, const int *row_indices,
                                    const int *row_offsets, const int *column_indices, const void *values,
                                    long long stride_values, const void *rhs_matrix, long long stride_rhs,
                                    void *output_matrix, long long stride_output, void *stream);

/*
 * Rows in parts: the row swizzle of the reference (SortedRowSwizzle, include/bm_test_utils.h:200-215, which
 * reorders the dispatch of whole rows) taken one step further - a row far longer than the rest is dispatched as
 * several parts, each to a workgroup of its own, so that no workgroup is left walking one row when the rest of
 * the launch has finished.  No counterpart in the reference.
 *
 * vs_spmm_row_parts (HOST function on HOST arrays, like the swizzles): the dispatch list of a pattern.  Rows of more
 * than limit_vec nonzero vectors (0 = the library's default: 1152 or four mean row lengths, whichever is more;
 * rounded up to a multiple of 64) are cut into
 * equal parts of whole 64-vector blocks, at most 255 per row; every other row, the empty ones included, is a
 * slot of its own; the slots are ordered longest first.  slots: four ints per slot {vector row, first nonzero,
 * end, part info (0 = a whole row)}, room for max_slots of them.  Returns the number of slots, of split rows, the
 * most parts any row has and the longest slot through the pointers; VS_ERROR_NOT_SUPPORTED with the counts set
 * when max_slots is too small.  At most 32767 rows are split (the first ones in row order; longer rows past
 * that number stay whole, which costs balance, not correctness).  Behind the n_slots entries the list holds
 * one more entry per split row ({vector row, parts, 0, 0}, for the launch that adds the parts when option
 * "spmm_parts_launches" is 2): n_slots + n_split entries in all, m_vec + 2 * (nonzeros_vec / limit) + 1 always
 * suffice.
 *
 * vs_wmma_spmm_f16_row_parts: the operator of vs_wmma_spmm_f16 (same operands, same contract for the output)
 * driven by that list (all n_slots + n_split entries), copied to DEVICE memory (16-byte aligned), in place of
 * row_indices and row_offsets.
 * nonzeros_vec and longest_part_vec size the launch as the hints of vs_wmma_spmm_f16_batched do.  The parts of
 * a split row leave fp32 partial tiles in `workspace` and the workgroup that brings the last one adds them in
 * ascending order (deterministic, no atomics on the output, nobody waits).  workspace: device memory, 16-byte
 * aligned, at least vs_wmma_spmm_row_parts_workspace_bytes(batch, vec_length, k, n_split, parts_max) bytes (0 when no
 * row is split), ZERO-FILLED before its first use; its arrival counters (an area that depends on
 * workspace_bytes alone) are left at zero by every call, so it serves any sequence of calls that do not
 * overlap, whatever their shapes, as long as it is passed with the same size.  Requires k % 4 == 0,
 * n * k < 2^31 and partial tiles (batch * n_split * parts_max * vec_length * k rounded up to 128, 4 bytes each) of
 * less than 2 GiB, else 801 - raise limit_vec in that case.  batch, stride_*: as in vs_wmma_spmm_f16_batched - `batch` problems share the pattern (and
 * the list), problem b reads values + b * stride_values and rhs_matrix + b * stride_rhs and writes output_matrix +
 * b * stride_output (strides in elements, 0 = shared operand; multiples of vec_length / 8 / 8); batch = 1 with
 * strides 0 is the single operator.
 */
int vs_spmm_row_parts(int m_vec, const int *row_offsets, int limit_vec, int *slots, int max_slots, int *n_slots,
                      int *n_split, int *parts_max, int *longest_part_vec);
long long vs_wmma_spmm_row_parts_workspace_bytes(int batch, int vec_length, int k, int n_split, int parts_max);
int vs_wmma_spmm_f16_row_parts(int batch, int vec_length, int k, int n, int n_slots, const int *slots, int n_split,
                               int parts_max, int nonzeros_vec, int longest_part_vec,
                               const int *column_indices,
                               const void *values, long long stride_values,
                               const void *rhs_matrix, long long stride_rhs,
                               void *output_matrix, long long stride_output,
                               void *workspace, long long workspace_bytes, void *stream);

/*
 * The SDDMM of vs_wmma_sddmm_f16 (sddmm::wmmaSddmm, include/wmma_sddmm.cuh:17-24; same operands, same contract for
 * the output values) driven by the dispatch list of vs_spmm_row_parts in place of row_indices and row_offsets: rows
 * far longer than the rest are served as several slots, each by waves of its own - the outputs of a part are the
 * part's nonzeros, so there is nothing to add up and no workspace.  The list needs only its n_slots entries, in
 * device memory, 16-byte aligned.  Requires k % 8 == 0 (else 801).  batch, stride_*: as in vs_wmma_sddmm_f16_batched
 * (the mask and its list shared, strides in elements, multiples of 8 / 8 / vec_length).  No counterpart in the reference, whose sorted
 * order only reorders the dispatch of whole rows (include/bm_test_utils.h:200-215).
 */
int vs_wmma_sddmm_f16_row_parts(int batch, int k, int n, int n_slots, const int *slots, int nonzeros_vec,
                                const int *col_indices,
                                const void *lhs_matrix, long long stride_lhs,
                                const void *rhs_matrix, long long stride_rhs,
                                void *output_values, long long stride_output,
                                int vec_length, void *stream);

int vs_cuda_spmm_f16_batched(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                             int longest_row_vec, const int *row_indices, const int *row_offsets,
                             const int *column_indices,
                             const void *values, long long stride_values,
                             const void *rhs_matrix, long long stride_rhs,
                             void *output_matrix, long long stride_output, void *stream);
int vs_wmma_sddmm_f16_batched(int batch, int m_vec, int k, int n, int nonzeros_vec,
                              const int *row_indices, const int *row_offsets,
                              const int *col_indices,
                              const void *lhs_matrix, long long stride_lhs,
                              const void *rhs_matrix, long long stride_rhs,
                              void *output_values, long long stride_output,
                              int vec_length, void *stream, int algorithm);
int vs_cuda_sddmm_f16_batched(int batch, int m_vec, int k, int n, int nonzeros_vec,
                              const int *row_indices, const int *row_offsets,
                              const int *col_indices,
                              const void *lhs_matrix, long long stride_lhs,
                              const void *rhs_matrix, long long stride_rhs,
                              void *output_values, long long stride_output,
                              int vec_length, void *stream);

/*
 * Row-wise softmax over the nonzeros of each SCALAR row of a column-vector CSR
 * matrix, on the [nnz_vec][vec_length] fp16 value layout SDDMM writes and SpMM
 * reads:  out = softmax_row(scale * in), computed in fp32.  `values_out` may
 * equal `values_in`.  Batched like the entry points above (batch = 1 and zero
 * strides for a single problem).  The reference does not ship this operator (it
 * includes Sputnik's sparse_softmax.h, include/sputnik.h:22, from an external
 * library); it is the middle step of SDDMM -> softmax -> SpMM sparse attention.
 */
int vs_sparse_softmax_f16(int batch, int m_vec, int vec_length,
                          const int *row_indices, const int *row_offsets,
                          const void *values_in, long long stride_in,
                          void *values_out, long long stride_out,
                          float scale, void *stream);

/*
 * vs_sparse_softmax_f16 driven by the dispatch list of vs_spmm_row_parts in place of row_indices and row_offsets
 * (its n_slots entries, in device memory, 16-byte aligned): a row far longer than the rest - a global token of an
 * attention mask - is normalised by as many waves as it has parts instead of by one.  The parts of a split row
 * leave a (maximum, sum) pair per scalar row in `workspace` (8-byte aligned, at least
 * vs_sparse_softmax_row_parts_workspace_bytes(...) bytes, 0 when no row is split; no need to clear it), a second
 * launch combines them in ascending order and normalises.  in == out is allowed.  No counterpart in the reference.
 */
long long vs_sparse_softmax_row_parts_workspace_bytes(int batch, int vec_length, int n_split, int parts_max);
int vs_sparse_softmax_f16_row_parts(int batch, int vec_length, int n_slots, const int *slots, int n_split,
                                    int parts_max, const void *values_in, long long stride_in,
                                    void *values_out, long long stride_out, float scale,
                                    void *workspace, long long workspace_bytes, void *stream);

/*
 * Softmax fused into SpMM:  out = softmax_row(scale * scores) * rhs_matrix, where `scores` has the
 * layout of `values` (for example the raw output of SDDMM).  Equivalent to vs_sparse_softmax_f16
 * followed by vs_wmma_spmm_f16_batched without writing the probabilities to memory: the kernel finds
 * each scalar row's maximum, exponentiates while staging the sparse operand and divides the
 * accumulated tile by the row sum.  Same requirements as vs_wmma_spmm_f16_batched.  No counterpart in
 * the reference (see vs_sparse_softmax_f16).
 */
int vs_wmma_spmm_softmax_f16_batched(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                                     int longest_row_vec, const int *row_indices, const int *row_offsets,
                                     const int *column_indices,
                                     const void *scores, long long stride_scores,
                                     const void *rhs_matrix, long long stride_rhs,
                                     void *output_matrix, long long stride_output,
                                     float scale, void *stream);

/*
 * One fixed-mask sparse attention layer in a single launch:
 *     out[b] = softmax_row(scale * (q[b] k[b]^T sampled on the mask)) v[b]
 * q: [m_vec*vec_length, d_qk], k: [n, d_qk], v: [n, d_v], out: [m_vec*vec_length, d_v], all fp16
 * row-major; the mask is a column-vector CSR pattern over [m, n] shared by the batch (heads).
 * Scores and probabilities stay in LDS (never written to memory); rows of any length are handled with
 * a running maximum / sum over chunks of the row.  Requirements: d_qk % 8 == 0, d_qk <= 128;
 * d_v % 4 == 0 and d_v <= 64, or d_v % 8 == 0 and d_v <= 128; operands aligned to 16 bytes, strides
 * multiples of 8 elements.  Empty rows produce zeros.  No counterpart in the reference (it links an
 * external sparse-transformer repository, README.md:76); same result as vs_wmma_sddmm_f16_batched ->
 * vs_sparse_softmax_f16 -> vs_wmma_spmm_f16_batched up to the fp16 rounding of the intermediates.
 * rows_per_workgroup: 0 or 1 = one vector row per workgroup, K / V rows gathered from memory per row
 * (any mask); 2..128 = about that many consecutive vector rows per workgroup (rounded up to whole waves
 * of 16 scalar rows, at most 8 waves) computed as a dense tile against the union of their columns, whose
 * K / V rows are gathered once into LDS - faster when neighbouring rows share most of their columns
 * (banded, blocky, strided masks), slower on random masks, same results up to rounding; row_indices is
 * then only validated, rows are taken in their natural order.  Workgroups whose union exceeds
 * vs_sparse_attention_union_capacity() columns fall back to per-row gathers inside the same launch.
 * plan: null, or (rows_per_workgroup >= 2 only) a buffer filled by vs_sparse_attention_plan for this mask,
 * these head widths and this rows_per_workgroup: the kernel then reads every workgroup's union and row
 * masks from it instead of rebuilding them at every launch (same results up to the order of summation).
 * With a plan, workgroups of eight waves (rows_per_workgroup >= 128 / vec_length) stream their union
 * through LDS 128 columns at a time with the next columns' K / V rows already on their way, keeping the
 * running maximum and sums of flash attention: the fastest path, and one that takes unions of up to 2048
 * columns.  plan_bytes is the size of the plan buffer: it must be at least
 * vs_sparse_attention_plan_bytes() for THIS shape (else 1, hipErrorInvalidValue, and no launch), so that the
 * kernels never read past it whatever it holds.  A plan made for another shape is detected and ignored
 * (every workgroup then takes the per-row path: correct, slower).
 */
int vs_sparse_attention_f16(int batch, int m_vec, int vec_length, int n, int d_qk, int d_v,
                            const int *row_indices, const int *row_offsets, const int *col_indices,
                            const void *q, long long stride_q, const void *k, long long stride_k,
                            const void *v, long long stride_v, void *out, long long stride_out,
                            float scale, int rows_per_workgroup, const void *plan, long long plan_bytes,
                            void *stream);

/*
 * Analysis step for rows_per_workgroup >= 2 of vs_sparse_attention_f16: writes into `plan` (device memory,
 * 16-byte aligned, at least vs_sparse_attention_plan_bytes() bytes, owned by the caller) the distinct
 * columns and the row masks of every workgroup.  The mask of an attention layer is fixed, so one plan
 * serves every head, layer and step; asynchronous on `stream`, nothing is kept by the library.
 * vs_sparse_attention_plan_bytes returns 0 for shapes the union kernel does not support.
 * No counterpart in the reference.
 */
long long vs_sparse_attention_plan_bytes(int m_vec, int vec_length, int n, int d_qk, int d_v,
                                         int rows_per_workgroup);
int vs_sparse_attention_plan(int m_vec, int vec_length, int n, int d_qk, int d_v, int rows_per_workgroup,
                             const int *row_offsets, const int *col_indices, void *plan,
                             long long plan_bytes, void *stream);

/*
 * Planning helper for rows_per_workgroup >= 2 of vs_sparse_attention_f16: the number of distinct columns
 * a workgroup can take for this shape (0: shape not supported by the union kernel), and in
 * *rows_used (may be null) the vector rows per workgroup the request is rounded to.  with_plan: nonzero
 * for launches that pass a plan: up to 2048 columns for workgroups of eight waves (streamed), up to 512 for
 * smaller ones (only the K / V rows and the row masks in LDS), against up to 480 without a plan (the column
 * bitmap and the column list share the LDS); a plan also accepts a larger n.  Host only, no launch.
 * No counterpart in the reference.
 */
int vs_sparse_attention_union_capacity(int vec_length, int n, int d_qk, int d_v, int rows_per_workgroup,
                                       int with_plan, int *rows_used);

/*
 * Host helpers (HOST pointers).  Replace IdentityRowSwizzle / SortedRowSwizzle —
 * include/bm_test_utils.h:196-198 and :200-215.  The sorted swizzle orders
 * vector rows by descending length; equal lengths keep ascending row order.
 */
void vs_identity_row_swizzle(int rows, int *row_indices);
void vs_sorted_row_swizzle(int rows, const int *row_offsets, int *row_indices);

/*
 * Reports the launch shape that vs_wmma_spmm_f16 (hints negative) or the batched SpMM entry points (hints as
 * passed to them) would choose for a problem, under the calling thread's options; touches no device.  shape[0]
 * dense columns per lane (4 or 8: tiles of 64 or 128 columns), [1] 32-vector steps of gathered rows a wave keeps
 * in flight (1, 2, 4), [2] waves per workgroup (1..16), [3] blocks of a row a wave takes before another wave joins
 * in, [4] leading entries of row_indices served by a team of waves (-1: all rows), [5] 1 for the variant for dense
 * widths that are not a multiple of 4, [6] 1 for the LDS-DMA variant, [7] 1 when waves pipeline successive blocks of
 * a row.  Returns
 * VS_ERROR_INVALID_VALUE for sizes the entry points reject.  No counterpart in the reference, whose launch shape
 * is fixed (src/wmma_spmm.cu:362-378: one warp per vector row and 64-column tile).
 */
int vs_wmma_spmm_launch_shape(int batch, int m_vec, int vec_length, int k, int n, int nonzeros_vec,
                              int longest_row_vec, int long_rows, int shape[8]);

/*
 * Launch-shape tuning knobs.  vs_set_option sets the process-wide default (not
 * synchronised: set it before launching from several threads).
 * vs_set_thread_option sets the value for the calling thread only: from its first
 * call on, that thread's launches use its own copy of the options (initialised
 * from the process-wide values at that moment) until vs_clear_thread_options().
 * Launch shapes are decided on the host inside each call, so a thread can also
 * change its options between two calls on different streams - every call sees
 * exactly what its thread last set, whatever other threads do.  Two variants that measured slower on every
 * shape - four 32-vector steps in flight ("spmm_steps" = 4) and the LDS-DMA gather ("spmm_gather" = 2) - are
 * compiled only when the library is built with VS_RETIRED_VARIANTS=1; otherwise those two values return 801.  Names: "spmm_waves" (waves per workgroup, 0 = automatic),
 * "spmm_cols_per_lane" (4, 8, 0 = automatic), "spmm_steps" (32-vector steps of gathered
 * rows a wave of the MFMA SpMM keeps in flight: 1, 2, 4, 0 = automatic), "spmm_guard_waves"
 * (MFMA SpMM through the entry points that do not know the row lengths, on grids that fill the
 * chip by themselves: waves per workgroup kept for rows far longer than expected, 1 = none,
 * 0 = automatic), "spmm_blocks_per_wave" (same launches: blocks of 64 vectors a wave takes of a row before the
 * next kept wave joins in, a power of two up to 64, 0 = automatic), "spmm_teams" (vs_wmma_spmm_f16_batched_sorted: 1 = ignore the long-row count, 2 = use it on every
 * launch, 0 = where it measured faster), "spmm_pipe" (two steps in flight: 2 = a wave that takes several
 * blocks of a row requests the next block behind each multiplication, 1 = after both, 0 = automatic; same
 * bits either way),
 * "spmm_gather" (how the MFMA SpMM
 * brings the gathered rows of the dense operand to the matrix cores: 1 = through
 * registers and an in-register transpose, 2 = global -> LDS loads and transposing LDS
 * reads, k % 8 == 0 only; 0 = automatic, which is 1: 2 measured 10-18 % slower),
 * "spmm_slab_parts" (vs_wmma_spmm_f16_slab: parts of the contraction, 1..64, 0 = automatic),
 * "spmm_flat_piece" (nonzero vectors
 * per wave of the split-row SpMM, rounded up to 32, 0 = automatic), "spmm_flat_waves"
 * (its waves per workgroup, 1..16, 0 = automatic), "spmm_flat_launches" (1 = partial tiles
 * added inside the launch, 2 = by a second launch, 0 = automatic), "spmm_parts_launches" (rows in
 * parts: 1 = the parts of a split row meet inside the launch, 2 = a second launch adds them, 0 = automatic -
 * the second launch on small problems; same bits either way), "spmm_flat_shared" (1 = every
 * row segment of the split-row SpMM starts a 32-vector step of its own, 2 = consecutive rows share
 * steps, 0 = automatic), "sddmm_slots" (waves per
 * vector row, 0 = automatic), "sddmm_group" (16-vector groups per wave step of the
 * MFMA SDDMM: 1, 2, 4, 0 = automatic), "sddmm_block_waves" (1..16, 0 = automatic),
 * "sddmm_flat_supers" (super-groups per wave of algorithm 2, 1..16, 0 = automatic),
 * "attention_waves" (1..8, 0 = automatic), "attention_chunk" (nonzero vectors per
 * LDS chunk of the one-row-per-workgroup attention kernel, 0 = automatic).
 * Returns 0, or 1 for an unknown name / bad value.
 * No counterpart in the reference, whose tile sizes are compile-time constants
 * (src/wmma_spmm.cu:396).
 */
int vs_set_option(const char *name, int value);
int vs_set_thread_option(const char *name, int value);
void vs_clear_thread_options(void);

#ifdef __cplusplus
}
#endif
#endif /* VSPARSE_H */

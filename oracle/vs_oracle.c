/*
 * CPU oracle for the column-vector-sparse SpMM / SDDMM path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is a plain-C restatement of the host
 * loops the reference benchmark executables use to verify their GPU kernels.
 * Only the test-suite, the smoke check and the CPU-baseline leg of the
 * benchmark may load it; the product library never links or calls it.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference tree).  fp16 is carried as raw IEEE binary16 bit patterns in
 * uint16_t because the host compiler has no half type; products of two
 * binary16 values are exact in binary32, so mul+add and fma give the same
 * bits and the result is fully determined by the order of the fp32 adds,
 * which is kept exactly as in the reference.
 *
 * Pinning (what fixes each function besides this restatement):
 *   vso_half_to_float / vso_float_to_half  exhaustive / randomized comparison with numpy's binary16
 *   vso_spmm_host_ref_f32                  float64 dense brute force, scipy CSR (V=1), closed forms
 *   vso_sddmm_host_ref_f16                 float64 dense brute force, full-mask == A*B^T
 *   vso_make_dense_matrix_f16              known-answer vectors produced by libstdc++'s own
 *                                          std::default_random_engine + uniform_real_distribution<float>
 *   vso_sorted_row_swizzle                 permutation + non-increasing length property
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ---------------------------------------------------------------- fp16 <-> fp32 */

float vso_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int shift = 0;
            while ((man & 0x400u) == 0) { man <<= 1; ++shift; }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

/* round-to-nearest-even, the rounding of the reference's half(float) constructor */
uint16_t vso_float_to_half(float f)
{
    uint32_t x;
    memcpy(&x, &f, sizeof x);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
    }
    if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* below the smallest normal half: subnormal or zero */
        if (ax < 0x33000000u) return sign; /* < 2^-25 -> 0 (2^-25 itself ties to even = 0) */
        uint32_t e = ax >> 23;               /* biased fp32 exponent, 102..112 */
        uint32_t m = (ax & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126 - e;            /* 14..24 : result = m >> shift in units of 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) ++q;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (ax >> 23) - (127 - 15);
    uint32_t m = ax & 0x7fffffu;
    uint32_t q = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) ++q; /* carry into the exponent is correct */
    return (uint16_t)(sign | q);
}

/* ---------------------------------------------------------------- SpMM host loop */

/*
 * Follows spmm_benchmark.cpp:66-86.  Dimension letters are the reference's:
 * A is (m_vec*vec_length) x n in column-vector CSR, B is n x k row-major,
 * out is (m_vec*vec_length) x k row-major fp32 (not rounded to fp16).
 * Loop order i (vector row) -> j (nonzero vector, CSR order) -> v -> l, so
 * every output element accumulates its terms in ascending j.
 */
void vso_spmm_host_ref_f32(int m_vec, int vec_length, int k, int n,
                           const int32_t *row_offsets, const int32_t *column_indices,
                           const uint16_t *values, const uint16_t *rhs_matrix,
                           float *output)
{
    (void)n;
    const size_t total = (size_t)m_vec * vec_length * k;
    for (size_t i = 0; i < total; ++i) output[i] = 0.0f;
    float *rhs_row = (float *)malloc(sizeof(float) * (size_t)(k > 0 ? k : 1));
    for (int i = 0; i < m_vec; ++i) {
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            const int col = column_indices[j];
            for (int l = 0; l < k; ++l) rhs_row[l] = vso_half_to_float(rhs_matrix[(size_t)col * k + l]);
            for (int v = 0; v < vec_length; ++v) {
                const float a = vso_half_to_float(values[(size_t)j * vec_length + v]);
                float *out_row = output + ((size_t)i * vec_length + v) * k;
                for (int l = 0; l < k; ++l) out_row[l] += a * rhs_row[l];
            }
        }
    }
    free(rhs_row);
}

/*
 * Same arithmetic, vector rows spread over OpenMP threads (rows are
 * independent, so the per-element order of adds and therefore the bits are
 * unchanged).  Used only to report an all-cores CPU figure.
 */
void vso_spmm_host_ref_f32_mt(int m_vec, int vec_length, int k, int n,
                              const int32_t *row_offsets, const int32_t *column_indices,
                              const uint16_t *values, const uint16_t *rhs_matrix,
                              float *output, int threads)
{
    (void)n;
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
#endif
    for (int i = 0; i < m_vec; ++i) {
        float *rhs_row = (float *)malloc(sizeof(float) * (size_t)(k > 0 ? k : 1));
        float *block = output + (size_t)i * vec_length * k;
        for (size_t t = 0; t < (size_t)vec_length * k; ++t) block[t] = 0.0f;
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            const int col = column_indices[j];
            for (int l = 0; l < k; ++l) rhs_row[l] = vso_half_to_float(rhs_matrix[(size_t)col * k + l]);
            for (int v = 0; v < vec_length; ++v) {
                const float a = vso_half_to_float(values[(size_t)j * vec_length + v]);
                float *out_row = block + (size_t)v * k;
                for (int l = 0; l < k; ++l) out_row[l] += a * rhs_row[l];
            }
        }
        free(rhs_row);
    }
}

/* ---------------------------------------------------------------- SDDMM host loop */

/*
 * Follows include/bm_test_utils.h:171-193 (Host_sddmm).  lhs is
 * (m_vec*vec_length) x k, rhs is n x k, both row-major; the mask is a
 * column-vector CSR; out[j*vec_length+v] = half( sum_l lhs[i*V+v][l]*rhs[col_j][l] ),
 * fp32 accumulate in ascending l, one rounding to binary16 at the end.
 */
void vso_sddmm_host_ref_f16(int m_vec, int k, int vec_length,
                            const int32_t *row_offsets, const int32_t *col_indices,
                            const uint16_t *lhs_matrix, const uint16_t *rhs_matrix,
                            uint16_t *output_values)
{
    float *lhs_rows = (float *)malloc(sizeof(float) * (size_t)vec_length * (size_t)(k > 0 ? k : 1));
    for (int i = 0; i < m_vec; ++i) {
        for (size_t t = 0; t < (size_t)vec_length * k; ++t)
            lhs_rows[t] = vso_half_to_float(lhs_matrix[(size_t)i * vec_length * k + t]);
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            const uint16_t *rhs_row = rhs_matrix + (size_t)col_indices[j] * k;
            for (int v = 0; v < vec_length; ++v) {
                float acc = 0.0f;
                const float *a = lhs_rows + (size_t)v * k;
                for (int l = 0; l < k; ++l) acc += a[l] * vso_half_to_float(rhs_row[l]);
                output_values[(size_t)j * vec_length + v] = vso_float_to_half(acc);
            }
        }
    }
    free(lhs_rows);
}

/* fp32-output flavour of the same loop (the reference template with OutType=float). */
void vso_sddmm_host_ref_f32(int m_vec, int k, int vec_length,
                            const int32_t *row_offsets, const int32_t *col_indices,
                            const uint16_t *lhs_matrix, const uint16_t *rhs_matrix,
                            float *output_values)
{
    for (int i = 0; i < m_vec; ++i) {
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            const uint16_t *rhs_row = rhs_matrix + (size_t)col_indices[j] * k;
            for (int v = 0; v < vec_length; ++v) {
                float acc = 0.0f;
                const uint16_t *a = lhs_matrix + ((size_t)i * vec_length + v) * k;
                for (int l = 0; l < k; ++l) acc += vso_half_to_float(a[l]) * vso_half_to_float(rhs_row[l]);
                output_values[(size_t)j * vec_length + v] = acc;
            }
        }
    }
}

void vso_sddmm_host_ref_f16_mt(int m_vec, int k, int vec_length,
                               const int32_t *row_offsets, const int32_t *col_indices,
                               const uint16_t *lhs_matrix, const uint16_t *rhs_matrix,
                               uint16_t *output_values, int threads)
{
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
#endif
    for (int i = 0; i < m_vec; ++i) {
        float *lhs_rows = (float *)malloc(sizeof(float) * (size_t)vec_length * (size_t)(k > 0 ? k : 1));
        for (size_t t = 0; t < (size_t)vec_length * k; ++t)
            lhs_rows[t] = vso_half_to_float(lhs_matrix[(size_t)i * vec_length * k + t]);
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j) {
            const uint16_t *rhs_row = rhs_matrix + (size_t)col_indices[j] * k;
            for (int v = 0; v < vec_length; ++v) {
                float acc = 0.0f;
                const float *a = lhs_rows + (size_t)v * k;
                for (int l = 0; l < k; ++l) acc += a[l] * vso_half_to_float(rhs_row[l]);
                output_values[(size_t)j * vec_length + v] = vso_float_to_half(acc);
            }
        }
        free(lhs_rows);
    }
}

/* ---------------------------------------------------------------- row swizzles */

/* include/bm_test_utils.h:196-198 */
void vso_identity_row_swizzle(int rows, int32_t *row_indices)
{
    for (int i = 0; i < rows; ++i) row_indices[i] = i;
}

/*
 * include/bm_test_utils.h:200-215: argsort of the rows by length, longest
 * first.  The reference uses std::sort, which leaves the order of equal-length
 * rows unspecified; this restatement breaks ties by ascending row index
 * (insertion-stable merge sort), which is one of the orders std::sort may
 * return.
 */
static void merge_sort_rows(int32_t *idx, int32_t *tmp, const int32_t *len, int lo, int hi)
{
    if (hi - lo < 2) return;
    int mid = lo + (hi - lo) / 2;
    merge_sort_rows(idx, tmp, len, lo, mid);
    merge_sort_rows(idx, tmp, len, mid, hi);
    int a = lo, b = mid, o = lo;
    while (a < mid && b < hi) {
        if (len[idx[b]] > len[idx[a]]) tmp[o++] = idx[b++];
        else tmp[o++] = idx[a++];
    }
    while (a < mid) tmp[o++] = idx[a++];
    while (b < hi) tmp[o++] = idx[b++];
    for (int t = lo; t < hi; ++t) idx[t] = tmp[t];
}

void vso_sorted_row_swizzle(int rows, const int32_t *row_offsets, int32_t *row_indices)
{
    if (rows <= 0) return;
    int32_t *len = (int32_t *)malloc(sizeof(int32_t) * (size_t)rows);
    int32_t *tmp = (int32_t *)malloc(sizeof(int32_t) * (size_t)rows);
    for (int i = 0; i < rows; ++i) {
        len[i] = row_offsets[i + 1] - row_offsets[i];
        row_indices[i] = i;
    }
    merge_sort_rows(row_indices, tmp, len, 0, rows);
    free(len);
    free(tmp);
}

/* ---------------------------------------------------------------- operand generator */

/*
 * include/bm_test_utils.h:130-142 (MakeDenseMatrix) as the benchmarks call it
 * (spmm_benchmark.cpp:38,59-60; sddmm_benchmark.cpp:189,212-213): a
 * default-constructed std::default_random_engine passed BY VALUE, so every
 * call starts from the same state.  With libstdc++ that engine is
 * minstd_rand0 (x <- 16807*x mod 2^31-1, seed 1) and
 * uniform_real_distribution<float>(-1,1) draws one engine value per sample:
 * c = float(x-1) / float(2147483646.0L) (the divisor rounds to 2^31), clamped
 * below 1, result c*2 + (-1) in fp32, then rounded to binary16.
 * `skip` discards that many leading draws (0 reproduces the reference).
 */
void vso_make_dense_matrix_f32(int64_t count, int64_t skip, float *out)
{
    uint64_t x = 1;
    const float denom = 2147483648.0f;
    for (int64_t i = 0; i < skip + count; ++i) {
        x = (x * 16807u) % 2147483647u;
        if (i < skip) continue;
        float c = (float)(uint32_t)(x - 1) / denom;
        if (c >= 1.0f) c = 0.99999994f; /* nextafter(1,0) */
        out[i - skip] = c * 2.0f + -1.0f;
    }
}

void vso_make_dense_matrix_f16(int64_t count, int64_t skip, uint16_t *out)
{
    uint64_t x = 1;
    const float denom = 2147483648.0f;
    for (int64_t i = 0; i < skip + count; ++i) {
        x = (x * 16807u) % 2147483647u;
        if (i < skip) continue;
        float c = (float)(uint32_t)(x - 1) / denom;
        if (c >= 1.0f) c = 0.99999994f;
        out[i - skip] = vso_float_to_half(c * 2.0f + -1.0f);
    }
}

int vso_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

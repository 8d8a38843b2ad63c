// A C++ caller written the way the reference's benchmarks call their operators
// (spmm_benchmark.cpp:127,131 and sddmm_benchmark.cpp:257,262: namespaces spmm / sddmm, overloads picked
// by the output pointer type), compiled against include/vsparse_shim.hpp and linked with libvsparse.so.
// It shows that the reference's call sites work unchanged on top of the C ABI: device buffers from
// hipMalloc, no Python, no torch.  Results are checked on the host with the reference's own acceptance
// rule (no element may differ by more than 0.5, spmm_benchmark.cpp:213) and a 1e-2 relative bound.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "vsparse_shim.hpp"

#define HIP_OK(call)                                                                         \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess) {                                                              \
            std::printf("%s failed: %s\n", #call, hipGetErrorString(e_));                    \
            std::exit(2);                                                                    \
        }                                                                                    \
    } while (0)

template <typename T>
static T *to_device(const std::vector<T> &h)
{
    T *d = nullptr;
    HIP_OK(hipMalloc(&d, std::max<size_t>(h.size(), 1) * sizeof(T)));
    if (!h.empty()) HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

static std::vector<half> random_halves(size_t count, std::default_random_engine &engine)
{
    std::uniform_real_distribution<float> dist(-1.f, 1.f);
    std::vector<half> v(count);
    for (auto &x : v) x = __float2half(dist(engine));
    return v;
}

// max over elements of |got - want| / max(|want|, 1e-2 * rms(want)); also counts |got - want| > 0.5
static bool close_enough(const char *what, const std::vector<float> &got, const std::vector<float> &want)
{
    double sq = 0;
    for (float w : want) sq += (double)w * w;
    const double floor_ = 1e-2 * std::sqrt(sq / std::max<size_t>(want.size(), 1));
    double worst = 0;
    int errors = 0;
    for (size_t i = 0; i < want.size(); ++i) {
        const double diff = std::fabs((double)got[i] - want[i]);
        if (diff > 0.5 || std::isnan(got[i])) ++errors;
        worst = std::max(worst, diff / std::max<double>(std::fabs(want[i]), std::max(floor_, 1e-30)));
    }
    const bool ok = errors == 0 && worst <= 1e-2;
    std::printf("%-22s errors>0.5: %d  max rel err %.2e  %s\n", what, errors, worst, ok ? "ok" : "FAILED");
    return ok;
}

int main()
{
    const int V = 8, m_vec = 48, n = 640, k_dense = 192, k_contract = 64;
    std::default_random_engine engine(7);
    // pattern: a different number of distinct, ascending columns per vector row (one row empty)
    std::vector<int> row_offsets(1, 0), column_indices;
    for (int i = 0; i < m_vec; ++i) {
        const int len = i == 5 ? 0 : 10 + (int)(engine() % 90);
        std::vector<int> cols(n);
        for (int c = 0; c < n; ++c) cols[c] = c;
        std::shuffle(cols.begin(), cols.end(), engine);
        std::sort(cols.begin(), cols.begin() + len);
        column_indices.insert(column_indices.end(), cols.begin(), cols.begin() + len);
        row_offsets.push_back((int)column_indices.size());
    }
    const int nnz_vec = row_offsets.back();
    std::vector<int> row_indices(m_vec);
    vs_sorted_row_swizzle(m_vec, row_offsets.data(), row_indices.data());

    const std::vector<half> values = random_halves((size_t)nnz_vec * V, engine);
    const std::vector<half> rhs = random_halves((size_t)n * k_dense, engine);
    const std::vector<half> lhs_s = random_halves((size_t)m_vec * V * k_contract, engine);
    const std::vector<half> rhs_s = random_halves((size_t)n * k_contract, engine);

    int *d_row_indices = to_device(row_indices), *d_row_offsets = to_device(row_offsets);
    int *d_cols = to_device(column_indices);
    half *d_values = to_device(values), *d_rhs = to_device(rhs), *d_lhs_s = to_device(lhs_s), *d_rhs_s = to_device(rhs_s);
    half *d_out_h = nullptr, *d_sd_h = nullptr;
    float *d_out_f = nullptr, *d_sd_f = nullptr;
    HIP_OK(hipMalloc(&d_out_h, (size_t)m_vec * V * k_dense * sizeof(half)));
    HIP_OK(hipMalloc(&d_out_f, (size_t)m_vec * V * k_dense * sizeof(float)));
    HIP_OK(hipMalloc(&d_sd_h, (size_t)nnz_vec * V * sizeof(half)));
    HIP_OK(hipMalloc(&d_sd_f, (size_t)nnz_vec * V * sizeof(float)));

    // host results: the loops of spmm_benchmark.cpp:66-86 and bm_test_utils.h:171-193 (fp32, in order)
    std::vector<float> want_spmm((size_t)m_vec * V * k_dense, 0.f), want_sddmm((size_t)nnz_vec * V, 0.f);
    for (int i = 0; i < m_vec; ++i)
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j)
            for (int v = 0; v < V; ++v)
                for (int l = 0; l < k_dense; ++l)
                    want_spmm[((size_t)i * V + v) * k_dense + l] +=
                        __half2float(values[(size_t)j * V + v]) * __half2float(rhs[(size_t)column_indices[j] * k_dense + l]);
    for (int i = 0; i < m_vec; ++i)
        for (int j = row_offsets[i]; j < row_offsets[i + 1]; ++j)
            for (int v = 0; v < V; ++v) {
                float acc = 0.f;
                for (int l = 0; l < k_contract; ++l)
                    acc += __half2float(lhs_s[((size_t)i * V + v) * k_contract + l]) *
                           __half2float(rhs_s[(size_t)column_indices[j] * k_contract + l]);
                want_sddmm[(size_t)j * V + v] = acc;
            }

    bool ok = true;
    std::vector<half> got_h;
    std::vector<float> got_f;
    auto fetch_h = [&](const half *d, size_t count) {
        got_h.resize(count);
        HIP_OK(hipMemcpy(got_h.data(), d, count * sizeof(half), hipMemcpyDeviceToHost));
        got_f.resize(count);
        for (size_t i = 0; i < count; ++i) got_f[i] = __half2float(got_h[i]);
    };
    auto fetch_f = [&](const float *d, size_t count) {
        got_f.resize(count);
        HIP_OK(hipMemcpy(got_f.data(), d, count * sizeof(float), hipMemcpyDeviceToHost));
    };

    // the reference's argument order: (m_vec, vec_length, k = dense width, n = columns of the sparse matrix, ...)
    HIP_OK(spmm::wmmaSpmm(m_vec, V, k_dense, n, d_row_indices, d_row_offsets, d_cols, d_values, d_rhs, d_out_h));
    HIP_OK(hipDeviceSynchronize());
    fetch_h(d_out_h, want_spmm.size());
    ok &= close_enough("spmm::wmmaSpmm half", got_f, want_spmm);
    HIP_OK(spmm::wmmaSpmm(m_vec, V, k_dense, n, d_row_indices, d_row_offsets, d_cols, d_values, d_rhs, d_out_f));
    HIP_OK(hipDeviceSynchronize());
    fetch_f(d_out_f, want_spmm.size());
    ok &= close_enough("spmm::wmmaSpmm float", got_f, want_spmm);
    HIP_OK(spmm::cudaSpmm(m_vec, V, k_dense, n, d_row_indices, d_row_offsets, d_cols, d_values, d_rhs, d_out_h));
    HIP_OK(hipDeviceSynchronize());
    fetch_h(d_out_h, want_spmm.size());
    ok &= close_enough("spmm::cudaSpmm half", got_f, want_spmm);

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    HIP_OK(sddmm::wmmaSddmm(m_vec, k_contract, n, nnz_vec, d_row_indices, d_row_offsets, d_cols, d_lhs_s, d_rhs_s, d_sd_h,
                            V, stream, /*algorithm=*/0));
    HIP_OK(hipStreamSynchronize(stream));
    fetch_h(d_sd_h, want_sddmm.size());
    ok &= close_enough("sddmm::wmmaSddmm half", got_f, want_sddmm);
    HIP_OK(sddmm::cudaSddmm(m_vec, k_contract, n, nnz_vec, d_row_indices, d_row_offsets, d_cols, d_lhs_s, d_rhs_s, d_sd_f,
                            V, stream));
    HIP_OK(hipStreamSynchronize(stream));
    fetch_f(d_sd_f, want_sddmm.size());
    ok &= close_enough("sddmm::cudaSddmm float", got_f, want_sddmm);

    // what the reference only prints about is an error here: float operands, the timing-only algorithm 3
    const float *no_f = nullptr;
    float *no_out = nullptr;
    const bool rejects = spmm::wmmaSpmm(m_vec, V, k_dense, n, d_row_indices, d_row_offsets, d_cols, no_f, no_f, no_out) != hipSuccess &&
                         sddmm::wmmaSddmm(m_vec, k_contract, n, nnz_vec, d_row_indices, d_row_offsets, d_cols, d_lhs_s,
                                          d_rhs_s, d_sd_h, V, stream, 3) != hipSuccess;
    std::printf("%-22s %s\n", "unsupported overloads", rejects ? "rejected: ok" : "FAILED");
    ok &= rejects;

    // how fast a plain C++ loop issues the operator (the reference's benchmark is such a loop, spmm_benchmark.cpp:127):
    // calls back to back on one stream, no HIP graph; printed for information
    {
        const int calls = 2000;
        for (int i = 0; i < 50; ++i)
            HIP_OK(spmm::wmmaSpmm(m_vec, V, k_dense, n, d_row_indices, d_row_offsets, d_cols, d_values, d_rhs, d_out_h));
        HIP_OK(hipDeviceSynchronize());
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < calls; ++i)
            HIP_OK(spmm::wmmaSpmm(m_vec, V, k_dense, n, d_row_indices, d_row_offsets, d_cols, d_values, d_rhs, d_out_h));
        const auto t1 = std::chrono::steady_clock::now();
        HIP_OK(hipDeviceSynchronize());
        const auto t2 = std::chrono::steady_clock::now();
        std::printf("%-22s %.2f us per call to issue, %.2f us per call until the last one has finished (%d calls)\n",
                    "spmm::wmmaSpmm loop", std::chrono::duration<double, std::micro>(t1 - t0).count() / calls,
                    std::chrono::duration<double, std::micro>(t2 - t0).count() / calls, calls);
    }

    // the same operator with long rows dispatched in parts: the host makes the dispatch list (limit 64 here, so
    // that several of these short rows are split), the entry point takes it in place of the swizzle and the offsets
    {
        int n_slots = 0, n_split = 0, parts_max = 0, longest = 0;
        std::vector<int> slots(4 * (size_t)(m_vec + 2 * (nnz_vec / 64) + 1));
        ok &= vs_spmm_row_parts(m_vec, row_offsets.data(), 64, slots.data(), (int)(slots.size() / 4), &n_slots, &n_split,
                                &parts_max, &longest) == 0;
        slots.resize(4 * (size_t)(n_slots + n_split));
        int *d_slots = to_device(slots);
        const long long bytes = vs_wmma_spmm_row_parts_workspace_bytes(1, V, k_dense, n_split, parts_max);
        void *workspace = nullptr;
        HIP_OK(hipMalloc(&workspace, (size_t)bytes));
        HIP_OK(hipMemset(workspace, 0, (size_t)bytes));  // zeroed once, before the first use
        for (int call = 0; call < 2; ++call) {
            HIP_OK(hipMemset(d_out_h, 0x7f, (size_t)m_vec * V * k_dense * sizeof(half)));
            HIP_OK((hipError_t)vs_wmma_spmm_f16_row_parts(1, V, k_dense, n, n_slots, d_slots, n_split, parts_max, nnz_vec,
                                                          longest, d_cols, d_values, 0, d_rhs, 0, d_out_h, 0, workspace, bytes,
                                                          nullptr));
            HIP_OK(hipDeviceSynchronize());
            fetch_h(d_out_h, want_spmm.size());
            ok &= close_enough(call == 0 ? "vs_wmma_spmm_f16_row_parts" : "vs_wmma_spmm_f16_row_parts again", got_f, want_spmm);
        }
        // the SDDMM on the same list: nothing to add up across parts, no workspace
        HIP_OK(hipMemset(d_sd_h, 0x7f, (size_t)nnz_vec * V * sizeof(half)));
        HIP_OK((hipError_t)vs_wmma_sddmm_f16_row_parts(1, k_contract, n, n_slots, d_slots, nnz_vec, d_cols, d_lhs_s, 0,
                                                       d_rhs_s, 0, d_sd_h, 0, V, nullptr));
        HIP_OK(hipDeviceSynchronize());
        fetch_h(d_sd_h, want_sddmm.size());
        ok &= close_enough("vs_wmma_sddmm_f16_row_parts", got_f, want_sddmm);
        // the row-wise softmax on the same list, in place on the SDDMM's outputs (layout [nonzero vector][V]: scalar
        // row v of a vector row owns every V-th value); expected values from the fp16 scores just fetched
        {
            const float scale = 0.125f;
            std::vector<float> want_softmax(got_f.size());
            for (int r = 0; r < m_vec; ++r)
                for (int v = 0; v < V; ++v) {
                    float top = -INFINITY;
                    double sum = 0;
                    for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j) top = std::max(top, scale * got_f[(size_t)j * V + v]);
                    for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j) sum += std::exp(scale * got_f[(size_t)j * V + v] - top);
                    for (int j = row_offsets[r]; j < row_offsets[r + 1]; ++j)
                        want_softmax[(size_t)j * V + v] = (float)(std::exp(scale * got_f[(size_t)j * V + v] - top) / sum);
                }
            const long long sm_bytes = vs_sparse_softmax_row_parts_workspace_bytes(1, V, n_split, parts_max);
            void *sm_workspace = nullptr;
            HIP_OK(hipMalloc(&sm_workspace, (size_t)std::max<long long>(sm_bytes, 8)));  // no need to clear it
            HIP_OK((hipError_t)vs_sparse_softmax_f16_row_parts(1, V, n_slots, d_slots, n_split, parts_max, d_sd_h, 0, d_sd_h, 0,
                                                               scale, sm_workspace, sm_bytes, nullptr));
            HIP_OK(hipDeviceSynchronize());
            fetch_h(d_sd_h, want_softmax.size());
            ok &= close_enough("vs_sparse_softmax_f16_row_parts", got_f, want_softmax);
            HIP_OK(hipFree(sm_workspace));
        }
        std::printf("%-22s %d slots, %d rows in up to %d parts\n", "", n_slots, n_split, parts_max);
        ok &= n_split > 0;
        HIP_OK(hipFree(workspace));
        HIP_OK(hipFree(d_slots));
    }

    HIP_OK(hipStreamDestroy(stream));
    for (void *p : {(void *)d_row_indices, (void *)d_row_offsets, (void *)d_cols, (void *)d_values, (void *)d_rhs,
                    (void *)d_lhs_s, (void *)d_rhs_s, (void *)d_out_h, (void *)d_out_f, (void *)d_sd_h, (void *)d_sd_f})
        HIP_OK(hipFree(p));
    std::printf(ok ? "PASSED\n" : "FAILED\n");
    return ok ? 0 : 1;
}

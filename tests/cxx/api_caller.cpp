// A C++ caller written the way the reference's test program is (RoDe_SDDMM/test.cu):
// seeded matrix, CPU check, GPU preprocessing, RoDeSDDMM_n32/_n128 and
// RoDeSpmm_n32/_n128 on two streams through the reference-signature headers, one JSON
// line on stdout.  Test code: built by __graft_entry__.build(), run by
// tests/test_gpu_cxx_caller.py.
//
//   api_caller <m> <n> <nnz_per_row> <k: 32|128> [seg]
#include "RoDePreprocess.h"
#include "RoDeSddmm.h"
#include "RoDeSpmm.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#define HIP_OK(call)                                                                              \
    do {                                                                                          \
        hipError_t e_ = (call);                                                                   \
        if (e_ != hipSuccess) {                                                                   \
            std::printf("{\"passed\": false, \"error\": \"%s at line %d\"}\n", hipGetErrorString(e_), __LINE__); \
            return 1;                                                                             \
        }                                                                                         \
    } while (0)

template <typename T>
static T* to_device(const std::vector<T>& h)
{
    T* d = nullptr;
    if (hipMalloc(&d, std::max<size_t>(h.size(), 1) * sizeof(T)) != hipSuccess) return nullptr;
    if (!h.empty()) (void)hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice);
    return d;
}

int main(int argc, char** argv)
{
    if (argc < 5) {
        std::printf("{\"passed\": false, \"error\": \"usage: api_caller m n nnz_per_row k [seg]\"}\n");
        return 1;
    }
    const int m = std::atoi(argv[1]), n = std::atoi(argv[2]), per_row = std::atoi(argv[3]), k = std::atoi(argv[4]);
    const int seg = argc > 5 ? std::atoi(argv[5]) : (k == 128 ? 32 : 512); // the reference's parameter sets

    // unpadded rows (any start offset), some empty, a few long
    std::mt19937 gen(42);
    std::uniform_real_distribution<float> uni(-1.f, 1.f);
    std::vector<int> row_ptr(1, 0), col;
    std::vector<float> val;
    for (int r = 0; r < m; ++r) {
        int len = (int)(gen() % (2 * per_row + 1));
        if (r % 97 == 5) len = std::min(n, 40 * per_row);
        len = std::min(len, n);
        std::vector<int> c(n);
        for (int i = 0; i < n; ++i) c[i] = i;
        for (int i = 0; i < len; ++i) std::swap(c[i], c[i + gen() % (n - i)]);
        std::sort(c.begin(), c.begin() + len);
        for (int i = 0; i < len; ++i) {
            col.push_back(c[i]);
            val.push_back(uni(gen));
        }
        row_ptr.push_back((int)col.size());
    }
    const int nnz = (int)col.size();
    std::vector<float> lhs((size_t)m * k), rhs((size_t)n * k);
    for (auto& x : lhs) x = uni(gen);
    for (auto& x : rhs) x = uni(gen);

    // CPU results in double
    std::vector<double> sddmm_ref(nnz), spmm_ref((size_t)m * k, 0.0), spmm_l1(m, 0.0);
    for (int r = 0; r < m; ++r)
        for (int idx = row_ptr[r]; idx < row_ptr[r + 1]; ++idx) {
            double dot = 0;
            for (int t = 0; t < k; ++t) dot += (double)lhs[(size_t)r * k + t] * rhs[(size_t)col[idx] * k + t];
            sddmm_ref[idx] = val[idx] * dot;
            for (int t = 0; t < k; ++t) spmm_ref[(size_t)r * k + t] += (double)val[idx] * rhs[(size_t)col[idx] * k + t];
        }
    for (int r = 0; r < m; ++r)
        for (int t = 0; t < k; ++t) spmm_l1[r] += std::fabs(spmm_ref[(size_t)r * k + t]);

    int *d_rp = to_device(row_ptr), *d_col = to_device(col);
    float *d_val = to_device(val), *d_lhs = to_device(lhs), *d_rhs = to_device(rhs);
    const int cap = (nnz + 3 * m) / seg + m + 1;
    int *d_blk, *d_st, *d_res, *d_cnt;
    float *d_out, *d_C;
    HIP_OK(hipMalloc(&d_blk, sizeof(int) * cap));
    HIP_OK(hipMalloc(&d_st, sizeof(int) * (cap + 1)));
    HIP_OK(hipMalloc(&d_res, sizeof(int) * std::max(m, 1)));
    HIP_OK(hipMalloc(&d_cnt, sizeof(int) * 2));
    HIP_OK(hipMalloc(&d_out, sizeof(float) * std::max(nnz, 1)));
    HIP_OK(hipMalloc(&d_C, sizeof(float) * (size_t)m * k));

    RoDe_preprocess(seg, 32, 4, m, d_rp, d_blk, d_st, d_res, d_cnt, d_cnt + 1);
    int cnt[2];
    HIP_OK(hipMemcpy(cnt, d_cnt, sizeof(cnt), hipMemcpyDeviceToHost));

    // the host-pointer twins (Preprocess_opt/_preprocess.cu:340 and main.cu:114-123 argument
    // orders) must give the arrays of the device routine
    bool twins_equal = true;
    {
        std::vector<int> g_blk(std::max(cnt[0], 1)), g_st(cnt[0] + 1), g_res(std::max(cnt[1], 1));
        if (cnt[0]) HIP_OK(hipMemcpy(g_blk.data(), d_blk, sizeof(int) * cnt[0], hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(g_st.data(), d_st, sizeof(int) * (cnt[0] + 1), hipMemcpyDeviceToHost));
        if (cnt[1]) HIP_OK(hipMemcpy(g_res.data(), d_res, sizeof(int) * cnt[1], hipMemcpyDeviceToHost));
        for (int variant = 0; variant < 2; ++variant) {
            std::vector<int> h_blk(cap, -1), h_st(cap + 1, -1), h_res(std::max(m, 1), -1);
            int n_blk = -1, n_res = -1;
            if (variant == 0)
                RoDe_preprocess_cpu(seg, 32, 4, m, row_ptr.data(), h_blk.data(), h_st.data(), h_res.data(), n_blk, n_res);
            else
                RoDe_preprocess(seg, 4, 32, m, row_ptr.data(), h_blk.data(), h_st.data(), h_res.data(), n_blk, n_res);
            twins_equal = twins_equal && n_blk == cnt[0] && n_res == cnt[1] &&
                          std::equal(g_blk.begin(), g_blk.begin() + cnt[0], h_blk.begin()) &&
                          std::equal(g_st.begin(), g_st.end(), h_st.begin()) &&
                          std::equal(g_res.begin(), g_res.begin() + cnt[1], h_res.begin()) &&
                          h_blk[cnt[0]] == -1 && h_st[cnt[0] + 1] == -1; // nothing written past the result
        }
    }

    hipStream_t s1, s2;
    HIP_OK(hipStreamCreate(&s1));
    HIP_OK(hipStreamCreate(&s2));
    HIP_OK(hipMemset(d_out, 0xff, sizeof(float) * std::max(nnz, 1))); // NaN pattern: every entry must be overwritten
    HIP_OK(hipMemset(d_C, 0, sizeof(float) * (size_t)m * k));
    HIP_OK(hipDeviceSynchronize());
    if (k == 32) {
        RoDeSDDMM_n32(cnt[0], cnt[1], n, k, d_blk, d_res, d_st, d_rp, d_col, d_val, d_lhs, d_rhs, d_out, s1, s2);
        RoDeSpmm_n32(cnt[0], cnt[1], n, k, d_val, d_col, d_rp, d_blk, d_res, d_st, d_rhs, d_C, s1, s2);
    } else {
        RoDeSDDMM_n128(cnt[0], cnt[1], n, k, d_blk, d_res, d_st, d_rp, d_col, d_val, d_lhs, d_rhs, d_out, s1, s2);
        RoDeSpmm_n128(cnt[0], cnt[1], n, k, d_val, d_col, d_rp, d_blk, d_res, d_st, d_rhs, d_C, s1, s2);
    }
    HIP_OK(hipStreamSynchronize(s1));
    HIP_OK(hipStreamSynchronize(s2));

    std::vector<float> out(nnz), C((size_t)m * k);
    if (nnz) HIP_OK(hipMemcpy(out.data(), d_out, sizeof(float) * nnz, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(C.data(), d_C, sizeof(float) * C.size(), hipMemcpyDeviceToHost));

    // the reference test's rule for SDDMM (abs AND rel above 1e-3), row-L1 rule for SpMM
    int errors = 0;
    double max_abs = 0, spmm_err = 0;
    for (int i = 0; i < nnz; ++i) {
        const double diff = std::fabs((double)out[i] - sddmm_ref[i]);
        max_abs = std::max(max_abs, diff);
        if (!(diff <= 1e-3) && !(diff / (std::fabs(sddmm_ref[i]) + 1e-6) <= 1e-3)) ++errors;
    }
    for (int r = 0; r < m; ++r)
        for (int t = 0; t < k; ++t) {
            const double diff = std::fabs((double)C[(size_t)r * k + t] - spmm_ref[(size_t)r * k + t]);
            if (spmm_l1[r] > 0) spmm_err = std::max(spmm_err, diff / spmm_l1[r]);
            else if (diff != 0) spmm_err = 1.0;
        }
    const bool passed = errors == 0 && spmm_err <= 1e-4 && twins_equal;
    std::printf("{\"passed\": %s, \"nnz\": %d, \"n_blk\": %d, \"n_res\": %d, \"sddmm_errors\": %d, "
                "\"sddmm_max_abs\": %.3e, \"spmm_rowL1_err\": %.3e, \"host_twins_equal\": %s}\n",
                passed ? "true" : "false", nnz, cnt[0], cnt[1], errors, max_abs, spmm_err,
                twins_equal ? "true" : "false");
    return passed ? 0 : 1;
}

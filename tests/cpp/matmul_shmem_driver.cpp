// Test driver in the role of the reference's main() for the SIMT kernel (matmul_shmem.cu:176-325) and its fixture
// (matmul_test.h:53-168): for every element type the reference instantiates (<half, float>, <float, float>,
// <int, int>) a correctness sweep over all legal (tile_dim, block_rows) pairs against the CPU loop - tolerance 0.1
// for the floating types, 0 for <int, int> - and a performance sweep that prints the reference's
//   (tile_dim, block_rows): TFLOP/s
// lines. Everything goes through ckopt::matmul_shmem<DT, DT_ACC> of include/ckopt.hpp, i.e. through the C ABI.
// Test infrastructure: it links the CPU oracle for the check.
//
//   matmul_shmem_driver correctness | performance [dim] | all [dim]
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "ckopt.hpp"

extern "C" int oracle_matmul(int dtype, const void* a, const void* b, void* out, int M, int N, int K, int b_transposed, int fused,
                             int row_begin, int row_end, int threads);

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); std::exit(2); } } while (0)

template <typename DT> struct Name;
template <> struct Name<ckopt::half_t> { static const char* get() { return "<half, float>"; } };
template <> struct Name<float> { static const char* get() { return "<float, float>"; } };
template <> struct Name<int> { static const char* get() { return "<int, int>"; } };

template <typename DT> static void fill(std::vector<DT>& v, uint64_t stream_id) {
    if (std::is_same<DT, int>::value) ckopt::check(ckopt_fill_int(CKOPT_DT_I32, v.data(), (int64_t)v.size(), 79, stream_id, -10, 10), "fill");
    else ckopt::check(ckopt_fill_uniform(ckopt::dtype_of<DT>::value, v.data(), (int64_t)v.size(), 79, stream_id, -1.f, 1.f), "fill");
}

// (tile_dim, block_rows) pairs the launcher accepts: the reference's three conditions (threads per block, values per
// thread, divisibility, matmul_shmem.cu:204-206) are ckopt_check_matmul_shmem_tuning here
// and the tile's shared memory fits the device (get_shmem_req<DT>(tile_dim), matmul_shmem.cu:138-141, :198-200)
template <typename DT, typename F> static void for_each_legal_pair(F f) {
    for (int tile_dim = 32; tile_dim <= 256; tile_dim *= 2)
        for (int block_rows = 1; block_rows <= tile_dim; block_rows *= 2)
            if (ckopt_check_matmul_shmem_tuning(tile_dim, block_rows) == CKOPT_OK && ckopt::get_shmem_req<DT>(tile_dim) <= 160 * 1024)
                f(tile_dim, block_rows);
}

template <typename DT> struct DeviceBuffers {
    DT *A = nullptr, *B = nullptr, *C = nullptr;
    size_t n;
    explicit DeviceBuffers(size_t elems) : n(elems) {
        HIP_OK(hipMalloc((void**)&A, n * sizeof(DT))); HIP_OK(hipMalloc((void**)&B, n * sizeof(DT))); HIP_OK(hipMalloc((void**)&C, n * sizeof(DT)));
    }
    ~DeviceBuffers() { (void)hipFree(A); (void)hipFree(B); (void)hipFree(C); }
};

// |cpu - gpu| <= atol for every element; the CPU sum is cast to DT before comparing (matmul_test.h:128-132)
template <typename DT> static bool is_correct(const std::vector<DT>& res, const std::vector<float>& ref_f, const std::vector<int>& ref_i, size_t n, float atol) {
    for (size_t i = 0; i < n; ++i) {
        if constexpr (std::is_same<DT, int>::value) {
            if (res[i] != ref_i[i]) return false;
        } else {
            const float want = ckopt::to_float((DT)ref_f[i]);
            if (!(std::fabs(ckopt::to_float(res[i]) - want) <= atol)) return false;
        }
    }
    return true;
}

template <typename DT>
static int run_correctness(int dim_max, int num_reps, float atol) {
    std::printf("\nmatmul_shmem_kernel, %s, correctness:\n", Name<DT>::get());
    const size_t n = (size_t)dim_max * dim_max;
    std::vector<DT> a(n), b(n), res(n);
    std::vector<float> ref_f(std::is_same<DT, int>::value ? 0 : n);
    std::vector<int> ref_i(std::is_same<DT, int>::value ? n : 0);
    fill(a, 0);
    fill(b, 1);
    DeviceBuffers<DT> d(n);
    int failed = 0;
    unsigned lcg = 2463534242u;
    for (int b_transposed = 0; b_transposed < 2; ++b_transposed) {   // 0: B is K x N as in the reference; 1: N x K
        for_each_legal_pair<DT>([&](int tile_dim, int block_rows) {
            bool ok = true;
            for (int rep = 0; rep < num_reps; ++rep) {
                // the first repetition at the full size, the others at a random multiple of the tile (role of Rerand/GetMatDim)
                lcg = lcg * 1664525u + 1013904223u;
                const int dim = rep == 0 ? dim_max : tile_dim * (1 + (int)((lcg >> 8) % (unsigned)(dim_max / tile_dim)));
                const size_t m = (size_t)dim * dim;
                HIP_OK(hipMemcpy(d.A, a.data(), m * sizeof(DT), hipMemcpyHostToDevice));
                HIP_OK(hipMemcpy(d.B, b.data(), m * sizeof(DT), hipMemcpyHostToDevice));
                HIP_OK(hipMemset(d.C, 0, n * sizeof(DT)));
                ckopt::matmul_shmem<DT, DT>(d.A, d.B, d.C, dim, dim, dim, tile_dim, block_rows, b_transposed != 0);
                HIP_OK(hipMemcpy(res.data(), d.C, m * sizeof(DT), hipMemcpyDeviceToHost));
                void* out = std::is_same<DT, int>::value ? (void*)ref_i.data() : (void*)ref_f.data();
                if (oracle_matmul(ckopt::dtype_of<DT>::value, a.data(), b.data(), out, dim, dim, dim, b_transposed, 0, 0, dim, 0) != 0) ok = false;
                ok = ok && is_correct(res, ref_f, ref_i, m, atol);
            }
            std::printf("(%d, %d)%s: %s\n", tile_dim, block_rows, b_transposed ? " Bt" : "", ok ? "passed" : "failed");
            failed += ok ? 0 : 1;
        });
    }
    return failed;
}

template <typename DT>
static int run_performance(int dim, int num_reps) {
    std::printf("\nmatmul_shmem_kernel, %s, [TFLOPS]:\n", Name<DT>::get());
    const size_t n = (size_t)dim * dim;
    std::vector<DT> a(n), b(n);
    fill(a, 0);
    fill(b, 1);
    DeviceBuffers<DT> d(n);
    HIP_OK(hipMemcpy(d.A, a.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.B, b.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start)); HIP_OK(hipEventCreate(&stop));
    for_each_legal_pair<DT>([&](int tile_dim, int block_rows) {
        if (dim % tile_dim) return;
        float ms = 0.f;
        ckopt::matmul_shmem<DT, DT>(d.A, d.B, d.C, dim, dim, dim, tile_dim, block_rows);
        HIP_OK(hipEventRecord(start, nullptr));
        for (int i = 0; i < num_reps; ++i) ckopt::matmul_shmem<DT, DT>(d.A, d.B, d.C, dim, dim, dim, tile_dim, block_rows);
        HIP_OK(hipEventRecord(stop, nullptr));
        HIP_OK(hipEventSynchronize(stop));
        HIP_OK(hipEventElapsedTime(&ms, start, stop));
        std::printf("(%d, %d): %.2f\n", tile_dim, block_rows, 2.0 * dim * dim * 1e-9 * dim * num_reps / ms);
    });
    HIP_OK(hipEventDestroy(start)); HIP_OK(hipEventDestroy(stop));
    return 0;
}

int main(int argc, char** argv) {
    const char* what = argc > 1 ? argv[1] : "all";
    const int perf_dim = argc > 2 ? std::atoi(argv[2]) : 4096;
    int failed = 0;
    try {
        if (!std::strcmp(what, "correctness") || !std::strcmp(what, "all")) {
            failed += run_correctness<ckopt::half_t>(256, 2, 0.1f);
            failed += run_correctness<float>(256, 2, 0.1f);
            failed += run_correctness<int>(256, 2, 0.f);
        }
        if (!std::strcmp(what, "performance") || !std::strcmp(what, "all")) {
            failed += run_performance<ckopt::half_t>(perf_dim, 2);
            failed += run_performance<float>(perf_dim, 2);
            failed += run_performance<int>(perf_dim, 2);
        }
    } catch (const ckopt::Error& e) {
        std::fprintf(stderr, "%s (code %d)\n", e.what(), e.code);
        return 3;
    }
    std::printf(failed ? "FAILED\n" : "PASSED\n");
    return failed ? 1 : 0;
}

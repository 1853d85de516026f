// Test driver in the role of the reference's per-file main() (matmul_shmem_tc_async_opt_port_2.cu:1171-1566) and
// its fixtures (matmul_test.h): constant-matrix correctness sweep, random accuracy counts against the CPU
// oracle, and a performance sweep that prints the reference's tuple-per-line format
//   (tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m,
//    num_stages, num_producer_warps, num_consumer_warps): TFLOP/s
// Everything goes through the launcher templates of include/ckopt.hpp, i.e. through the C ABI. Test
// infrastructure: it links the CPU oracle for the accuracy check.
//
//   gemm_driver correctness | accuracy | performance [dim] | all
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "ckopt.hpp"

extern "C" {
int oracle_gemm_blocked(int dtype, const uint16_t* a, const uint16_t* bt, const float* c, float* out, float alpha, float beta,
                        int M, int N, int K, int row0, int row1, int threads);
int64_t oracle_count_incorrect(const float* expected, const float* res, int64_t n, float atol);
}

#define HIP_OK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); std::exit(2); } } while (0)

using DT = ckopt::half_t;
using DT_ACC = float;

struct Tuple { int tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, rows_a, rows_b, tile_group_m, num_stages, producers, consumers; };

static void print_tuple(const Tuple& t) {
    std::printf("(%d, %d, %d, %d, %d, %d, %d, %d, %d, %d)", t.tile_dim, t.segment_dim_k, t.bar_steps_a, t.bar_steps_b, t.rows_a, t.rows_b,
                t.tile_group_m, t.num_stages, t.producers, t.consumers);
}

// every legal tuple of a small grid of knobs, all three granularities with all their bar_steps
static std::vector<Tuple> tuples(int stride) {
    std::vector<Tuple> out;
    int n = 0;
    const int tiles[] = {64, 128, 256}, cons[] = {4, 8}, segs[] = {32, 64, 128}, prods[] = {0, 2, 4};
    for (int tile : tiles) for (int c : cons) {
        if (ckopt_get_num_acc(tile, c) < 0 || ckopt_get_num_acc(tile, c) > 32) continue;
        const int wtr = ckopt::get_warp_tile_rows(tile, c), wtc = ckopt::get_num_acc(tile, c) / wtr;
        const int rows_a[3] = {16, wtr * 16, tile}, rows_b[3] = {16, wtc * 16, tile};
        const int sa_end[3] = {wtr - 1, c / 2, 0}, sb_end[3] = {wtc - 1, 2, 0};
        for (int sk : segs) for (int stages = 1; stages <= 4; ++stages) for (int p : prods) for (int g = 0; g < 3; ++g)
            for (int sa = 0; sa <= sa_end[g]; ++sa) for (int sb = 0; sb <= sb_end[g]; ++sb) {
                const Tuple t{tile, sk, sa, sb, rows_a[g], rows_b[g], 1 + (n % 5), stages, p, c};
                if (ckopt_check_gemm_tuning(tile, sk, sa, sb, t.rows_a, t.rows_b, t.tile_group_m, stages, p, c, 256) != CKOPT_OK) continue;
                if (n++ % stride == 0) out.push_back(t);
            }
    }
    return out;
}

struct Device {
    DT *A = nullptr, *B = nullptr;
    DT_ACC *C = nullptr, *D = nullptr;
    size_t n;
    explicit Device(size_t elems) : n(elems) {
        HIP_OK(hipMalloc((void**)&A, n * sizeof(DT))); HIP_OK(hipMalloc((void**)&B, n * sizeof(DT)));
        HIP_OK(hipMalloc((void**)&C, n * sizeof(DT_ACC))); HIP_OK(hipMalloc((void**)&D, n * sizeof(DT_ACC)));
    }
    ~Device() { (void)hipFree(A); (void)hipFree(B); (void)hipFree(C); (void)hipFree(D); }
};

static void launch(const Device& d, float alpha, float beta, int dim, const Tuple& t, int cus) {
    ckopt::gemm_shmem_tc_async_opt_port<DT, DT_ACC>(d.A, d.B, d.C, d.D, alpha, beta, dim, dim, dim, t.tile_dim, t.segment_dim_k, t.bar_steps_a,
                                                     t.bar_steps_b, t.rows_a, t.rows_b, t.tile_group_m, t.num_stages, t.producers, t.consumers, cus);
}
// the same launch, waited for and checked: a bounded wait that was given up throws instead of leaving a wrong D behind
static void launch_checked(const Device& d, float alpha, float beta, int dim, const Tuple& t, int cus) {
    ckopt::checked(nullptr, [&] { launch(d, alpha, beta, dim, t, cus); });
}

// A = 1, B = 10, C = 1: every element of D is alpha * 10 * dim + beta (the reference's closed form)
static int correctness(int cus) {
    const int dim_max = 1024;
    const size_t n = (size_t)dim_max * dim_max;
    std::vector<DT> a(n), b(n);
    std::vector<DT_ACC> c(n), res(n);
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F16, a.data(), (int64_t)n, 1.f), "fill");
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F16, b.data(), (int64_t)n, 10.f), "fill");
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F32, c.data(), (int64_t)n, 1.f), "fill");
    Device d(n);
    HIP_OK(hipMemcpy(d.A, a.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.B, b.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.C, c.data(), n * sizeof(DT_ACC), hipMemcpyHostToDevice));
    int failed = 0, run = 0;
    unsigned lcg = 12345u;
    for (const Tuple& t : tuples(7)) {
        lcg = lcg * 1664525u + 1013904223u;
        const int dim = (run % 4 == 0) ? dim_max : std::max(t.tile_dim, (int)((lcg >> 8) % (dim_max + 1)) / t.tile_dim * t.tile_dim);
        HIP_OK(hipMemset(d.D, 0, n * sizeof(DT_ACC)));
        bool ok = true;
        try {
            launch_checked(d, 1.f, 1.f, dim, t, cus);
        } catch (const ckopt::DeviceStatusError&) {
            ok = false;
        }
        HIP_OK(hipMemcpy(res.data(), d.D, n * sizeof(DT_ACC), hipMemcpyDeviceToHost));
        const float want = 10.f * dim + 1.f;
        for (size_t i = 0; ok && i < (size_t)dim * dim; ++i) ok = std::fabs(res[i] - want) <= 0.001f;
        for (size_t i = (size_t)dim * dim; ok && i < n; ++i) ok = res[i] == 0.f;
        ++run;
        if (!ok) { ++failed; std::printf("FAILED dim %d ", dim); print_tuple(t); std::printf("\n"); }
    }
    std::printf("correctness: %d tuples, %d failed\n", run, failed);
    return failed;
}

// The same closed form through the port_0 launcher over its own legal set (matmul_shmem_tc_async_opt_port_0.cu:515-540,
// driver sweep :867): 1, 2, 4 and 8 producer warps, segment depths that are multiples of tile_dim / 2; and through the
// <half, half> instances of the port_0 and port_1 launchers (port_0.cu:866, :906; port_1.cu:1292, :1332), whose results
// 10 * dim + 1 are exact in fp16 up to dim 204.
static int correctness_port_0(int cus) {
    const int dim_max = 512;
    const size_t n = (size_t)dim_max * dim_max;
    std::vector<DT> a(n), b(n), c16(n), res16(n);
    std::vector<DT_ACC> c(n), res(n);
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F16, a.data(), (int64_t)n, 1.f), "fill");
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F16, b.data(), (int64_t)n, 10.f), "fill");
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F32, c.data(), (int64_t)n, 1.f), "fill");
    ckopt::check(ckopt_fill_constant(CKOPT_DT_F16, c16.data(), (int64_t)n, 1.f), "fill");
    Device d(n);
    DT *C16 = nullptr, *D16 = nullptr;
    HIP_OK(hipMalloc((void**)&C16, n * sizeof(DT))); HIP_OK(hipMalloc((void**)&D16, n * sizeof(DT)));
    HIP_OK(hipMemcpy(d.A, a.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.B, b.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.C, c.data(), n * sizeof(DT_ACC), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(C16, c16.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    int failed = 0, run = 0;
    const int tiles[] = {64, 128}, cons[] = {4, 8}, prods[] = {1, 2, 4, 8};
    for (int tile : tiles) for (int cw : cons) for (int p : prods) for (int sk = tile / 2; sk <= 128; sk *= 2) for (int stages = 1; stages <= 3; ++stages) {
        // the caller's job, as in the reference's drivers (port_0.cu:642-645): only tuples whose ring fits the shared memory
        if (sk < 32 || ckopt::get_shmem_req<DT, DT_ACC>(tile, sk, 0, 0, tile, tile, stages, cw) > 160 * 1024) continue;
        const int dim = run % 3 == 0 ? dim_max : (1 + run % (dim_max / tile)) * tile;
        HIP_OK(hipMemset(d.D, 0, n * sizeof(DT_ACC)));
        ckopt::gemm_shmem_tc_async_opt_port<DT, DT_ACC>(d.A, d.B, d.C, d.D, 1.f, 1.f, dim, dim, dim, tile, sk, 1 + run % 4, stages, p, cw, cus);
        HIP_OK(hipMemcpy(res.data(), d.D, n * sizeof(DT_ACC), hipMemcpyDeviceToHost));
        const float want = 10.f * dim + 1.f;
        bool ok = ckopt_device_status(nullptr) == 0;
        for (size_t i = 0; ok && i < (size_t)dim * dim; ++i) ok = std::fabs(res[i] - want) <= 0.001f;
        for (size_t i = (size_t)dim * dim; ok && i < n; ++i) ok = res[i] == 0.f;
        ++run;
        if (!ok) { ++failed; std::printf("FAILED port_0 dim %d (%d, %d, %d, %d, %d, %d)\n", dim, tile, sk, 1 + (run - 1) % 4, stages, p, cw); }
    }
    // <half, half>: alpha, beta, C and D in fp16
    const int dim16 = 192;
    for (int p : prods) for (int which = 0; which < 2; ++which) {
        if (which == 1 && p == 1) continue;   // port_1 takes 2, 4 or 8 producer warps
        HIP_OK(hipMemset(D16, 0, n * sizeof(DT)));
        if (which == 0)
            ckopt::gemm_shmem_tc_async_opt_port<DT, DT>(d.A, d.B, C16, D16, (DT)1.f, (DT)1.f, dim16, dim16, dim16, 64, 64, 2, 2, p, 4, cus);
        else
            ckopt::gemm_shmem_tc_async_opt_port<DT, DT>(d.A, d.B, C16, D16, (DT)1.f, (DT)1.f, dim16, dim16, dim16, 64, 64, 32, 32, 2, 2, p, 4, cus);
        HIP_OK(hipMemcpy(res16.data(), D16, n * sizeof(DT), hipMemcpyDeviceToHost));
        bool ok = ckopt_device_status(nullptr) == 0;
        for (size_t i = 0; ok && i < (size_t)dim16 * dim16; ++i) ok = (float)res16[i] == 10.f * dim16 + 1.f;
        ++run;
        if (!ok) { ++failed; std::printf("FAILED <half, half> %s, %d producer warps\n", which ? "port_1" : "port_0", p); }
    }
    (void)hipFree(C16); (void)hipFree(D16);
    std::printf("correctness, port_0 legal set and <half, half> of port_0 / port_1: %d launches, %d failed\n", run, failed);
    return failed;
}

// uniform[-1,1) operands; number of elements with |cpu - gpu| > 0.1 (the reference's accuracy count) must be 0.
// T is the element type (fp16 or bf16); M, N, K need not be multiples of anything.
template <typename T>
static int accuracy_shape(int M, int N, int K, int stride, int cus) {
    const int dtype = ckopt::dtype_of<T>::value;
    std::vector<T> a((size_t)M * K), b((size_t)N * K);
    std::vector<DT_ACC> c((size_t)M * N), res((size_t)M * N), ref((size_t)M * N);
    ckopt::check(ckopt_fill_uniform(dtype, a.data(), (int64_t)a.size(), 77, 0, -1.f, 1.f), "fill");
    ckopt::check(ckopt_fill_uniform(dtype, b.data(), (int64_t)b.size(), 77, 1, -1.f, 1.f), "fill");
    ckopt::check(ckopt_fill_uniform(CKOPT_DT_F32, c.data(), (int64_t)c.size(), 77, 2, -1.f, 1.f), "fill");
    if (oracle_gemm_blocked(dtype, (const uint16_t*)a.data(), (const uint16_t*)b.data(), c.data(), ref.data(), 1.f, 1.f, M, N, K, 0, M, 0) != 0) return 1;
    T *dA = nullptr, *dB = nullptr;
    DT_ACC *dC = nullptr, *dD = nullptr;
    HIP_OK(hipMalloc((void**)&dA, a.size() * sizeof(T))); HIP_OK(hipMalloc((void**)&dB, b.size() * sizeof(T)));
    HIP_OK(hipMalloc((void**)&dC, c.size() * sizeof(DT_ACC))); HIP_OK(hipMalloc((void**)&dD, c.size() * sizeof(DT_ACC)));
    HIP_OK(hipMemcpy(dA, a.data(), a.size() * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dB, b.data(), b.size() * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dC, c.data(), c.size() * sizeof(DT_ACC), hipMemcpyHostToDevice));
    int failed = 0, run = 0;
    for (const Tuple& t : tuples(stride)) {
        HIP_OK(hipMemset(dD, 0, c.size() * sizeof(DT_ACC)));
        ckopt::gemm_shmem_tc_async_opt_port<T, DT_ACC>(dA, dB, dC, dD, 1.f, 1.f, M, N, K, t.tile_dim, t.segment_dim_k, t.bar_steps_a, t.bar_steps_b,
                                                      t.rows_a, t.rows_b, t.tile_group_m, t.num_stages, t.producers, t.consumers, cus);
        HIP_OK(hipMemcpy(res.data(), dD, c.size() * sizeof(DT_ACC), hipMemcpyDeviceToHost));
        const long long bad = (long long)oracle_count_incorrect(ref.data(), res.data(), (int64_t)c.size(), 0.1f);
        ++run;
        if (bad != 0 || ckopt_device_status(nullptr) != 0) { ++failed; print_tuple(t); std::printf(": %lld incorrect\n", bad); }
    }
    (void)hipFree(dA); (void)hipFree(dB); (void)hipFree(dC); (void)hipFree(dD);
    std::printf("accuracy: %s %d x %d x %d, %d tuples, %d with incorrect elements\n", dtype == CKOPT_DT_F16 ? "fp16" : "bf16", M, N, K, run, failed);
    return failed;
}

// The <DT, DT> instance (port_2.cu:968-1055, run by the reference's main at :1519, :1533, :1545, :1559): C and D in the
// operands' 16-bit type, alpha = beta = 1. Checked against the fp32 oracle on the same operands; the bound is the
// reference's 0.1 plus one 16-bit rounding of a result of that size (sums of K products of uniform[-1,1) values).
template <typename T>
static int accuracy_shape_16_bit_cd(int M, int N, int K, int stride, int cus, float atol) {
    const int dtype = ckopt::dtype_of<T>::value;
    std::vector<T> a((size_t)M * K), b((size_t)N * K), c16((size_t)M * N), res((size_t)M * N);
    std::vector<float> c((size_t)M * N), ref((size_t)M * N);
    ckopt::check(ckopt_fill_uniform(dtype, a.data(), (int64_t)a.size(), 79, 0, -1.f, 1.f), "fill");
    ckopt::check(ckopt_fill_uniform(dtype, b.data(), (int64_t)b.size(), 79, 1, -1.f, 1.f), "fill");
    ckopt::check(ckopt_fill_uniform(dtype, c16.data(), (int64_t)c16.size(), 79, 2, -1.f, 1.f), "fill");
    for (size_t i = 0; i < c.size(); ++i) c[i] = ckopt::to_float(c16[i]);
    if (oracle_gemm_blocked(dtype, (const uint16_t*)a.data(), (const uint16_t*)b.data(), c.data(), ref.data(), 1.f, 1.f, M, N, K, 0, M, 0) != 0) return 1;
    T *dA = nullptr, *dB = nullptr, *dC = nullptr, *dD = nullptr;
    HIP_OK(hipMalloc((void**)&dA, a.size() * sizeof(T))); HIP_OK(hipMalloc((void**)&dB, b.size() * sizeof(T)));
    HIP_OK(hipMalloc((void**)&dC, c16.size() * sizeof(T))); HIP_OK(hipMalloc((void**)&dD, c16.size() * sizeof(T)));
    HIP_OK(hipMemcpy(dA, a.data(), a.size() * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dB, b.data(), b.size() * sizeof(T), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dC, c16.data(), c16.size() * sizeof(T), hipMemcpyHostToDevice));
    T one;
    if constexpr (std::is_same<T, ckopt::half_t>::value) one = (ckopt::half_t)1.f; else one = ckopt::bfloat16_t{0x3f80};
    int failed = 0, run = 0;
    for (const Tuple& t : tuples(stride)) {
        HIP_OK(hipMemset(dD, 0xff, c16.size() * sizeof(T)));
        ckopt::gemm_shmem_tc_async_opt_port<T, T>(dA, dB, dC, dD, one, one, M, N, K, t.tile_dim, t.segment_dim_k, t.bar_steps_a, t.bar_steps_b,
                                                  t.rows_a, t.rows_b, t.tile_group_m, t.num_stages, t.producers, t.consumers, cus);
        HIP_OK(hipMemcpy(res.data(), dD, c16.size() * sizeof(T), hipMemcpyDeviceToHost));
        long long bad = 0;
        for (size_t i = 0; i < res.size(); ++i) bad += !(std::fabs(ckopt::to_float(res[i]) - ref[i]) <= atol);
        ++run;
        if (bad != 0 || ckopt_device_status(nullptr) != 0) { ++failed; print_tuple(t); std::printf(": %lld incorrect\n", bad); }
    }
    (void)hipFree(dA); (void)hipFree(dB); (void)hipFree(dC); (void)hipFree(dD);
    std::printf("accuracy: <%s, %s> %d x %d x %d, %d tuples, %d with incorrect elements\n", dtype == CKOPT_DT_F16 ? "fp16" : "bf16",
                dtype == CKOPT_DT_F16 ? "fp16" : "bf16", M, N, K, run, failed);
    return failed;
}

static int accuracy(int cus) {
    int failed = accuracy_shape<ckopt::half_t>(512, 512, 512, 23, cus);        // the reference's own accuracy size
    failed += accuracy_shape<ckopt::bfloat16_t>(512, 512, 512, 41, cus);
    failed += accuracy_shape<ckopt::half_t>(500, 392, 520, 41, cus);           // ragged in every dimension, K not a multiple of 64
    failed += accuracy_shape<ckopt::bfloat16_t>(333, 257, 1001, 67, cus);      // rows off 16-byte boundaries: zero-padded copies
    // results reach about 60 in magnitude: one fp16 rounding there is at most 0.016, one bf16 rounding 0.125
    failed += accuracy_shape_16_bit_cd<ckopt::half_t>(512, 512, 512, 29, cus, 0.1f + 0.016f);
    failed += accuracy_shape_16_bit_cd<ckopt::bfloat16_t>(512, 512, 512, 43, cus, 0.1f + 0.125f);
    failed += accuracy_shape_16_bit_cd<ckopt::half_t>(500, 392, 520, 47, cus, 0.1f + 0.016f);
    return failed;
}

static int performance(int dim, int cus) {
    const size_t n = (size_t)dim * dim;
    std::vector<DT> a(n), b(n);
    ckopt::check(ckopt_fill_uniform(CKOPT_DT_F16, a.data(), (int64_t)n, 78, 0, -1.f, 1.f), "fill");
    ckopt::check(ckopt_fill_uniform(CKOPT_DT_F16, b.data(), (int64_t)n, 78, 1, -1.f, 1.f), "fill");
    Device d(n);
    HIP_OK(hipMemcpy(d.A, a.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(d.B, b.data(), n * sizeof(DT), hipMemcpyHostToDevice));
    HIP_OK(hipMemset(d.C, 0, n * sizeof(DT_ACC)));
    hipEvent_t start, stop;
    HIP_OK(hipEventCreate(&start)); HIP_OK(hipEventCreate(&stop));
    const int num_reps = 20;
    const Tuple sweep[] = {{256, 64, 0, 0, 256, 256, 4, 2, 2, 8}, {256, 64, 0, 0, 256, 256, 4, 2, 0, 8}, {256, 32, 0, 0, 256, 256, 4, 4, 4, 8},
                           {256, 32, 0, 0, 256, 256, 4, 5, 0, 8}, {256, 64, 2, 1, 64, 128, 4, 2, 2, 8}, {128, 64, 0, 0, 128, 128, 4, 4, 2, 8},
                           {128, 64, 2, 2, 32, 64, 4, 4, 4, 8}, {128, 64, 1, 3, 16, 16, 4, 4, 4, 8}, {128, 128, 0, 0, 128, 128, 4, 2, 0, 8},
                           {64, 64, 0, 0, 64, 64, 4, 4, 2, 4}};
    for (const Tuple& t : sweep) {
        if (ckopt_check_gemm_tuning(t.tile_dim, t.segment_dim_k, t.bar_steps_a, t.bar_steps_b, t.rows_a, t.rows_b, t.tile_group_m, t.num_stages,
                                    t.producers, t.consumers, cus) != CKOPT_OK) continue;
        launch(d, 1.f, 0.f, dim, t, cus);
        HIP_OK(hipEventRecord(start, nullptr));
        for (int j = 0; j < num_reps; ++j) launch(d, 1.f, 0.f, dim, t, cus);
        HIP_OK(hipEventRecord(stop, nullptr));
        HIP_OK(hipEventSynchronize(stop));
        float ms = 0.f;
        HIP_OK(hipEventElapsedTime(&ms, start, stop));
        print_tuple(t);
        std::printf(": %.2f\n", 2.0 * dim * dim * 1e-9 * dim * num_reps / ms);
    }
    const int st = ckopt_device_status(nullptr);
    HIP_OK(hipEventDestroy(start)); HIP_OK(hipEventDestroy(stop));
    return st != 0;
}

int main(int argc, char** argv) {
    const char* what = argc > 1 ? argv[1] : "all";
    int cus = 0;
    HIP_OK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0));
    int failed = 0;
    try {
        if (!std::strcmp(what, "correctness") || !std::strcmp(what, "all")) failed += correctness(cus) + correctness_port_0(cus);
        if (!std::strcmp(what, "accuracy") || !std::strcmp(what, "all")) failed += accuracy(cus);
        if (!std::strcmp(what, "performance") || !std::strcmp(what, "all")) failed += performance(argc > 2 ? std::atoi(argv[2]) : 4096, cus);
    } catch (const ckopt::Error& e) {
        std::fprintf(stderr, "%s (code %d)\n", e.what(), e.code);
        return 3;
    }
    std::printf(failed ? "FAILED\n" : "PASSED\n");
    return failed ? 1 : 0;
}

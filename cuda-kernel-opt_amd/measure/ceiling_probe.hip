// Measurement kernel, no counterpart in the reference: the inner loop of the 256 x 256 tile GEMM with
// everything removed that a real GEMM adds on top - no flags, no barrier, no waiting for data, no
// epilogue. Eight waves per CU; per wave and k-step 32 MFMAs (16x16x32 f16) on fragments fetched from
// LDS one k-step ahead (12 ds_read_b128 at the fragment addresses of the seg_k 64 ring), optionally
// four direct-to-LDS loads of 8 rows x 128 bytes that stream through an L2-resident window. What it
// sustains is the ceiling a kernel of this shape can reach on the device at hand: with constant
// operand values the matrix cores run near their nominal rate, with random operand values the
// device's power limit lowers the clock well below it.
// A second shape of the same loop answers whether bigger wave tiles would pay: four waves per CU (one per SIMD, all
// 512 registers each) with wave tiles of 128 x 128 - 64 MFMAs on 16 fragment reads per k-step, a third fewer LDS
// bytes per MFMA than the eight-wave shape's 32 on 12, at the price of one wave per SIMD.
#include <hip/hip_runtime.h>

#include <stdint.h>

#include "../csrc/ck_common.h"

namespace {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define CKP_LDS __attribute__((address_space(3)))

constexpr int PROBE_LDS_BYTES = 128 * 1024;
constexpr uint32_t WINDOW_BYTES = 512u * 1024u;  // per workgroup class; 4 classes per XCD stay L2 resident
constexpr int WINDOW_CLASSES = 32;

__device__ __forceinline__ void probe_dma_b128(i32x4 rsrc, uint32_t lds_dst, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" : : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

template <int WAVES, bool RANDOM, bool LOADS>
__global__ __launch_bounds__(WAVES * 64) void ceiling_probe_kernel(const char* window, int ksteps, float* sink) {
    constexpr int NT = WAVES * 64;
    constexpr int WTC = 8, WTR = 32 / WAVES;         // 16 x 16 blocks per wave tile: 4 x 8 (eight waves) or 8 x 8 (four)
    constexpr int NF = WTR + WTC;                    // fragments per k-step
    constexpr int FPJ = (NF + WTC - 1) / WTC;        // of which fetched per column of MFMAs
    constexpr int LOADS_PER_KSTEP = 32 / WAVES;      // 1 KiB loads per wave and k-step: 32 KiB per workgroup either way
    static_assert(WAVES == 8 || WAVES == 4, "two waves per SIMD with 64 x 128 wave tiles, or one with 128 x 128");
    extern __shared__ __attribute__((aligned(1024))) char probe_smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(CKP_LDS char*)probe_smem;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    // the first 64 KiB play the ring stage the fragments come from, the second 64 KiB receive the loads
    for (int i = threadIdx.x; i < PROBE_LDS_BYTES / 4; i += NT) {
        uint32_t v = 0x3c003c00u;  // two fp16 ones
        if (RANDOM) {
            uint32_t h = (uint32_t)i * 2654435761u + blockIdx.x * 40503u;
            h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
            // two fp16 values of random sign and mantissa, magnitude 2^-5 .. 2^-1
            v = ((h & 0x83ffu) | ((10u + ((h >> 10) & 3u)) << 10)) | ((((h >> 16) & 0x83ffu) | ((10u + ((h >> 26) & 3u)) << 10)) << 16);
        }
        ((CKP_LDS uint32_t*)probe_smem)[i] = v;
    }
    const uint64_t p = (uint64_t)(uintptr_t)(window + (size_t)(blockIdx.x % WINDOW_CLASSES) * WINDOW_BYTES);
    i32x4 rsrc;
    rsrc[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    rsrc[1] = __builtin_amdgcn_readfirstlane((int)((p >> 32) & 0xffffu));
    rsrc[2] = (int)WINDOW_BYTES;
    rsrc[3] = 0x00020000;
    // 8 rows x 128 bytes per wave load, rows 16 KiB apart (the pitch of a K = 8192 fp16 operand)
    const uint32_t voff = (uint32_t)(lane / 8) * 16384u + (uint32_t)(lane % 8) * 16u;
    const int lr = lane & 15, lg = lane >> 4, key = (lr >> 1) % 8;
    const uint32_t a_lane = lds0 + (uint32_t)((wave / 2) * WTR * 16 + lr) * 128u + (uint32_t)((lg ^ key) * 16);
    const uint32_t b_lane = lds0 + 32768u + (uint32_t)((wave % 2) * 128 + lr) * 128u + (uint32_t)((lg ^ key) * 16);
    u32x4 fr[2][NF];
#pragma unroll
    for (int i = 0; i < NF; ++i) {
        fr[0][i] = u32x4{0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};
        fr[1][i] = fr[0][i];
    }
    f32x4 acc[WTR][WTC];
#pragma unroll
    for (int i = 0; i < WTR; ++i)
#pragma unroll
        for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
    uint32_t gpos = 0;
    for (int it = 0; it < ksteps; it += 2) {
#pragma unroll
        for (int P = 0; P < 2; ++P) {
#pragma unroll
            for (int j = 0; j < WTC; ++j) {
#pragma unroll
                for (int q = 0; q < FPJ; ++q) {
                    const int f = j * FPJ + q;
                    if (f < WTR) fr[1 - P][f] = *(const CKP_LDS u32x4*)(uintptr_t)((a_lane ^ (uint32_t)(P * 64)) + f * 2048);
                    else if (f < NF) fr[1 - P][f] = *(const CKP_LDS u32x4*)(uintptr_t)((b_lane ^ (uint32_t)(P * 64)) + (f - WTR) * 2048);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (LOADS) {
                    // distinct lines per wave and load; the window (4 row groups x 16 KiB of k) wraps
#pragma unroll
                    for (int d = j * LOADS_PER_KSTEP / WTC; d < (j + 1) * LOADS_PER_KSTEP / WTC; ++d)
                        probe_dma_b128(rsrc, lds0 + 65536u + (uint32_t)(wave * LOADS_PER_KSTEP + d) * 1024u, voff,
                                       ((gpos + (uint32_t)(wave * LOADS_PER_KSTEP + d) * 128u) & 0x3fffu) + ((gpos >> 14) & 3u) * 131072u);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < WTR; ++i)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, fr[P][WTR + j]), __builtin_bit_cast(f16x8, fr[P][i]), acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            // the loads of the two k-steps before this one may still fly
            if (LOADS) {
                if (LOADS_PER_KSTEP == 4) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
                else asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            }
            gpos += 32u * 128u;
        }
    }
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < WTR; ++i)
#pragma unroll
        for (int j = 0; j < WTC; ++j) s += acc[i][j][0] + acc[i][j][3];
    sink[blockIdx.x * NT + threadIdx.x] = s;
}

template <int WAVES, bool RANDOM, bool LOADS>
hipError_t launch_probe(int cus, const char* window, int ksteps, float* sink, hipStream_t s) {
    auto kern = ceiling_probe_kernel<WAVES, RANDOM, LOADS>;
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, ck::LDS_BYTES_PER_CU);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3(cus), dim3(WAVES * 64), PROBE_LDS_BYTES, s, window, ksteps, sink);
    return hipGetLastError();
}

// The fp32 vector ALUs alone: what the matmul_shmem kernel's multiply-add stream sustains when nothing feeds it (no
// LDS reads, no global loads, no barrier). 512 threads per workgroup, four workgroups per CU (eight waves per SIMD, the
// kernel's occupancy); per thread an 8 x 4 accumulator micro-tile in registers and 32 v_fmac_f32 per iteration on 8 + 4
// operand registers. Accumulator rows and the B values are even-aligned runs of four registers with column j of an
// accumulator row in element j + 1, as in the kernel, so that no multiply-add has its three registers in one bank
// (those run at half rate).
typedef float probe_f4 __attribute__((ext_vector_type(4)));
template <bool RANDOM>
__global__ __launch_bounds__(512) void valu_probe_kernel(int iters, float* sink) {
    const uint32_t tid = blockIdx.x * 512u + threadIdx.x;
    float a[8];
    probe_f4 b, acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t h = (tid * 8u + i) * 2654435761u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        a[i] = RANDOM ? (float)(h >> 8) * (2.0f / 16777216.0f) - 1.0f : 1.0f;
        acc[i] = probe_f4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t h = (tid * 4u + j + 977u) * 2246822519u;
        h ^= h >> 15; h *= 2654435761u; h ^= h >> 13;
        b[j] = RANDOM ? (float)(h >> 8) * (2.0f / 16777216.0f) - 1.0f : 1.0f;
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(acc[i]));
        asm volatile("" : "+v"(b));
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            asm volatile("" : "+v"(a[i]));
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][(j + 1) % 4] = __builtin_fmaf(a[i], b[j], acc[i][(j + 1) % 4]);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    sink[tid] = s;
}

}  // namespace

// TFLOP/s of the bare fp32 multiply-add stream on every CU (see valu_probe_kernel): iters iterations of 32
// multiply-adds per thread after a warm-up; random_operands selects random instead of constant operand values.
extern "C" int ckmeasure_valu_ceiling(int random_operands, int iters, double* tflops_out) {
    using namespace ck;
    if (!tflops_out || iters < 2 || iters > (1 << 28)) return CK_ERR_BAD_PARAM;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return CK_ERR_HIP;
    const int blocks = cus * 4;
    float* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = CK_ERR_HIP;
    do {
        if (hipMalloc((void**)&sink, (size_t)blocks * 512 * sizeof(float)) != hipSuccess) break;
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) break;
        auto go = [&](int n) {
            if (random_operands) hipLaunchKernelGGL(valu_probe_kernel<true>, dim3(blocks), dim3(512), 0, nullptr, n, sink);
            else hipLaunchKernelGGL(valu_probe_kernel<false>, dim3(blocks), dim3(512), 0, nullptr, n, sink);
            return hipGetLastError();
        };
        if (go(iters / 4 + 2) != hipSuccess) break;   // warm-up
        if (hipEventRecord(e0, nullptr) != hipSuccess) break;
        if (go(iters) != hipSuccess) break;
        if (hipEventRecord(e1, nullptr) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) break;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess || ms <= 0.f) break;
        *tflops_out = (double)blocks * 512.0 * iters * 32.0 * 2.0 / (ms * 1e-3) * 1e-12;
        rc = CK_OK;
    } while (false);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (sink) (void)hipFree(sink);
    return rc;
}

// Built into lib/libckmeasure.so, a measurement aid that bench.py loads next to the product library (which does not
// contain it). random_operands: random instead of constant fragment values; with_loads: also the direct-to-LDS loads;
// runs ksteps k-steps per wave on every CU after a warm-up, allocates and frees its own buffers, synchronises, and
// returns the rate in TFLOP/s. waves: 8 (wave tiles of 64 x 128, the GEMM kernels' shape) or 4 (128 x 128).
extern "C" int ckmeasure_mfma_ceiling_shape(int waves, int random_operands, int with_loads, int ksteps, double* tflops_out) {
    using namespace ck;
    if (!tflops_out || ksteps < 2 || ksteps > (1 << 26) || !(waves == 8 || waves == 4)) return CK_ERR_BAD_PARAM;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return CK_ERR_HIP;
    // the last load of a window reaches 7 rows x 16 KiB + 3 row groups x 128 KiB + 16 KiB past its start
    const size_t window_bytes = (size_t)WINDOW_CLASSES * WINDOW_BYTES + (1u << 20);
    char* window = nullptr;
    float* sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = CK_ERR_HIP;
    do {
        if (hipMalloc((void**)&window, window_bytes) != hipSuccess) break;
        if (hipMalloc((void**)&sink, (size_t)cus * 512 * sizeof(float)) != hipSuccess) break;
        if (hipMemset(window, 0, window_bytes) != hipSuccess) break;
        if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) break;
        auto go = [&](int n) {
            if (waves == 4) {
                if (random_operands) return with_loads ? launch_probe<4, true, true>(cus, window, n, sink, nullptr) : launch_probe<4, true, false>(cus, window, n, sink, nullptr);
                return with_loads ? launch_probe<4, false, true>(cus, window, n, sink, nullptr) : launch_probe<4, false, false>(cus, window, n, sink, nullptr);
            }
            if (random_operands) return with_loads ? launch_probe<8, true, true>(cus, window, n, sink, nullptr) : launch_probe<8, true, false>(cus, window, n, sink, nullptr);
            return with_loads ? launch_probe<8, false, true>(cus, window, n, sink, nullptr) : launch_probe<8, false, false>(cus, window, n, sink, nullptr);
        };
        if (go(ksteps / 8 + 2) != hipSuccess) break;   // warm-up
        if (hipEventRecord(e0, nullptr) != hipSuccess) break;
        if (go(ksteps) != hipSuccess) break;
        if (hipEventRecord(e1, nullptr) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) break;
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess || ms <= 0.f) break;
        const int n = (ksteps + 1) / 2 * 2;
        // per CU and k-step: 256 MFMAs (8 waves x 32 or 4 x 64) x 16*16*32*2 flop = a 256 x 256 x 32 block
        *tflops_out = (double)cus * n * 256.0 * 16384.0 / (ms * 1e-3) * 1e-12;
        rc = CK_OK;
    } while (false);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (window) (void)hipFree(window);
    if (sink) (void)hipFree(sink);
    return rc;
}

extern "C" int ckmeasure_mfma_ceiling(int random_operands, int with_loads, int ksteps, double* tflops_out) {
    return ckmeasure_mfma_ceiling_shape(8, random_operands, with_loads, ksteps, tflops_out);
}

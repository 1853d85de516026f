// matmul_shmem for gfx950: C = A * B on the vector ALUs only (no matrix cores).
//
// Reference role: matmul_shmem_3_kernel, matmul_shmem.cu:38-102 - one tile_dim x tile_dim C tile per
// workgroup, tile_dim/block_rows accumulators per thread, operands staged through shared memory.
// Here the accumulators of a thread form an RM x RN register micro-tile (outer product per k, RM+RN
// LDS values per RM*RN FMAs instead of the reference's 2 LDS reads per FMA), operand tiles are
// TILE x 16 slices stored k-major in LDS (so a thread's RM / RN values are contiguous and come in
// with ds_read_b128), and the next slice is fetched from global memory into registers while the
// current one is being multiplied (double-buffered LDS, one workgroup barrier per slice).
//
// Every output element is a single accumulator that sees k in ascending order, one fused
// multiply-add per k, so the fp32 result is bit-identical to a sequential fmaf loop and the int32
// result is exact.
#ifndef CK_SIMT_KERNEL_HIP_H
#define CK_SIMT_KERNEL_HIP_H

#include <hip/hip_runtime.h>
#include "ck_common.h"

namespace ck {

struct SimtArgs {
    const void* A;
    const void* B;
    void* C;
    int M, N, K;
};

template <typename DT> struct SimtIo;
template <> struct SimtIo<float> {
    static constexpr int VEC = 4;
    typedef float acc_t;
    static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
        const float4 x = *reinterpret_cast<const float4*>(p);
        v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    }
    static __device__ __forceinline__ float out(float x) { return x; }
    static __device__ __forceinline__ float mad(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
};
template <> struct SimtIo<int> {
    static constexpr int VEC = 4;
    typedef int acc_t;
    static __device__ __forceinline__ void load(const int* p, int (&v)[4]) {
        const int4 x = *reinterpret_cast<const int4*>(p);
        v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    }
    static __device__ __forceinline__ int out(int x) { return x; }
    static __device__ __forceinline__ int mad(int a, int b, int c) { return a * b + c; }
};
template <> struct SimtIo<_Float16> {
    static constexpr int VEC = 8;
    typedef float acc_t;
    static __device__ __forceinline__ void load(const _Float16* p, float (&v)[8]) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 x = *reinterpret_cast<const h8*>(p);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)x[i];
    }
    static __device__ __forceinline__ _Float16 out(float x) { return (_Float16)x; }
    static __device__ __forceinline__ float mad(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
};

// BT: B is given transposed (N x K row-major); otherwise K x N row-major as in the reference.
template <typename DT, int TILE, int RM, int RN, bool BT>
__global__ __launch_bounds__(TILE * TILE / (RM * RN)) void matmul_shmem_kernel(const SimtArgs g) {
    typedef typename SimtIo<DT>::acc_t ACC;
    constexpr int KT = SIMT_KT;
    constexpr int VEC = SimtIo<DT>::VEC;
    constexpr int NT = TILE * TILE / (RM * RN);   // threads
    constexpr int LD = TILE + SIMT_PAD;           // LDS row pitch (elements), k-major
    constexpr int TX = TILE / RN;                 // threads along N
    constexpr int CPRK = KT / VEC;                // 16-byte chunks per row of a row-major (rows x KT) slice
    constexpr int CH_RK = TILE * CPRK;            // chunks of such a slice
    constexpr int IT_RK = (CH_RK + NT - 1) / NT;
    constexpr int CPRN = TILE / VEC;              // chunks per k-row of a (KT x TILE) slice of untransposed B
    constexpr int CH_KN = KT * CPRN;
    constexpr int IT_KN = (CH_KN + NT - 1) / NT;
    constexpr int IT_B = BT ? IT_RK : IT_KN;
    // How far the k loop of a slice is unrolled. All 16 steps let the scheduler hoist every LDS read of the
    // slice: 240-256 registers for the 32- and 64-accumulator micro-tiles (1-2 waves per SIMD), spills with
    // 1024 threads (128 registers each). 8 steps keep those at 64-120 registers, 4 and more waves per SIMD
    // (fp32 4096^3, 128 tile, 32 accumulators: 90 TFLOP/s against 70); the small tile is better unrolled whole.
    constexpr int K_UNROLL = NT >= 1024 ? 4 : (TILE == 32 ? KT : 8);

    extern __shared__ __attribute__((aligned(16))) char ck_simt_smem[];
    ACC* lds = reinterpret_cast<ACC*>(ck_simt_smem);
    // [buf][operand][k][LD]
    auto a_s = [&](int buf) { return lds + (buf * 2 + 0) * KT * LD; };
    auto b_s = [&](int buf) { return lds + (buf * 2 + 1) * KT * LD; };

    const DT* A = static_cast<const DT*>(g.A);
    const DT* B = static_cast<const DT*>(g.B);
    DT* C = static_cast<DT*>(g.C);
    const int tid = threadIdx.x;
    const int tx = tid % TX, ty = tid / TX;
    // blockIdx.x walks C tile rows, blockIdx.y tile columns (matmul_shmem.cu:49-51)
    const int64_t m0 = (int64_t)blockIdx.x * TILE, n0 = (int64_t)blockIdx.y * TILE;
    const int K = g.K, N = g.N;

    // Register banks. A v_fmac_f32 whose three registers lie in the same bank (register number mod 4) issues
    // at half rate (register-only loops on this chip: 71 TFLOP/s with all three in one bank, 137-147 with any
    // other placement), and the allocator's natural layout puts a fifth of the multiply-adds there (the
    // accumulators of a row and the B values are both runs of four, so column j of each lands in the same bank).
    // A B value arrives in a 16-byte LDS read, an even-aligned run of four registers, so column j sits in bank
    // base + j with an even base. Accumulator rows are therefore kept as even-aligned runs of four as well (the
    // empty asm below pins them to such a run at the top of every slice), with column j stored in element j + 1:
    // base_acc + j + 1 and base_b + j then always differ, whatever the A register is.
    // Rows of two columns: the same with pairs (an 8-byte LDS read delivers an even-aligned pair).
    constexpr bool ROT = RN % 2 == 0;
    constexpr int VW = RN % 4 == 0 ? 4 : 2;       // registers per aligned run
    constexpr int RG = ROT ? RN / VW : 1;         // runs per accumulator row
    typedef ACC accv_t __attribute__((ext_vector_type(VW)));
    accv_t accq[RM][RG];
    ACC accs[ROT ? 1 : RM][ROT ? 1 : RN];
    auto acc_get = [&](int i, int j) -> ACC {
        if constexpr (ROT) return accq[i][j / VW][(j + 1) % VW];
        else return accs[i][j];
    };
    auto acc_set = [&](int i, int j, ACC v) {
        if constexpr (ROT) accq[i][j / VW][(j + 1) % VW] = v;
        else accs[i][j] = v;
    };
#pragma unroll
    for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < RN; ++j) acc_set(i, j, (ACC)0);

    ACC ra[IT_RK][VEC], rb[IT_B][VEC];

    auto fetch = [&](int k0) {
#pragma unroll
        for (int it = 0; it < IT_RK; ++it) {
            const int ch = it * NT + tid;
            if (CH_RK % NT == 0 || ch < CH_RK) {
                const int r = ch / CPRK, c = ch % CPRK;
                SimtIo<DT>::load(A + (m0 + r) * K + k0 + c * VEC, ra[it]);
            }
        }
#pragma unroll
        for (int it = 0; it < IT_B; ++it) {
            const int ch = it * NT + tid;
            if (BT) {
                if (CH_RK % NT == 0 || ch < CH_RK) {
                    const int r = ch / CPRK, c = ch % CPRK;
                    SimtIo<DT>::load(B + (n0 + r) * K + k0 + c * VEC, rb[it]);
                }
            } else {
                if (CH_KN % NT == 0 || ch < CH_KN) {
                    const int kk = ch / CPRN, c = ch % CPRN;
                    SimtIo<DT>::load(B + (int64_t)(k0 + kk) * N + n0 + c * VEC, rb[it]);
                }
            }
        }
    };
    auto stash = [&](int buf) {
        ACC* as = a_s(buf);
        ACC* bs = b_s(buf);
#pragma unroll
        for (int it = 0; it < IT_RK; ++it) {
            const int ch = it * NT + tid;
            if (CH_RK % NT == 0 || ch < CH_RK) {
                const int r = ch / CPRK, c = ch % CPRK;
#pragma unroll
                for (int e = 0; e < VEC; ++e) as[(c * VEC + e) * LD + r] = ra[it][e];
            }
        }
#pragma unroll
        for (int it = 0; it < IT_B; ++it) {
            const int ch = it * NT + tid;
            if (BT) {
                if (CH_RK % NT == 0 || ch < CH_RK) {
                    const int r = ch / CPRK, c = ch % CPRK;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) bs[(c * VEC + e) * LD + r] = rb[it][e];
                }
            } else {
                if (CH_KN % NT == 0 || ch < CH_KN) {
                    const int kk = ch / CPRN, c = ch % CPRN;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) bs[kk * LD + c * VEC + e] = rb[it][e];
                }
            }
        }
    };

    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += KT) {
        const bool more = k0 + KT < K;
        if (more) fetch(k0 + KT);
        if (ROT) {
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int q = 0; q < RG; ++q) asm volatile("" : "+v"(accq[i][q]));
        }
        const ACC* as = a_s(buf) + ty * RM;
        const ACC* bs = b_s(buf) + tx * RN;
#pragma unroll(K_UNROLL)
        for (int k = 0; k < KT; ++k) {
            ACC av[RM], bv[RN];
#pragma unroll
            for (int i = 0; i < RM; ++i) av[i] = as[k * LD + i];
#pragma unroll
            for (int j = 0; j < RN; ++j) bv[j] = bs[k * LD + j];
#pragma unroll
            for (int i = 0; i < RM; ++i)
#pragma unroll
                for (int j = 0; j < RN; ++j) acc_set(i, j, SimtIo<DT>::mad(av[i], bv[j], acc_get(i, j)));
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }

#pragma unroll
    for (int i = 0; i < RM; ++i) {
        DT* crow = C + (m0 + ty * RM + i) * N + n0 + tx * RN;
#pragma unroll
        for (int j = 0; j < RN; ++j) crow[j] = SimtIo<DT>::out(acc_get(i, j));
    }
}

}  // namespace ck
#endif  // CK_SIMT_KERNEL_HIP_H

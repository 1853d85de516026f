// The synchronous ancestor of the pipelined kernels, kept as their A/B partner (role of gemm_shmem_tc_kernel,
// matmul_shmem_tc.cu:105-231): no producer waves, ONE stage, no overlap of any kind. Per K segment every wave
// loads its share of the A and Bt tiles into LDS, all waves wait for their loads and meet at the workgroup
// barrier, every wave multiplies its wave tile out of LDS, and a second barrier frees the stage for the next
// segment (load, __syncthreads, mma, __syncthreads in the reference, matmul_shmem_tc.cu:176-209).
// Selected by num_producer_waves == 0 with num_stages == 1.
//
// Everything else is what the other kernels use, so that a difference in speed is the schedule's alone: the same
// direct-to-LDS 16-byte loads, the same unpadded XOR-swizzled rows, the same 16x16x32 MFMA wave tiles
// ((CW/2) x 2 waves over the tile), the same persistent grouped tile order and the same epilogue straight from
// the accumulators (the reference stages C and D through shared memory, matmul_shmem_tc.cu:140-166, :212-229).
// The instruction order inside a segment is left to the compiler.
#ifndef CK_GEMM_SYNC_KERNEL_HIP_H
#define CK_GEMM_SYNC_KERNEL_HIP_H

#include "gemm_fused_kernel.hip.h"

namespace ck {

template <typename DT, int TILE, int SEGK, int CW>
__global__ __launch_bounds__(CW * 64) void gemm_sync_kernel(const GemmArgs g) {
    constexpr int WTR = TILE / (CW / 2) / MFMA_M, WTC = TILE / 2 / MFMA_N;
    constexpr int CPR = SEGK / CHUNK_ELEMS;   // 16-byte chunks per LDS row
    constexpr int RB = SEGK * 2;              // bytes per LDS row
    constexpr int RPI = WAVE / CPR;           // rows one wave load covers
    constexpr int OPB = TILE * RB;            // one operand's tile
    constexpr int KSTEPS = SEGK / MFMA_K;
    constexpr int NI = TILE / RPI;            // wave loads per operand and segment

    extern __shared__ __attribute__((aligned(1024))) char ck_smem[];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(CK_LDS char*)ck_smem;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const unsigned long long clk0 = clock64(), wall0 = wall_clock64();

    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    const int64_t total_tiles = (int64_t)g.tiles_m * g.tiles_n;
    const uint32_t pitch32 = (uint32_t)g.K * 2u;
    const int lane_row = lane / CPR, lane_slot = lane % CPR;

    const int R = wave / 2, Cc = wave % 2;
    const int lr = lane & 15, lg = lane >> 4;

    for (int64_t tc = slot; tc < total_tiles; tc += grid) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
        const int row_a = rc.row * TILE, row_b = rc.col * TILE;
        const int ra = g.M - row_a < TILE ? g.M - row_a : TILE, rb = g.N - row_b < TILE ? g.N - row_b : TILE;
        const uint32_t nrec_a = (uint32_t)ra * pitch32, nrec_b = (uint32_t)rb * pitch32;
        const i32x4 rsrc_a = make_rsrc((const char*)g.A + (int64_t)row_a * pitch32, nrec_a);
        const i32x4 rsrc_b = make_rsrc((const char*)g.Bt + (int64_t)row_b * pitch32, nrec_b);

        f32x4 acc[WTR][WTC];
#pragma unroll
        for (int i = 0; i < WTR; ++i)
#pragma unroll
            for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        for (int seg = 0; seg < g.nseg; ++seg) {
            const int k0 = seg * SEGK;
            // wave loads E = wave, wave + CW, ... of the 2 * NI that make up the segment (A first, then Bt). Lane
            // (lane_row, lane_slot) fetches the chunk that belongs at its linear LDS position under the swizzle;
            // rows past the tile's edge and k past K lie outside the descriptor and read as zeros.
            for (int E = wave; E < 2 * NI; E += CW) {
                const bool is_a = E < NI;
                const int e = is_a ? E : E - NI;
                const int row = e * RPI + lane_row;
                const int chunk = swizzle_slot(row, lane_slot, CPR, g.swizzle);
                uint32_t voff = (uint32_t)row * pitch32 + (uint32_t)(k0 + chunk * CHUNK_ELEMS) * 2u;
                if (k0 + chunk * CHUNK_ELEMS >= g.K) voff = is_a ? nrec_a : nrec_b;
                const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + (is_a ? 0u : (uint32_t)OPB) + (uint32_t)e * 1024u);
                if (is_a) dma_load_b128(rsrc_a, dst, voff, 0u);
                else dma_load_b128(rsrc_b, dst, voff, 0u);
            }
            wait_vmcnt_imm<0>();
            wg_barrier();
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                u32x4 fa[WTR], fb[WTC];
#pragma unroll
                for (int i = 0; i < WTR; ++i) {
                    const int row = R * WTR * 16 + i * 16 + lr;
                    fa[i] = *(const CK_LDS u32x4*)(uintptr_t)(lds_base + (uint32_t)(row * RB + swizzle_slot(row, ks * 4 + lg, CPR, g.swizzle) * CHUNK_BYTES));
                }
#pragma unroll
                for (int j = 0; j < WTC; ++j) {
                    const int row = Cc * WTC * 16 + j * 16 + lr;
                    fb[j] = *(const CK_LDS u32x4*)(uintptr_t)(lds_base + (uint32_t)(OPB + row * RB + swizzle_slot(row, ks * 4 + lg, CPR, g.swizzle) * CHUNK_BYTES));
                }
#pragma unroll
                for (int j = 0; j < WTC; ++j)
#pragma unroll
                    for (int i = 0; i < WTR; ++i) acc[i][j] = MfmaOp<DT>::run(fb[j], fa[i], acc[i][j]);
            }
            wait_lgkmcnt0();   // every fragment is in registers before the stage is overwritten
            wg_barrier();
        }

        const int m_base = rc.row * TILE + R * WTR * 16 + lr;
        const int n_base = rc.col * TILE + Cc * WTC * 16 + lg * 4;
        const bool vec_cols = g.vec_store && (rc.col + 1) * TILE <= g.N;
#pragma unroll
        for (int i = 0; i < WTR; ++i)
#pragma unroll
            for (int j = 0; j < WTC; ++j) epilogue_block<DT>(g, m_base + i * 16, n_base + j * 16, acc[i][j], vec_cols);
    }

    if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
        const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
        g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
        g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
    }
}

}  // namespace ck
#endif  // CK_GEMM_SYNC_KERNEL_HIP_H

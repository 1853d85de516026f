// Producer/consumer waves synchronised by the hardware workgroup barrier (tile granularity): dedicated
// producer waves stream the segments into the LDS ring, consumer waves multiply, and all of them meet at
// one s_barrier per segment instead of exchanging counters through LDS.
//
//   barrier B_G: every producer has seen its loads of segment G land (in-order vmcnt), every consumer has
//                finished reading segment G-1.
//   producers behind B_G: the stage of segment G-1 is free -> issue segment G-1+S into it (S-1 segments of slack)
//   consumers behind B_G: read and multiply segment G.
//
// Compared with the fused variant the waves that multiply never issue a load and never wait for one, so the
// epilogue's stores do not stand in front of any landing wait; compared with the counter protocol there is
// no polling. The price is the third wave per SIMD: 168 registers per wave, fragments not double-buffered.
#ifndef CK_GEMM_PCB_KERNEL_HIP_H
#define CK_GEMM_PCB_KERNEL_HIP_H

#include "gemm_fused_kernel.hip.h"

namespace ck {

template <typename DT, int TILE, int SEGK, int CW, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void gemm_pcb_kernel(const GemmArgs g) {
    constexpr int WTR = TILE / (CW / 2) / MFMA_M, WTC = TILE / 2 / MFMA_N;
    constexpr int CPR = SEGK / CHUNK_ELEMS;
    constexpr int RB = SEGK * 2;
    constexpr int RPI = WAVE / CPR;
    constexpr int OPB = TILE * RB;
    constexpr int KSTEPS = SEGK / MFMA_K;
    constexpr int NI = TILE / RPI;  // wave loads per operand stage
    constexpr int VAR = CPR == 4 ? 1 : CPR == 8 ? 2 : 4;

    extern __shared__ __attribute__((aligned(1024))) char ck_smem[];
    const uint32_t ring_base = (uint32_t)(uintptr_t)(CK_LDS char*)ck_smem;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const unsigned long long clk0 = clock64(), wall0 = wall_clock64();

    const int S = g.num_stages;
    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    const int total_tiles = g.tiles_m * g.tiles_n;
    const int my_tiles = slot < total_tiles ? (total_tiles - slot + grid - 1) / grid : 0;
    const int nseg = g.nseg;
    const int total_segs = my_tiles * nseg;
    const int P = g.pa + g.pb;

    if (wave < P) {
        // ---- producer wave q of px on one operand: wave loads E = q, q + px, ...
        const bool is_a = wave < g.pa;
        const int q = is_a ? wave : wave - g.pa;
        const int px = is_a ? g.pa : g.pb;
        const int nloads = NI / px;  // px divides NI (px in {1, 2, 4}, NI >= 4)
        const uint32_t pitch32 = (uint32_t)g.K * 2u;
        const int lane_row = lane / CPR, lane_slot = lane % CPR;
        // px <= 4 <= VAR's multiples only when px is a multiple of VAR; otherwise the key variant changes with E
        uint32_t lane_off[VAR];
        int lane_chunk[VAR];
#pragma unroll
        for (int v = 0; v < VAR; ++v) {
            lane_chunk[v] = swizzle_slot(v * RPI + lane_row, lane_slot, CPR, g.swizzle);
            lane_off[v] = (uint32_t)lane_row * pitch32 + (uint32_t)lane_chunk[v] * CHUNK_BYTES;
        }
        const uint32_t load_step = (uint32_t)RPI * pitch32;
        int l_tc = slot, l_seg = 0, l_stage = 0, issued = 0;
        i32x4 rsrc = {0, 0, 0, 0};
        uint32_t nrec = 0;
        bool full_rows = false;
        auto issue_segment = [&]() __attribute__((always_inline)) {
            if (l_seg == 0) {
                const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, l_tc);
                const int row0 = __builtin_amdgcn_readfirstlane((is_a ? rc.row : rc.col) * TILE);
                const int rows_total = is_a ? g.M : g.N;
                const int rows = rows_total - row0 < TILE ? rows_total - row0 : TILE;
                nrec = (uint32_t)rows * pitch32;
                full_rows = rows == TILE;
                rsrc = make_rsrc((const char*)(is_a ? g.A : g.Bt) + (int64_t)row0 * pitch32, nrec);
            }
            const uint32_t k0x2 = (uint32_t)l_seg * (SEGK * 2);
            const bool ktail = (l_seg + 1) * SEGK > g.K;
            const uint32_t dst0 = ring_base + (uint32_t)l_stage * (2 * OPB) + (is_a ? 0u : (uint32_t)OPB);
            if (full_rows && !ktail) {
                for (int i = 0; i < nloads; ++i) {
                    const int E = q + i * px;
                    uint32_t loff = lane_off[0];
#pragma unroll
                    for (int v = 1; v < VAR; ++v) {
                        if (E % VAR == v) loff = lane_off[v];
                    }
                    dma_load_b128(rsrc, dst0 + (uint32_t)E * 1024u, loff, (uint32_t)E * load_step + k0x2);
                }
            } else {
                for (int i = 0; i < nloads; ++i) {
                    const int E = q + i * px;
                    uint32_t loff = lane_off[0];
                    int lchunk = lane_chunk[0];
#pragma unroll
                    for (int v = 1; v < VAR; ++v) {
                        if (E % VAR == v) { loff = lane_off[v]; lchunk = lane_chunk[v]; }
                    }
                    uint32_t voff = loff + (uint32_t)E * load_step + k0x2;
                    if (ktail && (int)(k0x2 >> 1) + lchunk * CHUNK_ELEMS >= g.K) voff = nrec;
                    dma_load_b128(rsrc, dst0 + (uint32_t)E * 1024u, voff, 0u);
                }
            }
            ++issued;
            if (++l_seg == nseg) { l_seg = 0; l_tc += grid; }
            if (++l_stage == S) l_stage = 0;
        };
        for (int p = 0; p < S && issued < total_segs; ++p) issue_segment();
        for (int G = 0; G < total_segs; ++G) {
            wait_vmcnt_le((uint32_t)((issued - 1 - G) * nloads));  // my loads of segment G have landed
            wg_barrier();                                           // B_G
            if (G >= 1 && issued < total_segs) issue_segment();     // into the stage of segment G-1
        }
        wait_vmcnt_imm<0>();
    } else {
        // ---- consumer wave
        const int cw = wave - P;
        const int R = cw / 2, Cc = cw % 2;
        const int lr = lane & 15, lg = lane >> 4;
        const int key = g.swizzle ? swizzle_key(lr, CPR) : 0;
        const uint32_t a_lane = (uint32_t)(R * WTR * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);
        const uint32_t b_lane = (uint32_t)OPB + (uint32_t)(Cc * WTC * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);
        int stage = 0;
        int G = 0;  // segment being multiplied, over all tiles of this workgroup
        if (total_segs > 0) wg_barrier();  // B_0
        // B_{G+1} is met inside segment G's last k-step, as soon as the last fragments of the segment are in
        // registers: the MFMAs still to be issued cover the barrier and the producers' next loads.
        auto meet_next = [&](auto& a, auto& b) __attribute__((always_inline)) {
            use_fragment_array(a);
            use_fragment_array(b);
            if (G + 1 < total_segs) wg_barrier();
        };
        for (int t = 0; t < my_tiles; ++t) {
            const int tc = slot + t * grid;
            const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
            f32x4 acc[WTR][WTC];
#pragma unroll
            for (int i = 0; i < WTR; ++i)
#pragma unroll
                for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            for (int seg = 0; seg < nseg; ++seg) {
                const uint32_t st = ring_base + (uint32_t)stage * (2 * OPB);
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) {
                    const uint32_t pa_k = (st + a_lane) ^ (uint32_t)(ks * 64), pb_k = (st + b_lane) ^ (uint32_t)(ks * 64);
                    constexpr int JB = WTC > 4 ? RESIDENT_BT_FRAGS : WTC;
                    u32x4 a[WTR], b[JB];
#pragma unroll
                    for (int i = 0; i < WTR; ++i) a[i] = *(const CK_LDS u32x4*)(uintptr_t)(pa_k + i * 16 * RB);
#pragma unroll
                    for (int j = 0; j < JB; ++j) b[j] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + j * 16 * RB);
                    __builtin_amdgcn_sched_barrier(0);
                    if (ks == KSTEPS - 1 && JB == WTC) meet_next(a, b);
#pragma unroll
                    for (int j = 0; j < WTC; ++j) {
#pragma unroll
                        for (int i = 0; i < WTR; ++i) acc[i][j] = MfmaOp<DT>::run(b[j % JB], a[i], acc[i][j]);
                        if (j + JB < WTC) {
                            __builtin_amdgcn_sched_barrier(0);
                            b[j % JB] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + (j + JB) * 16 * RB);
                            __builtin_amdgcn_sched_barrier(0);
                            if (ks == KSTEPS - 1 && j + JB == WTC - 1) meet_next(a, b);
                        }
                    }
                }
                ++G;
                if (++stage == S) stage = 0;
            }
            const int m_base = rc.row * TILE + R * WTR * 16 + (int)(threadIdx.x & 15);
            const int n_base = rc.col * TILE + Cc * WTC * 16 + (int)((threadIdx.x >> 4) & 3) * 4;
            const bool vec_cols = g.vec_store && (rc.col + 1) * TILE <= g.N;
#pragma unroll
            for (int i = 0; i < WTR; ++i) {
#pragma unroll
                for (int j = 0; j < WTC; ++j) epilogue_block<DT>(g, m_base + i * 16, n_base + j * 16, acc[i][j], vec_cols);
            }
        }
        if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
            const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
            g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
            g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
        }
    }
}

}  // namespace ck
#endif  // CK_GEMM_PCB_KERNEL_HIP_H

// gemm_shmem_tc_async_opt_port with num_producer_waves == 0: the same LDS ring, direct-to-LDS loads,
// MFMA wave tiles and flag counters as the producer/consumer kernel, but every wave is both: it
// streams its 1/CW share of each K-segment into the ring and multiplies out of it.
//
// Why this variant exists: all waves of a kernel get the same register allocation, so dedicated
// producer waves push a 256 x 256 tile (8 consumer waves, 128 accumulator registers each) to three
// waves per SIMD and 168 registers per wave - no room to hold the next k-step's fragments while the
// current one is being multiplied, and the LDS latency of every k-step is exposed unless the
// partner wave happens to cover it. With 8 waves (two per SIMD) each wave has 256 registers: the
// fragments are double-buffered in registers, the loads of k-step t+1 are issued before the MFMAs of
// k-step t, and flag waits fall behind a whole k-step of matrix-core work.
//
// Per stage two counters: full (+1 per wave once ITS loads into the stage have landed; vmcnt on the
// wave's in-order queue) and empty (+1 per wave once the stage's fragments are in ITS registers).
// Segment X is loaded S-1 segments before it is multiplied, its "landed" signal is sent one segment
// before its fragments are first wanted, and when a stage is not full yet at prefetch time the wave
// multiplies first and fetches afterwards instead of stalling in front of the matrix core.
#ifndef CK_GEMM_FUSED_KERNEL_HIP_H
#define CK_GEMM_FUSED_KERNEL_HIP_H

#include <type_traits>

#include "gemm_pc_kernel.hip.h"

namespace ck {

template <int N> __device__ __forceinline__ void wait_lgkmcnt_imm() { asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory"); }

template <typename DT, int TILE, int SEGK, int CW>
__global__ __launch_bounds__(CW * 64) void gemm_fused_kernel(const GemmArgs g) {
    constexpr int WTR = TILE / (CW / 2) / MFMA_M, WTC = TILE / 2 / MFMA_N;
    constexpr int CPR = SEGK / CHUNK_ELEMS;
    constexpr int RB = SEGK * 2;
    constexpr int RPI = WAVE / CPR;
    constexpr int OPB = TILE * RB;
    constexpr int KSTEPS = SEGK / MFMA_K;
    constexpr int NI = TILE / RPI;             // wave loads per operand stage
    constexpr int LPW = 2 * NI / CW;           // wave loads per wave and stage
    constexpr bool STATIC_SPLIT = NI % CW == 0;  // the first LPW/2 loads of a wave are A, the rest Bt
    constexpr int VAR = CPR == 4 ? 1 : CPR == 8 ? 2 : 4;
    static_assert(2 * NI % CW == 0 && LPW >= 1, "stage must split evenly over the waves");

    extern __shared__ __attribute__((aligned(1024))) char ck_smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(CK_LDS char*)ck_smem;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const unsigned long long clk0 = clock64(), wall0 = wall_clock64();

    const int S = g.num_stages;
    const int fregion = flag_region_bytes(CK_SYNC_TILE, CW, 0, 0, S);
    for (int i = threadIdx.x; i < fregion / 4; i += blockDim.x) ((CK_LDS uint32_t*)ck_smem)[i] = 0;
    __syncthreads();
    const uint32_t flags_base = lds0, ring_base = lds0 + fregion;
    // per stage: [full, empty]
    auto full_addr = [&](int stage) { return flags_base + (uint32_t)stage * 8u; };
    auto empty_addr = [&](int stage) { return flags_base + (uint32_t)stage * 8u + 4u; };

    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    const int total_tiles = g.tiles_m * g.tiles_n;
    const int my_tiles = slot < total_tiles ? (total_tiles - slot + grid - 1) / grid : 0;
    const int nseg = g.nseg;
    const int total_segs = my_tiles * nseg;
    Spin sp{g.spin_limit, g.status, CK_STATUS_CONSUMER_TIMEOUT, false};

    // ---- loader side: which segment this wave issues next, descriptors of that segment's tile ------
    const uint32_t pitch32 = (uint32_t)g.K * 2u;
    const int lane_row = lane / CPR, lane_slot = lane % CPR;
    uint32_t lane_off[VAR];
    int lane_chunk[VAR];
#pragma unroll
    for (int v = 0; v < VAR; ++v) {
        lane_chunk[v] = swizzle_slot(v * RPI + lane_row, lane_slot, CPR, g.swizzle);
        lane_off[v] = (uint32_t)lane_row * pitch32 + (uint32_t)lane_chunk[v] * CHUNK_BYTES;
    }
    const uint32_t load_step = (uint32_t)RPI * pitch32;
    int l_tc = slot, l_seg = 0, l_stage = 0;
    uint32_t l_fill = 0;
    int issued_segs = 0;     // segments this wave has issued loads for
    int signalled = 0;       // segments whose "landed" signal this wave has sent
    __amdgpu_buffer_rsrc_t rsrc_a, rsrc_b;
    uint32_t nrec_a = 0, nrec_b = 0;
    bool full_a = false, full_b = false;

    auto open_tile = [&]() {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, l_tc);
        const int row_a = __builtin_amdgcn_readfirstlane(rc.row * TILE), row_b = __builtin_amdgcn_readfirstlane(rc.col * TILE);
        const int ra = g.M - row_a < TILE ? g.M - row_a : TILE, rb = g.N - row_b < TILE ? g.N - row_b : TILE;
        nrec_a = (uint32_t)ra * pitch32;
        nrec_b = (uint32_t)rb * pitch32;
        full_a = ra == TILE;
        full_b = rb == TILE;
        rsrc_a = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)g.A + (int64_t)row_a * pitch32), 0, (int)nrec_a, 0x00020000);
        rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)((const char*)g.Bt + (int64_t)row_b * pitch32), 0, (int)nrec_b, 0x00020000);
    };

    // issues this wave's LPW loads of segment `issued_segs` and advances the loader
    auto issue_segment = [&]() {
        if (l_seg == 0) open_tile();
        const int k0 = l_seg * SEGK;
        const uint32_t st_base = ring_base + (uint32_t)l_stage * (2 * OPB);
        const bool k_full = k0 + SEGK <= g.K;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            const int e = wave + i * CW;  // index over the 2 * NI wave loads of the stage
            const bool is_a = STATIC_SPLIT ? (i < NI / CW) : (e < NI);
            const int E = STATIC_SPLIT ? (wave + (i % (NI / CW > 0 ? NI / CW : 1)) * CW) : (is_a ? e : e - NI);
            const __amdgpu_buffer_rsrc_t rsrc = is_a ? rsrc_a : rsrc_b;
            const uint32_t nrec = is_a ? nrec_a : nrec_b;
            CK_LDS void* dst = (CK_LDS void*)(uintptr_t)(st_base + (is_a ? 0u : (uint32_t)OPB) + (uint32_t)E * 1024u);
            uint32_t loff = lane_off[0];
            int lchunk = lane_chunk[0];
#pragma unroll
            for (int v = 1; v < VAR; ++v) {
                if (E % VAR == v) { loff = lane_off[v]; lchunk = lane_chunk[v]; }
            }
            if ((is_a ? full_a : full_b) && k_full) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, dst, 16, loff, (uint32_t)E * load_step + (uint32_t)k0 * 2u, 0, 0);
            } else {
                uint32_t voff = loff + (uint32_t)E * load_step + (uint32_t)k0 * 2u;
                if (k0 + lchunk * CHUNK_ELEMS >= g.K) voff = nrec;  // absent k: zero fill
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, dst, 16, voff, 0, 0, 0);
            }
        }
        ++issued_segs;
        if (++l_seg == nseg) { l_seg = 0; l_tc += grid; }
        if (++l_stage == S) { l_stage = 0; ++l_fill; }
    };
    // my loads of segment `signalled` have landed when at most the later-issued ones are outstanding
    int sig_stage = 0;       // stage of segment `signalled`
#if defined(CK_PROBE_TIMING)
    unsigned long long t_vm = 0, t_lgkm = 0, t_mid = 0;
#define CK_T0() const unsigned long long ck_t0 = clock64()
#define CK_T1(acc) acc += clock64() - ck_t0
#else
#define CK_T0()
#define CK_T1(acc)
#endif
    auto signal_one = [&]() {
        CK_T0();
        const uint32_t later = (uint32_t)((issued_segs - 1 - signalled) * LPW);
        if (later == LPW) wait_vmcnt_imm<LPW>();  // steady state with four stages
        else if (later == 0) wait_vmcnt_imm<0>();
        else wait_vmcnt_le(later);
        CK_T1(t_vm);
        flag_add(full_addr(sig_stage));
        ++signalled;
        if (++sig_stage == S) sig_stage = 0;
    };

    // ---- consumer side -------------------------------------------------------------------------------
    const int R = wave / 2, Cc = wave % 2;
    const int lr = lane & 15, lg = lane >> 4;
    const int key = g.swizzle ? swizzle_key(lr, CPR) : 0;
    const uint32_t a_lane = (uint32_t)(R * WTR * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);
    const uint32_t b_lane = (uint32_t)OPB + (uint32_t)(Cc * WTC * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);

    u32x4 fa[2][WTR], fb[2][WTC];  // fragments of the k-step being multiplied and of the next one
    f32x4 acc[WTR][WTC];
#pragma unroll
    for (int i = 0; i < WTR; ++i)
#pragma unroll
        for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_frags = [&](auto parity, int stage, int ks) {
        constexpr int P = decltype(parity)::value;
        const uint32_t st = ring_base + (uint32_t)stage * (2 * OPB);
        const uint32_t pa_k = (st + a_lane) ^ (uint32_t)(ks * 64), pb_k = (st + b_lane) ^ (uint32_t)(ks * 64);
#pragma unroll
        for (int i = 0; i < WTR; ++i) fa[P][i] = *(const CK_LDS u32x4*)(uintptr_t)(pa_k + i * 16 * RB);
#pragma unroll
        for (int j = 0; j < WTC; ++j) fb[P][j] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + j * 16 * RB);
    };

    // prologue: fill S-1 stages (at least one), then fetch the fragments of k-step 0
    for (int p = 0; p < (S > 1 ? S - 1 : 1) && issued_segs < total_segs; ++p) issue_segment();
    if (total_segs > 0) {
        signal_one();
        wait_flag_ge(full_addr(0), (uint32_t)CW, sp);
        asm volatile("" ::: "memory");
        load_frags(std::integral_constant<int, 0>{}, 0, 0);
    }

    int c_stage = 0;  // stage of the segment being multiplied
    uint32_t c_fill = 0;
    int G = 0;        // index of the segment being multiplied, over all tiles of this workgroup

    // ---- steady-state fast path ---------------------------------------------------------------------
    // A wave issues roughly one instruction every four to five cycles, so next to the 32 MFMAs of a
    // k-step (512 cycles) there is room for well under a hundred other instructions. kstep() above
    // handles every case (stream start and end, tile changes of the loader, K tails, edge tiles, one
    // or two stages) and is far heavier than that; kstep_fast() is the same protocol for a segment
    // where nothing special happens: a next segment exists, the loader stays inside a full tile with
    // all k present, it is exactly S-1 segments ahead and the signal for segment G+1 is due now.
    // fast_run counts how many upcoming segments are known to be of that kind.
    int fast_run = 0;
    const uint32_t loff_w = lane_off[wave % VAR];  // CW is a multiple of VAR: a wave's loads share one key variant
    const uint32_t wave_goff = (uint32_t)wave * load_step, cw_goff = (uint32_t)CW * load_step;
    auto recompute_fast_run = [&]() {
        fast_run = 0;
        if (!STATIC_SPLIT || S < 3) return;
        if (issued_segs != G + S - 1 || signalled != G + 1 || l_seg == 0 || !(full_a && full_b)) return;
        int run = nseg - l_seg - ((g.K % SEGK) ? 1 : 0);
        run = run < total_segs - issued_segs ? run : total_segs - issued_segs;
        run = run < total_segs - 1 - G ? run : total_segs - 1 - G;
        fast_run = run > 0 ? run : 0;
    };
    auto issue_fast = [&]() {
        const uint32_t st_base = ring_base + (uint32_t)l_stage * (2 * OPB) + (uint32_t)wave * 1024u;
        const uint32_t soff = (uint32_t)l_seg * (SEGK * 2) + wave_goff;
        constexpr int HALF = NI / CW > 0 ? NI / CW : 1;
#pragma unroll
        for (int i = 0; i < LPW; ++i) {
            const bool is_a = i < HALF;
            const int ii = i % HALF;
            CK_LDS void* dst = (CK_LDS void*)(uintptr_t)(st_base + (is_a ? 0u : (uint32_t)OPB) + (uint32_t)(ii * CW) * 1024u);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(is_a ? rsrc_a : rsrc_b, dst, 16, loff_w, soff + (uint32_t)ii * cw_goff, 0, 0);
        }
        ++issued_segs;
        if (++l_seg == nseg) { l_seg = 0; l_tc += grid; }
        if (++l_stage == S) { l_stage = 0; ++l_fill; }
    };
    // One k-step. Its fragments are in f[P] (possibly still arriving); the next k-step's go to f[1-P].
    //   start : the fragments have arrived -> the stage is released if this is its last k-step; at a
    //           segment's first k-step the "landed" signal of the next segment is sent
    //   half 1: first MFMA, then the two counters this k-step depends on are sampled (the answers
    //           arrive under the remaining MFMAs of the half)
    //   middle: at a segment's first k-step the stage released one segment ago is refilled (after
    //           making sure every wave has released it); the next fragments are fetched (after making
    //           sure their stage is full); both waits are normally satisfied by the samples
    //   half 2: second half of the MFMAs, covering the latency of what the middle issued
    // `fast` selects the lean control path of a steady-state segment; the MFMA code is shared, so the
    // accumulators stay in place whatever path the control sections take.
    auto kstep = [&](auto parity, auto kstep_index, const bool fast) {
        constexpr int P = decltype(parity)::value;
        constexpr int KS = decltype(kstep_index)::value;
        constexpr bool last_ks = KS == KSTEPS - 1;
        int n_stage = c_stage;
        uint32_t n_fill = c_fill;
        if (last_ks) {
            if (++n_stage == S) { n_stage = 0; ++n_fill; }
        }
        bool more = true, refill_now = KS == 0, need_full = last_ks;
        wait_lgkmcnt_imm<0>();
        if (last_ks) flag_add(empty_addr(c_stage));
        if (fast) {
            if (KS == 0) {
                if (S == 4) wait_vmcnt_imm<LPW>();
                else if (S == 3) wait_vmcnt_imm<0>();
                else wait_vmcnt_le((uint32_t)((S - 3) * LPW));
                flag_add(full_addr(sig_stage));
                ++signalled;
                if (++sig_stage == S) sig_stage = 0;
            }
        } else {
            more = !(last_ks && G + 1 >= total_segs);  // is there a next k-step at all
            // with two or more stages the ring is refilled at a segment's first k-step (the stage of the
            // previous segment is free by then); with one the refill has to follow this segment's release
            refill_now = (S >= 2 ? KS == 0 : last_ks) && issued_segs < total_segs && issued_segs - S <= (last_ks ? G : G - 1);
            need_full = more && last_ks;
            if (S >= 3 && KS == 0 && signalled <= G + 1 && signalled < issued_segs) signal_one();
        }
        __builtin_amdgcn_sched_barrier(0);
        // first MFMA, then the two counter reads: the compiler's own fragment wait in front of the
        // first MFMA must not see newer LDS operations, or it would wait for them as well
        acc[0][0] = MfmaOp<DT>::run(fb[P][0], fa[P][0], acc[0][0]);
        __builtin_amdgcn_sched_barrier(0);
        uint32_t s_full = flag_peek(full_addr(n_stage));
        uint32_t s_empty = flag_peek(empty_addr(l_stage));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < WTC / 2; ++j)
#pragma unroll
            for (int i = 0; i < WTR; ++i) {
                if (i + j > 0) acc[i][j] = MfmaOp<DT>::run(fb[P][j], fa[P][i], acc[i][j]);
            }
        __builtin_amdgcn_sched_barrier(0);
        if (refill_now) {
            if (l_fill > 0 && (int32_t)(__builtin_amdgcn_readfirstlane(s_empty) - (uint32_t)CW * l_fill) < 0)
                wait_flag_ge(empty_addr(l_stage), (uint32_t)CW * l_fill, sp);
            if (fast) issue_fast();
            else issue_segment();
        }
        if (more) {
            if (need_full) {
                if (!fast && S < 3) {
                    // with one or two stages the next segment's signal cannot be sent any earlier
                    while (signalled <= G + 1 && signalled < issued_segs) signal_one();
                }
                if ((int32_t)(__builtin_amdgcn_readfirstlane(s_full) - (uint32_t)CW * (n_fill + 1)) < 0)
                    wait_flag_ge(full_addr(n_stage), (uint32_t)CW * (n_fill + 1), sp);
            }
            asm volatile("" ::: "memory");
            load_frags(std::integral_constant<int, 1 - P>{}, last_ks ? n_stage : c_stage, last_ks ? 0 : KS + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = WTC / 2; j < WTC; ++j)
#pragma unroll
            for (int i = 0; i < WTR; ++i) acc[i][j] = MfmaOp<DT>::run(fb[P][j], fa[P][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
    };

    // ---- epilogue: D = alpha * acc + beta * C straight from the accumulators, then clear them
    auto epilogue = [&](int tc) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
        const int m_base = rc.row * TILE + R * WTR * 16 + (int)(threadIdx.x & 15);
        const int n_base = rc.col * TILE + Cc * WTC * 16 + (int)((threadIdx.x >> 4) & 3) * 4;
        const float alpha = g.alpha, beta = g.beta;
        const bool interior = g.vec_store && (rc.row + 1) * TILE <= g.M && (rc.col + 1) * TILE <= g.N;
#pragma unroll
        for (int i = 0; i < WTR; ++i) {
            const int m = m_base + i * 16;
#pragma unroll
            for (int j = 0; j < WTC; ++j) {
                const int n = n_base + j * 16;
                const int64_t off = (int64_t)m * g.N + n;
                f32x4 v = acc[i][j] * alpha;
                if (interior) {
                    if (beta != 0.f) v += *(const f32x4*)(g.C + off) * beta;
                    *(f32x4*)(g.D + off) = v;
                } else if (m < g.M) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (n + e < g.N) {
                            float x = v[e];
                            if (beta != 0.f) x += g.C[off + e] * beta;
                            g.D[off + e] = x;
                        }
                    }
                }
                acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };
    int seg_in_tile = 0, c_tc = slot;
    auto end_segment = [&]() {
        ++G;
        if (++c_stage == S) { c_stage = 0; ++c_fill; }
        if (++seg_in_tile == nseg) {
            epilogue(c_tc);
            seg_in_tile = 0;
            c_tc += grid;
        }
    };

    // The two fragment buffers alternate per k-step. The stream of k-steps is walked in blocks of
    // lcm(2, KSTEPS) k-steps so that buffer index and k-step index are compile-time constants inside
    // a block: two segments per block when a segment is one k-step, one segment otherwise.
    constexpr int SPB = KSTEPS == 1 ? 2 : 1;   // segments per block
    using P0 = std::integral_constant<int, 0>;
    using P1 = std::integral_constant<int, 1>;
    while (G + SPB <= total_segs) {
        const bool tile_end_inside = SPB == 2 && seg_in_tile + 1 == nseg;
        const bool fast = fast_run >= SPB && !tile_end_inside;
        if (fast) fast_run -= SPB;
        if constexpr (KSTEPS == 1) {
            kstep(P0{}, std::integral_constant<int, 0>{}, fast);
            end_segment();
            kstep(P1{}, std::integral_constant<int, 0>{}, fast);
            end_segment();
        } else {
            kstep(P0{}, std::integral_constant<int, 0>{}, fast);
            kstep(P1{}, std::integral_constant<int, 1>{}, fast);
            if constexpr (KSTEPS == 4) {
                kstep(P0{}, std::integral_constant<int, 2>{}, fast);
                kstep(P1{}, std::integral_constant<int, 3>{}, fast);
            }
            end_segment();
        }
        if (!fast) recompute_fast_run();
    }
    if (SPB == 2 && G < total_segs) {  // odd number of one-k-step segments: the last one
        kstep(P0{}, std::integral_constant<int, 0>{}, false);
        end_segment();
    }

#if defined(CK_PROBE_TIMING)
    if (blockIdx.x == 0 && lane == 0) {
        unsigned* o = g.status + 8 + wave * 8;
        o[0] = (unsigned)sp.wait_cycles; o[1] = (unsigned)(sp.wait_cycles >> 32); o[2] = sp.wait_calls; o[3] = sp.wait_polls;
        o[4] = (unsigned)(t_vm >> 4); o[5] = (unsigned)(t_lgkm >> 4); o[6] = (unsigned)(t_mid >> 4);
    }
#endif
    if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
        const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
        g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
        g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
    }
}

}  // namespace ck
#endif  // CK_GEMM_FUSED_KERNEL_HIP_H

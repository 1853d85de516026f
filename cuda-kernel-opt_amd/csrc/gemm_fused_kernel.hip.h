// gemm_shmem_tc_async_opt_port with num_producer_waves == 0: the same LDS ring, direct-to-LDS loads
// and MFMA wave tiles as the producer/consumer kernel, but every wave is both. It streams its 1/CW
// share of each K-segment into the ring and multiplies out of it, and the waves of a workgroup meet
// at the hardware workgroup barrier once per segment instead of exchanging flag counters.
//
// Why this variant exists: all waves of a kernel get the same register allocation, so dedicated
// producer waves push a 256 x 256 tile (8 consumer waves, 128 accumulator registers each) to three
// waves per SIMD and 168 registers per wave - no room to hold the next k-step's fragments while the
// current one is being multiplied. With 8 waves (two per SIMD) each wave has 256 registers: the
// fragments are double-buffered in registers and the LDS reads of k-step t+1 are issued under the
// MFMAs of k-step t.
//
// Schedule of one wave (segment G, k-steps 0 .. KSTEPS-1, fragments of a k-step fetched one k-step
// ahead):
//   at the segment's LAST k-step, once its fragments are in registers:
//     wait until this wave's own loads of segment G+1 have landed (in-order vmcnt),
//     a few MFMAs that need registers only, then the workgroup barrier. Behind the barrier
//       (a) every wave's share of segment G+1 is in LDS  -> its fragments may be fetched, and
//       (b) every wave holds the last fragments of segment G -> its stage is free,
//     so the wave issues its loads of segment G+S into that stage (S-1 segments of slack before
//     they are wanted) and fetches the first fragments of segment G+1 under the remaining MFMAs.
// The stream of segments runs across the tiles of the persistent workgroup: the loads of the next
// tile are in flight while the current one is finished and written out.
//
// The direct-to-LDS loads are issued from inline assembly. The compiler cannot tell which LDS bytes
// such a load will write, so with the builtin it drains ALL outstanding loads (vmcnt 0) in front of
// every LDS read of the wave - which would serialise global latency into every k-step. Which loads
// must have landed before which LDS read is exactly what the barrier protocol above establishes.
#ifndef CK_GEMM_FUSED_KERNEL_HIP_H
#define CK_GEMM_FUSED_KERNEL_HIP_H

#include <type_traits>

#include "gemm_pc_kernel.hip.h"

namespace ck {

typedef int i32x4 __attribute__((ext_vector_type(4)));

// 16 bytes per lane from a raw buffer straight into LDS at lds_dst + lane * 16. voff is range
// checked against the descriptor (out of range lanes write zeros), soff is not.
__device__ __forceinline__ void dma_load_b128(i32x4 rsrc, uint32_t lds_dst, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_dst), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory");
}
// The same load with one of two per-lane offsets, chosen by a wave-uniform flag through a scalar branch inside the
// statement (a select in vector registers would put a vector ALU instruction in front of every load, and those share
// the matrix cores' issue port; a branch the compiler can see would split the caller's loop body into basic blocks).
__device__ __forceinline__ void dma_load_b128_select(i32x4 rsrc, uint32_t lds_dst, uint32_t voff, uint32_t voff_if_flag, uint32_t soff,
                                                     uint32_t flag) {
    asm volatile("s_mov_b32 m0, %0\n\ts_cmp_lg_u32 %5, 0\n\ts_cbranch_scc1 1f\n\tbuffer_load_dwordx4 %1, %3, %4 offen lds\n\ts_branch 2f\n1:\n\t"
                 "buffer_load_dwordx4 %2, %3, %4 offen lds\n2:"
                 :
                 : "s"(lds_dst), "v"(voff), "v"(voff_if_flag), "s"(rsrc), "s"(soff), "s"(flag)
                 : "memory", "scc");
}
__device__ __forceinline__ i32x4 make_rsrc(const void* base, uint32_t num_records) {
    const uint64_t p = (uint64_t)(uintptr_t)base;
    i32x4 r;
    r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
    r[1] = __builtin_amdgcn_readfirstlane((int)(uint32_t)((p >> 32) & 0xffffu));  // stride 0: raw buffer
    r[2] = __builtin_amdgcn_readfirstlane((int)num_records);
    r[3] = 0x00020000;
    return r;
}
// workgroup barrier that the compiler treats as a full memory clobber (no LDS access moves across)
__device__ __forceinline__ void wg_barrier() { asm volatile("s_barrier" ::: "memory"); }
__device__ __forceinline__ void wait_lgkmcnt0() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

template <int N> __device__ __forceinline__ void use_fragment_array(const u32x4 (&f)[N]) {
    if constexpr (N == 8) asm volatile("" ::"v"(f[0]), "v"(f[1]), "v"(f[2]), "v"(f[3]), "v"(f[4]), "v"(f[5]), "v"(f[6]), "v"(f[7]) : "memory");
    else if constexpr (N == 4) asm volatile("" ::"v"(f[0]), "v"(f[1]), "v"(f[2]), "v"(f[3]) : "memory");
    else if constexpr (N == 2) asm volatile("" ::"v"(f[0]), "v"(f[1]) : "memory");
    else {
#pragma unroll
        for (int i = 0; i < N; ++i) asm volatile("" ::"v"(f[i]) : "memory");
    }
}
template <int NA, int NB> __device__ __forceinline__ void use_fragments(const u32x4 (&a)[NA], const u32x4 (&b)[NB]) {
    use_fragment_array(a);
    use_fragment_array(b);
}

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
    constexpr int HALF = NI / CW > 0 ? NI / CW : 1;
    constexpr int VAR = CPR == 4 ? 1 : CPR == 8 ? 2 : 4;
    constexpr int LPK = LPW / KSTEPS;          // wave loads per wave and k-step
    constexpr int PRE = 1;                     // columns of 16 x 16 blocks multiplied between the landing wait and the barrier
    static_assert(2 * NI % CW == 0 && LPW >= 1 && LPK * KSTEPS == LPW && LPK >= 1, "stage must split evenly over waves and k-steps");

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

    // ---- loader side -----------------------------------------------------------------------------------
    // A wave load E covers rows [E*RPI, (E+1)*RPI) of an operand stage; lane (lane_row, lane_slot)
    // fetches the 16-byte chunk that belongs at its linear LDS slot under the XOR swizzle. Wave w
    // issues the loads E = w, w + CW, ... of A and then of Bt (with fewer loads than waves: one load of
    // one operand). CW is a multiple of the swizzle key's period in E, so one per-lane offset serves
    // all loads of a wave. The loads of a segment are issued in KSTEPS chunks of LPK loads, one chunk
    // per k-step and inside it one load every few MFMA columns: eight waves that issue all their
    // loads back to back right behind the barrier queue up at the CU's one address unit and stall in
    // front of their MFMAs.
    const uint32_t pitch32 = (uint32_t)g.K * 2u;
    const int lane_row = lane / CPR, lane_slot = lane % CPR;
    const int lchunk_w = swizzle_slot((wave % VAR) * RPI + lane_row, lane_slot, CPR, g.swizzle);
    const uint32_t loff_w = (uint32_t)lane_row * pitch32 + (uint32_t)lchunk_w * CHUNK_BYTES;
    const uint32_t load_step = (uint32_t)RPI * pitch32;
    int l_tc = slot, l_seg = 0, l_stage = 0;
    int opened_segs = 0;       // segments whose first chunk has been issued
    int issued_loads = 0;      // loads this wave has issued so far
    i32x4 rsrc_a = {0, 0, 0, 0}, rsrc_b = {0, 0, 0, 0};
    uint32_t nrec_a = 0, nrec_b = 0;
    // the segment being issued
    uint32_t ld_base = 0, ld_k0x2 = 0;
    bool ld_ktail = false, full_tile = false;
    int ld_mode = 0;                      // 0: no segment open, 1: fast form, 2: slow form
    uint32_t ld_dst_w = 0, ld_goff_w = 0;  // fast form: LDS address and global offset of this wave's load 0
    uint32_t goff_step[HALF];              // global offset of load ii relative to load 0
#pragma unroll
    for (int ii = 0; ii < HALF; ++ii) goff_step[ii] = (uint32_t)(ii * CW) * load_step;

    auto open_tile = [&]() __attribute__((always_inline)) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, l_tc);
        const int row_a = __builtin_amdgcn_readfirstlane(rc.row * TILE), row_b = __builtin_amdgcn_readfirstlane(rc.col * TILE);
        const int ra = g.M - row_a < TILE ? g.M - row_a : TILE, rb = g.N - row_b < TILE ? g.N - row_b : TILE;
        nrec_a = (uint32_t)ra * pitch32;
        nrec_b = (uint32_t)rb * pitch32;
        full_tile = ra == TILE && rb == TILE;
        rsrc_a = make_rsrc((const char*)g.A + (int64_t)row_a * pitch32, nrec_a);
        rsrc_b = make_rsrc((const char*)g.Bt + (int64_t)row_b * pitch32, nrec_b);
    };
    // starts the next segment: its stage, its k offset, whether it reaches past K
    auto open_segment = [&]() __attribute__((always_inline)) {
        if (l_seg == 0) open_tile();
        ld_base = ring_base + (uint32_t)l_stage * (2 * OPB);
        ld_k0x2 = (uint32_t)l_seg * (SEGK * 2);
        ld_ktail = (l_seg + 1) * SEGK > g.K;
        ld_mode = STATIC_SPLIT && full_tile && !ld_ktail ? 1 : 2;
        ld_dst_w = ld_base + (uint32_t)wave * 1024u;
        ld_goff_w = (uint32_t)wave * load_step + ld_k0x2;
        ++opened_segs;
        if (++l_seg == nseg) { l_seg = 0; l_tc += grid; }
        if (++l_stage == S) l_stage = 0;
    };
    // load i (0 .. LPW-1) of the open segment. Fast form (whole tile, whole segment inside the
    // operands, nothing can be out of range): the per-lane offset is a constant of the wave and
    // everything else is scalar - M0 and the (unchecked) scalar offset, one add each. Slow form (edge
    // tiles, K tail): the whole global offset goes through the range-checked vector offset, so rows
    // past the tile edge and k past K land outside the descriptor and read as zero.
    auto issue_load = [&](int i) __attribute__((always_inline)) {
        bool is_a;
        int E, ii;
        if (STATIC_SPLIT) {
            is_a = i < HALF;
            ii = i % HALF;
            E = wave + ii * CW;
        } else {
            is_a = wave < NI;
            ii = 0;
            E = is_a ? wave : wave - NI;
        }
        if (ld_mode == 1) {
            dma_load_b128(is_a ? rsrc_a : rsrc_b, ld_dst_w + (is_a ? 0u : (uint32_t)OPB) + (uint32_t)(ii * CW) * 1024u, loff_w,
                          ld_goff_w + goff_step[ii]);
            ++issued_loads;
        } else if (ld_mode == 2) {
            const uint32_t dst = ld_base + (is_a ? 0u : (uint32_t)OPB) + (uint32_t)E * 1024u;
            uint32_t voff = loff_w + ((uint32_t)E * load_step + ld_k0x2);
            if (ld_ktail && (int)(ld_k0x2 >> 1) + lchunk_w * CHUNK_ELEMS >= g.K) voff = is_a ? nrec_a : nrec_b;
            dma_load_b128(is_a ? rsrc_a : rsrc_b, dst, voff, 0u);
            ++issued_loads;
        }
    };

    // ---- multiplier side -------------------------------------------------------------------------------
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

    int c_stage = 0;  // stage of the segment being multiplied
    int G = 0;        // index of the segment being multiplied, over all tiles of this workgroup
    int seg_in_tile = 0, c_tc = slot;

    // ---- epilogue: D = alpha * acc + beta * C straight from the accumulators, then clear them
    auto epilogue = [&](int tc) __attribute__((always_inline)) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
        const int m_base = rc.row * TILE + R * WTR * 16 + (int)(threadIdx.x & 15);
        const int n_base = rc.col * TILE + Cc * WTC * 16 + (int)((threadIdx.x >> 4) & 3) * 4;
        const bool vec_cols = g.vec_store && (rc.col + 1) * TILE <= g.N;
#pragma unroll
        for (int i = 0; i < WTR; ++i) {
#pragma unroll
            for (int j = 0; j < WTC; ++j) {
                epilogue_block<DT>(g, m_base + i * 16, n_base + j * 16, acc[i][j], vec_cols);
                acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
    };

    // this wave's loads of segment X have landed when at most the loads it issued after them are
    // outstanding (a wave's loads complete in issue order; other memory operations in flight only
    // make the wait longer, never shorter)
    auto wait_landed = [&](int X) __attribute__((always_inline)) {
        const int later = issued_loads - (X + 1) * LPW;
        if (later == 2 * LPW) wait_vmcnt_imm<2 * LPW>();   // four stages in steady state
        else if (later == LPW) wait_vmcnt_imm<LPW>();      // three stages
        else if (later == 3 * LPW && 3 * LPW < 64) wait_vmcnt_imm<(3 * LPW < 64 ? 3 * LPW : 0)>();  // five stages
        else if (later <= 0) wait_vmcnt_imm<0>();
        else wait_vmcnt_le((uint32_t)later);
    };

    // One k-step. Its fragments are in f[P] (possibly still arriving); the next k-step's go to f[1-P].
    auto kstep = [&](auto parity, auto kstep_index) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        constexpr int KS = decltype(kstep_index)::value;
        constexpr bool last_ks = KS == KSTEPS - 1;
        const bool has_next_seg = G + 1 < total_segs;
        int n_stage = c_stage;
        if (last_ks && ++n_stage == S) n_stage = 0;
        const uint32_t st = ring_base + (uint32_t)(last_ks ? n_stage : c_stage) * (2 * OPB);
        const uint32_t pa_k = (st + a_lane) ^ (uint32_t)((last_ks ? 0 : KS + 1) * 64);
        const uint32_t pb_k = (st + b_lane) ^ (uint32_t)((last_ks ? 0 : KS + 1) * 64);

        if (last_ks) {
            // The next segment's parameters are worked out here, ahead of the waits: behind the barrier
            // nothing but the loads themselves stands between the waves and their MFMAs. (All chunks of
            // the previous segment were issued by the k-step before this one.)
            ld_mode = 0;
            if (has_next_seg && opened_segs < total_segs) open_segment();
            // The last fragments of this segment must be in registers before the barrier releases
            // their stage. The wait is requested through a use of the registers the compiler can
            // see: behind a bare s_waitcnt in inline assembly it would still count these reads as
            // outstanding and pad every later fragment wait with the reads issued after the barrier.
            use_fragments(fa[P], fb[P]);
            if (has_next_seg) wait_landed(G + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < PRE; ++j)
#pragma unroll
            for (int i = 0; i < WTR; ++i) acc[i][j] = MfmaOp<DT>::run(fb[P][j], fa[P][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        // chunk of LPK loads this k-step issues: at a segment's last k-step (behind the barrier) chunk 0
        // of the segment that goes into the stage just released, otherwise the next chunk of the
        // segment opened at the previous segment's last k-step
        if (last_ks && has_next_seg) {
            wg_barrier();
        }
        constexpr int CHUNK = last_ks ? 0 : KS + 1;
        __builtin_amdgcn_sched_barrier(0);
        // remaining columns; between them the fetch of the next k-step's fragments (A fragments
        // first, then Bt) and this k-step's loads, one every LSTRIDE columns
        constexpr int NF = WTR + WTC;                 // fragments to fetch
        constexpr int COLS = WTC - PRE;               // columns left to multiply
        constexpr int PER = (NF + COLS - 1) / COLS;   // fetches per column
        constexpr int LSTRIDE = (COLS + LPK - 1) / LPK;
#pragma unroll
        for (int j = PRE; j < WTC; ++j) {
            // (after the very last k-step of the stream this fetches fragments nobody uses: the
            // addresses are inside the ring, and skipping them would put a branch in every column)
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const int f = (j - PRE) * PER + q;
                if (f < WTR) fa[1 - P][f] = *(const CK_LDS u32x4*)(uintptr_t)(pa_k + f * 16 * RB);
                else if (f < NF) fb[1 - P][f - WTR] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + (f - WTR) * 16 * RB);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int l = 0; l < LPK; ++l) {
                const int col = l * LSTRIDE < COLS ? l * LSTRIDE : COLS - 1;
                if (col == j - PRE) issue_load(CHUNK * LPK + l);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < WTR; ++i) acc[i][j] = MfmaOp<DT>::run(fb[P][j], fa[P][i], acc[i][j]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    bool tile_done = false;  // the segment just finished was the last of its tile: write it out
    auto end_segment = [&]() __attribute__((always_inline)) {
        ++G;
        if (++c_stage == S) c_stage = 0;
        if (++seg_in_tile == nseg) {
            seg_in_tile = 0;
            tile_done = true;
        }
    };

    if (total_segs > 0) {
        // prologue: fill every stage, then fetch the fragments of k-step 0 once segment 0 is in LDS
        for (int p = 0; p < S && opened_segs < total_segs; ++p) {
            open_segment();
#pragma unroll
            for (int i = 0; i < LPW; ++i) issue_load(i);
        }
        ld_mode = 0;  // everything opened so far is issued
        wait_landed(0);
        wg_barrier();
        {
            const uint32_t pa_k = ring_base + a_lane, pb_k = ring_base + b_lane;
#pragma unroll
            for (int i = 0; i < WTR; ++i) fa[0][i] = *(const CK_LDS u32x4*)(uintptr_t)(pa_k + i * 16 * RB);
#pragma unroll
            for (int j = 0; j < WTC; ++j) fb[0][j] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + j * 16 * RB);
        }

        // The two fragment buffers alternate per k-step, and the buffer index is a compile-time
        // constant: the loop body is one segment when that is an even number of k-steps, otherwise
        // (one k-step per segment) two segments. A tile that ends between the two moves the fragments
        // that were just fetched into buffer 0 and starts the body again, so there is one copy of
        // the epilogue in the code.
        using P0 = std::integral_constant<int, 0>;
        using P1 = std::integral_constant<int, 1>;
        using K0 = std::integral_constant<int, 0>;
        using K1 = std::integral_constant<int, 1>;
        using K2 = std::integral_constant<int, 2>;
        using K3 = std::integral_constant<int, 3>;
        for (;;) {
            if (tile_done) {
                epilogue(c_tc);
                c_tc += grid;
                tile_done = false;
            }
            if (G >= total_segs) break;
            kstep(P0{}, K0{});
            if constexpr (KSTEPS == 1) {
                end_segment();
                if (tile_done || G >= total_segs) {
#pragma unroll
                    for (int i = 0; i < WTR; ++i) fa[0][i] = fa[1][i];
#pragma unroll
                    for (int j = 0; j < WTC; ++j) fb[0][j] = fb[1][j];
                    continue;
                }
                kstep(P1{}, K0{});
                end_segment();
            } else {
                kstep(P1{}, K1{});
                if constexpr (KSTEPS == 4) {
                    kstep(P0{}, K2{});
                    kstep(P1{}, K3{});
                }
                end_segment();
            }
        }
    }

    if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
        const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
        g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
        g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
    }
}

}  // namespace ck
#endif  // CK_GEMM_FUSED_KERNEL_HIP_H

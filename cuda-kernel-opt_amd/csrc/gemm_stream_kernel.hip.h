// The straight-line form of the fused (no dedicated producer waves) kernel for the shape the headline
// sizes use: 256 x 256 tiles, eight waves, K a multiple of 64 (M and N are free: ragged tiles read
// zeros past the edge and store element by element), and a ring of five 32-deep K segments
// ("quarters", 32 KiB each) - all of the CU's LDS. With those fixed the loop body is two k-steps,
// the loader runs exactly two bodies ahead of the multiplier, and every wait is an immediate - no
// mode flags, no wait ladder, no per-segment bookkeeping between the MFMAs.
//
// Why five quarters and "pair fetch": a 32-deep segment is 64 bytes of each operand row, half a
// cache line. Fetching the halves in different k-steps makes the L1 ask the L2 for every line twice
// (measured: 17.9 TB/s of useful bytes for this access pattern against 26 TB/s with whole lines -
// below what the MFMAs consume at full rate). So a wave fetches both halves of its rows back to back
// (the second request merges with the first in the L1) into two quarters at once, every second
// k-step. Four quarters would leave two k-steps between issue and use, as a ring of two 64-deep
// stages does; the fifth buys a third.
//
// Even k-step j (quarter q = j % 5), fragments of j on their way to registers:
//     fragments in registers; first column of MFMAs; workgroup barrier -> quarter q is free
//     7 columns of MFMAs; under them the fragments of j+1 from quarter q+1 and this wave's four
//     loads of A for k-steps j+4 and j+5 into quarters q+4 (free since the previous barrier) and q
// Odd k-step j+1:
//     fragments in registers; own loads of k-steps j+2, j+3 landed (the four just issued may fly);
//     first column; barrier -> quarters q+2, q+3 complete; 7 columns, fragments of j+2 from q+2 and
//     the four loads of Bt for k-steps j+4 and j+5
// ODD_ONLY (an option, not the default) drops the even k-step's barrier: all four pairs of a body are
// then issued in the odd k-step, behind its barrier (by then quarter q is free as well), and the odd
// k-step waits for all of the wave's loads. That leaves the loads two k-steps instead of three and
// bunches them: at 8192^3 on random operands 1.5 % faster on one device and 0.7 % slower on another, and
// slower wherever the loads take longer (16384^3: 7 %, split-K items: 6 to 12 %), the clock is free
// (all-zero operands: 3 %) or the tiles are 256 x 128 (4 to 13 %).
// The stream of k-steps runs across the tiles of the persistent workgroup; the loader moves to the
// next tile two bodies before the multiplier does, so its first quarters are in flight while the
// current tile is finished and written out.
//
// Vector memory operations of a wave complete in issue order, stores included, so "the loads of
// k-step X have landed" is "at most as many operations outstanding as were issued after them".
// In the body that follows an epilogue the 32 stores of the epilogue sit between the loads already
// in flight and the new ones, and the immediate accounts for them - waiting for the stores
// themselves would put their whole latency in front of the first MFMAs of every tile.
#ifndef CK_GEMM_STREAM_KERNEL_HIP_H
#define CK_GEMM_STREAM_KERNEL_HIP_H

#include "gemm_fused_kernel.hip.h"

namespace ck {

constexpr int STREAM_TILE = 256;
constexpr int STREAM_SEGK = 32;
constexpr int STREAM_STAGES = 5;
constexpr int STREAM_K_MULTIPLE = 2 * STREAM_SEGK;  // one loop body
constexpr int STREAM_TILE_N_HALF = 128;   // the half-width form: 256 x 128 tiles (wave tiles of 64 x 64)
constexpr int STREAM_TILE_N_THREE_QUARTERS = 192;   // 256 x 192 tiles (wave tiles of 64 x 96)
// bytes of the ring for tiles of 256 x tile_n
constexpr int stream_ring_bytes(int tile_n) { return STREAM_STAGES * (STREAM_TILE + tile_n) * STREAM_SEGK * 2; }
// dynamic LDS of a launch: the ring, and for 256 x 192 tiles 1 KiB behind it that takes the zeros of the loads half of
// the waves issue only to keep every wave's load count the same
constexpr int stream_lds_bytes(int tile_n) { return stream_ring_bytes(tile_n) + (tile_n == STREAM_TILE_N_THREE_QUARTERS ? 1024 : 0); }
constexpr int STREAM_LDS_BYTES = stream_lds_bytes(STREAM_TILE);
constexpr int FIX_STATE_STRIDE_BYTES = 128;  // bytes between the announcement counters of two (sliced tile, wave) units

// KTAIL: K is a multiple of 8 but not of 64. The last loop body of a tile then reaches past K: its loads take
// per-lane offsets in which every 16-byte chunk at or beyond K lies outside the descriptor (reads as zeros), chosen
// by a scalar branch inside the load's asm statement, so that nothing is added to the other bodies but two scalar
// instructions per load. Launches with K % 64 == 0 run the instance without any of it.
// WTC: 16-column blocks per wave tile. 8: 256 x 256 tiles (wave tiles of 64 x 128); 4: 256 x 128 tiles (wave tiles of
// 64 x 64) for launches whose 256 x 256 tiles would leave most of the device idle - twice the tiles, half the MFMAs
// per k-step and wave, a ring of 24 KiB quarters, one load pair of Bt per wave and body instead of two; 6: 256 x 192
// tiles (wave tiles of 64 x 96) for tile counts that fill the last round badly at the other widths (6144^3: 768 tiles
// = exactly three rounds of 256) - quarters of 28 KiB; Bt's 192 rows are twelve 16-row loads, so waves 0 .. 3 issue a
// second pair of Bt and waves 4 .. 7 a pair that fetches nothing (every lane out of range, zeros into a spare KiB of
// LDS): all waves issue the same number of loads, which the counted waits rely on.
template <typename DT, bool ODD_ONLY, bool KTAIL, int WTC>
__global__ __launch_bounds__(512) void gemm_stream_kernel(const GemmArgs g) {
    constexpr int TILE = STREAM_TILE, NQ = STREAM_STAGES;
    constexpr int WTR = 4;                   // 16 x 16 blocks per wave tile: WTR x WTC (64 rows x 128 or 64 columns)
    constexpr int TILE_N = 2 * WTC * 16;     // two wave tiles side by side
    constexpr int RB = STREAM_SEGK * 2;      // bytes per LDS row
    constexpr int OPB = TILE * RB;           // A's part of a quarter
    constexpr int OPB_B = TILE_N * RB;       // Bt's part
    constexpr int QB = OPB + OPB_B;          // one quarter
    constexpr int B_PAIRS = (TILE_N + 127) / 128;   // load pairs of Bt per wave and body (16 rows each; 256 x 192: the second one real in waves 0 .. 3 only)
    constexpr bool PARTIAL_B3 = TILE_N % 128 != 0;
    constexpr int LPB = (2 + B_PAIRS) * 2;   // loads per wave and body: (A rows w, w + 8; Bt rows w [, w + 8]) x (two halves)
    constexpr int EVEN_LOADS = 4;            // of those, issued in the even k-step when every k-step has a barrier: A's
    static_assert(WTC == 8 || WTC == 6 || WTC == 4, "wave tiles of 64 x 128, 64 x 96 or 64 x 64");
    // Stores one wave issues in the epilogue of an interior tile. The landing wait of the body behind an epilogue
    // counts them (they sit between the loads in flight and the new ones), so the loops below and the wait
    // immediates are written in terms of the same constants.
    constexpr int F32_GROUP = 2, H16_GROUP = 4;     // accumulator blocks exchanged between lanes into whole lines
    constexpr int STORES_PER_GROUP = 2;             // rows 0..7 and 8..15 of the group
    constexpr int EPILOGUE_STORES = WTR * (WTC / F32_GROUP) * STORES_PER_GROUP;        // fp32 output
    // 16-bit output in whole lines needs groups of four blocks; a wave tile of six block columns (256 x 192 tiles) writes
    // 16-bit output block by block instead, WTR * WTC = EPILOGUE_STORES stores, and its landing wait counts those
    constexpr bool H16_WHOLE_LINES = WTC % H16_GROUP == 0;
    constexpr int EPILOGUE_STORES_16 = H16_WHOLE_LINES ? WTR * (WTC / H16_GROUP) * STORES_PER_GROUP : EPILOGUE_STORES / 2;     // 16-bit output
    static_assert(WTC % F32_GROUP == 0, "whole groups per wave-tile row");
    static_assert(EPILOGUE_STORES_16 * 2 == EPILOGUE_STORES, "count_stores selects between the two with a shift by one");
    constexpr int PRE = 1;               // columns of MFMAs in front of the barrier
    constexpr int LOAD_COL_0 = WTC == 8 ? 3 : WTC == 6 ? 2 : 1;  // columns behind which a k-step's two load pairs are issued
    constexpr int LOAD_COL_1 = WTC == 8 ? 6 : WTC == 6 ? 4 : 3;
    constexpr int FPC = (WTR + WTC + (WTC - PRE) - 1) / (WTC - PRE);   // fragments of the next k-step fetched per column
    static_assert(PRE >= 1 && (WTC - PRE) * FPC >= WTR + WTC && LOAD_COL_0 >= PRE && LOAD_COL_1 > LOAD_COL_0 && LOAD_COL_1 < WTC, "schedule");
    static_assert(LPB + EPILOGUE_STORES < 64 && EPILOGUE_STORES_16 < EPILOGUE_STORES, "the wait immediates must fit the 6-bit counter");
    // 16-bit output whose rows are off the 16-byte boundaries (d16_misaligned) goes through the per-block epilogue, one
    // store per accumulator block, while the landing wait behind it counts EPILOGUE_STORES: an epilogue that issues fewer
    // stores than the wait counts would let fragments be read before their loads have landed
    static_assert(WTR * WTC >= EPILOGUE_STORES, "the per-block epilogue issues at least the stores the landing wait counts");
    static_assert(NQ * QB == stream_ring_bytes(TILE_N) && stream_lds_bytes(TILE_N) <= LDS_BYTES_PER_CU, "the ring (all of the LDS for 256 x 256 tiles)");

    extern __shared__ __attribute__((aligned(1024))) char ck_smem[];
    const uint32_t ring_base = (uint32_t)(uintptr_t)(CK_LDS char*)ck_smem;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const unsigned long long clk0 = clock64(), wall0 = wall_clock64();

    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    // Work items, dealt like tile counts (slot, slot + grid, ...): first the tile counts [0, T1) over all of K, then one
    // item per (tile, K slice) for the tile counts from T1 on - the partly filled last round of a large launch, or every
    // tile of a launch with fewer tiles than CUs. 32 consecutive sliced items - what one XCD runs at a time - are 32
    // consecutive tile counts of ONE slice (all sliced tiles, if they do not come in whole runs of 32), so they share
    // operand panels in that XCD's L2 exactly as whole tiles do. Without split-K every item is a tile count.
    const int S = g.split_k;
    const int T = g.tiles_m * g.tiles_n;
    const int T1 = S > 1 ? g.whole_tiles : T;
    const int total_items = T1 + (T - T1) * S;
    const int my_tiles = slot < total_items ? (total_items - slot + grid - 1) / grid : 0;
    const int kslice = g.K / S;                  // the host makes this a multiple of one loop body (KTAIL: S is 1, of 8)
    const uint32_t kslice_bytes = (uint32_t)kslice * 2u, kwhole_bytes = (uint32_t)g.K * 2u;
    const int nb_slice = (kslice + STREAM_K_MULTIPLE - 1) / STREAM_K_MULTIPLE;   // loop bodies per sliced item
    const int nb_whole = (g.K + STREAM_K_MULTIPLE - 1) / STREAM_K_MULTIPLE;      // and per whole tile
    const int CH = g.split_chunk;
    // tile count of an item; slice: its K slice, or -1 for a whole tile
    auto item_tile = [&](int64_t item, int& slice) __attribute__((always_inline)) {
        if (item < T1) {
            slice = -1;
            return item;
        }
        const int64_t j = item - T1, chunk = j / CH;
        slice = (int)(chunk % S);
        return T1 + (chunk / S) * CH + j % CH;
    };

    // ---- loader ------------------------------------------------------------------------------------
    // A wave load covers 16 rows x 64 bytes of an operand quarter; wave w issues the loads of rows
    // 16w.. and 16(w+8).. of A and of Bt. Lane (row, slot) fetches the 16-byte chunk that belongs at
    // its linear LDS position under the XOR swizzle (the key depends on the row inside the 16-row
    // block only).
    const uint32_t pitch32 = (uint32_t)g.K * 2u;
    const int lane_row = lane / 4, lane_slot = lane % 4;
    // The row part of the address goes through the range-checked per-lane offset (rows past the edge
    // of a ragged tile lie outside the descriptor and read as zeros), the k part through the
    // unchecked scalar offset.
    const uint32_t loff_lo = (uint32_t)(wave * 16 + lane_row) * pitch32 + (uint32_t)swizzle_slot(lane_row, lane_slot, 4, 1) * CHUNK_BYTES;
    const uint32_t loff_hi = loff_lo + 8u * 16u * pitch32;   // rows 16(w+8)..
    // KTAIL: the same offsets for the body that holds the end of K (rem of its 64 k exist): a lane whose chunk starts at
    // or beyond rem gets an offset outside any descriptor, per half (first / second 32 k) of the body
    uint32_t toff_lo[2] = {0, 0}, toff_hi[2] = {0, 0};
    if constexpr (KTAIL) {
        const int rem = kslice % STREAM_K_MULTIPLE;
        const int chunk_k = swizzle_slot(lane_row, lane_slot, 4, 1) * CHUNK_ELEMS;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const bool absent = h * STREAM_SEGK + chunk_k >= rem;
            toff_lo[h] = absent ? 0x7fffff00u : loff_lo;
            toff_hi[h] = absent ? 0x7fffff00u : loff_hi;
        }
    }
    // 256 x 192 tiles: pair 3 (Bt rows 128 + 16w ..) exists in waves 0 .. 3; in the others every lane's offset lies outside
    // any descriptor (nothing is fetched) and the zeros go to the spare KiB behind the ring
    const bool b3_absent = PARTIAL_B3 && wave >= 4;
    const uint32_t loff_b3 = b3_absent ? 0x7fffff00u : loff_hi;
    const uint32_t toff_b3[2] = {b3_absent ? 0x7fffff00u : toff_hi[0], b3_absent ? 0x7fffff00u : toff_hi[1]};
    const uint32_t spare_lds = ring_base + (uint32_t)(NQ * QB);
    uint32_t l_tail = 0;  // KTAIL: nonzero while the body being loaded is the one that holds the end of K
    if constexpr (KTAIL) asm volatile("s_mov_b32 %0, %1" : "=s"(l_tail) : "s"(__builtin_amdgcn_readfirstlane((uint32_t)(kslice <= STREAM_K_MULTIPLE))));
    uint32_t l_kbytes = kwhole_bytes;  // extent along K, in bytes, of the item being loaded
    const uint32_t dst_w = ring_base + (uint32_t)wave * 1024u;
    i32x4 rsrc_a = {0, 0, 0, 0x00020000}, rsrc_b = {0, 0, 0, 0x00020000};  // empty descriptors: loads read zeros
    uint32_t l_koff = 0;  // byte offset along K of the body being loaded
    int l_tile = 0;       // index (in this workgroup's list) of the tile being loaded
    auto loader_open_tile = [&]() __attribute__((always_inline)) {
        if (l_tile < my_tiles) {
            int slice = 0;
            const int64_t tc = item_tile(slot + (int64_t)l_tile * grid, slice);
            const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
            const int row_a = __builtin_amdgcn_readfirstlane(rc.row * TILE), row_b = __builtin_amdgcn_readfirstlane(rc.col * TILE_N);
            const int ra = g.M - row_a < TILE ? g.M - row_a : TILE, rb = g.N - row_b < TILE_N ? g.N - row_b : TILE_N;
            const int64_t k0 = slice < 0 ? 0 : (int64_t)slice * kslice_bytes;  // the slice starts k0 bytes into every row
            l_kbytes = slice < 0 ? kwhole_bytes : kslice_bytes;
            // (the descriptor's extent is counted from the shifted base: the last row ends k0 bytes early)
            rsrc_a = make_rsrc((const char*)g.A + (int64_t)row_a * pitch32 + k0, (uint32_t)ra * pitch32 - (uint32_t)k0);
            rsrc_b = make_rsrc((const char*)g.Bt + (int64_t)row_b * pitch32 + k0, (uint32_t)rb * pitch32 - (uint32_t)k0);
        } else {
            rsrc_a[2] = 0;  // past the last tile: nothing is fetched (the ring receives zeros nobody reads)
            rsrc_b[2] = 0;
            l_kbytes = kwhole_bytes;
        }
    };
    auto loader_advance = [&]() __attribute__((always_inline)) {
        l_koff += STREAM_K_MULTIPLE * 2;
        if (l_koff >= l_kbytes) {
            l_koff = 0;
            ++l_tile;
            loader_open_tile();
        }
        if constexpr (KTAIL)   // (kept in one opaque scalar register, like stores_in_flight below)
            asm volatile("s_mov_b32 %0, %1" : "=s"(l_tail) : "s"(__builtin_amdgcn_readfirstlane((uint32_t)(l_koff + STREAM_K_MULTIPLE * 2 > l_kbytes))));
    };
    // Load pair P (0, 1: A rows 16w.. / 16(w+8)..; 2, 3: Bt likewise; 256 x 128 tiles have no pair 3) of the body at l_koff: the two
    // halves of each row's line, back to back, into the quarters at byte offsets q_lo and q_hi.
    auto issue_pair = [&](auto index, uint32_t q_lo, uint32_t q_hi) __attribute__((always_inline)) {
        constexpr int P = decltype(index)::value;
        constexpr bool IS_A = P < 2;
        constexpr int HI = P % 2;
        if constexpr (P == 3 && B_PAIRS < 2) return;
        const uint32_t dst = dst_w + (uint32_t)((IS_A ? 0 : OPB) + HI * 8 * 1024);
        if constexpr (P == 3 && PARTIAL_B3) {
            const uint32_t d_lo = b3_absent ? spare_lds : dst + q_lo, d_hi = b3_absent ? spare_lds : dst + q_hi;
            if constexpr (KTAIL) {
                dma_load_b128_select(rsrc_b, d_lo, loff_b3, toff_b3[0], l_koff, l_tail);
                dma_load_b128_select(rsrc_b, d_hi, loff_b3, toff_b3[1], l_koff + (uint32_t)(STREAM_SEGK * 2), l_tail);
            } else {
                dma_load_b128(rsrc_b, d_lo, loff_b3, l_koff);
                dma_load_b128(rsrc_b, d_hi, loff_b3, l_koff + (uint32_t)(STREAM_SEGK * 2));
            }
        } else if constexpr (KTAIL) {
            dma_load_b128_select(IS_A ? rsrc_a : rsrc_b, dst + q_lo, HI ? loff_hi : loff_lo, HI ? toff_hi[0] : toff_lo[0], l_koff, l_tail);
            dma_load_b128_select(IS_A ? rsrc_a : rsrc_b, dst + q_hi, HI ? loff_hi : loff_lo, HI ? toff_hi[1] : toff_lo[1],
                                 l_koff + (uint32_t)(STREAM_SEGK * 2), l_tail);
        } else {
            dma_load_b128(IS_A ? rsrc_a : rsrc_b, dst + q_lo, HI ? loff_hi : loff_lo, l_koff);
            dma_load_b128(IS_A ? rsrc_a : rsrc_b, dst + q_hi, HI ? loff_hi : loff_lo, l_koff + (uint32_t)(STREAM_SEGK * 2));
        }
    };

    // ---- multiplier --------------------------------------------------------------------------------
    const int R = wave / 2, Cc = wave % 2;
    const int lr = lane & 15, lg = lane >> 4;
    const int key = swizzle_key(lr, 4);
    const uint32_t a_lane = ring_base + (uint32_t)(R * WTR * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);
    const uint32_t b_lane = ring_base + (uint32_t)OPB + (uint32_t)(Cc * WTC * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);

    u32x4 fa[2][WTR], fb[2][WTC];
    f32x4 acc[WTR][WTC];
#pragma unroll
    for (int i = 0; i < WTR; ++i)
#pragma unroll
        for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // How many stores an interior tile's epilogue leaves in flight, as the code the landing wait takes:
    // 0 = wait for everything (beta is not zero: the epilogue also loads C), 2 = 32 stores (beta is plus or
    // minus zero), 1 = 16 stores (beta zero, 16-bit output through the 16-byte store path below, which
    // needs D and its rows on 16-byte boundaries). Worked out on the scalar unit in asm: a flag the compiler
    // derives from a compare ends up in a vector register, which the "s" operands of the asm statements
    // below cannot take.
    const uint32_t d16_misaligned = H16_WHOLE_LINES ? ((uint32_t)(uintptr_t)g.D | ((uint32_t)g.N << 1)) & 15u : 1u;
    uint32_t count_stores, count_tmp;
    asm volatile("s_lshl_b32 %0, %2, 1\n\ts_cmp_eq_u32 %0, 0\n\ts_cselect_b32 %0, 2, 0\n\t"
                 "s_cmp_eq_u32 %4, 0\n\ts_cselect_b32 %1, %3, 0\n\ts_lshr_b32 %0, %0, %1"
                 : "=&s"(count_stores), "=&s"(count_tmp)
                 : "s"(__builtin_amdgcn_readfirstlane(__builtin_bit_cast(uint32_t, g.beta))),
                   "s"(__builtin_amdgcn_readfirstlane((uint32_t)g.out16)), "s"(__builtin_amdgcn_readfirstlane(d16_misaligned))
                 : "scc");
    uint32_t stores_in_flight;  // nonzero in the loop body that follows an epilogue whose stores count in the wait
    asm volatile("s_mov_b32 %0, 0" : "=s"(stores_in_flight));
    // byte offsets in the ring of the quarters of the even k-step (q0) and of the four after it
    uint32_t q0 = 0, q1 = QB, q2 = 2 * QB, q4 = 4 * QB;

    // One k-step: P selects the fragment buffers; qn is the quarter of the next k-step (its fragments
    // are fetched here); its loads go into quarters q4 and q0.
    auto kstep = [&](auto parity, uint32_t qn) __attribute__((always_inline)) {
        constexpr int P = decltype(parity)::value;
        use_fragments(fa[P], fb[P]);
        if constexpr (P == 1) {
            // loads of the next two k-steps landed: after them this wave issued the four loads of
            // this body's even k-step and, behind an epilogue, the epilogue's stores. (The choice
            // between the two immediates is a scalar branch inside one asm statement: a branch the
            // compiler can see would split the k-step into basic blocks with all 224 accumulator
            // and fragment registers live across them.)
            asm volatile("s_cmp_lg_u32 %0, 0\n\ts_cbranch_scc1 1f\n\ts_waitcnt vmcnt(%1)\n1:\n\t"
                         "s_cmp_eq_u32 %0, 2\n\ts_cbranch_scc1 2f\n\ts_waitcnt vmcnt(%2)\n2:\n\ts_waitcnt vmcnt(%3)"
                         :
                         : "s"(stores_in_flight), "n"(ODD_ONLY ? 0 : EVEN_LOADS), "n"((ODD_ONLY ? 0 : EVEN_LOADS) + EPILOGUE_STORES_16),
                           "n"((ODD_ONLY ? 0 : EVEN_LOADS) + EPILOGUE_STORES)
                         : "memory", "scc");
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < PRE; ++j)
#pragma unroll
            for (int i = 0; i < WTR; ++i) acc[i][j] = MfmaOp<DT>::run(fb[P][j], fa[P][i], acc[i][j]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (!ODD_ONLY || P == 1) wg_barrier();
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t pa = a_lane + qn, pb = b_lane + qn;
#pragma unroll
        for (int j = PRE; j < WTC; ++j) {
#pragma unroll
            for (int q = 0; q < FPC; ++q) {
                const int f = (j - PRE) * FPC + q;
                if (f < WTR) fa[1 - P][f] = *(const CK_LDS u32x4*)(uintptr_t)(pa + (uint32_t)(f * 16 * RB));
                else if (f < WTR + WTC) fb[1 - P][f - WTR] = *(const CK_LDS u32x4*)(uintptr_t)(pb + (uint32_t)((f - WTR) * 16 * RB));
            }
            __builtin_amdgcn_sched_barrier(0);
            // this k-step's share of the loads, spread over the columns (a wave stalls on back-to-back
            // loads, and both waves of a SIMD run in step); with a barrier in every k-step: the pairs of
            // A in the even k-step, those of Bt in the odd one
            if constexpr (ODD_ONLY) {
                // all four pairs in the odd k-step, behind its barrier (the only one of the body)
                if constexpr (P == 1 && WTC == 8) {
                    if (j == 2) issue_pair(std::integral_constant<int, 0>{}, q4, q0);
                    if (j == 4) issue_pair(std::integral_constant<int, 1>{}, q4, q0);
                    if (j == 6) issue_pair(std::integral_constant<int, 2>{}, q4, q0);
                    if (j == 7) issue_pair(std::integral_constant<int, 3>{}, q4, q0);
                }
                if constexpr (P == 1 && WTC == 6) {
                    if (j == 1) issue_pair(std::integral_constant<int, 0>{}, q4, q0);
                    if (j == 2) issue_pair(std::integral_constant<int, 1>{}, q4, q0);
                    if (j == 4) issue_pair(std::integral_constant<int, 2>{}, q4, q0);
                    if (j == 5) issue_pair(std::integral_constant<int, 3>{}, q4, q0);
                }
                if constexpr (P == 1 && WTC == 4) {
                    if (j == 1) issue_pair(std::integral_constant<int, 0>{}, q4, q0);
                    if (j == 2) issue_pair(std::integral_constant<int, 1>{}, q4, q0);
                    if (j == 3) issue_pair(std::integral_constant<int, 2>{}, q4, q0);
                }
            } else {
                if (j == LOAD_COL_0) issue_pair(std::integral_constant<int, 2 * P>{}, q4, q0);
                if (j == LOAD_COL_1) issue_pair(std::integral_constant<int, 2 * P + 1>{}, q4, q0);
            }
            __builtin_amdgcn_sched_barrier(0);
            // every other column runs its rows backwards: one operand register changes per MFMA instead of
            // two at the column boundaries (+0.7 % on random operands, where the device is power-limited)
#pragma unroll
            for (int ii = 0; ii < WTR; ++ii) {
                const int i = (j & 1) ? WTR - 1 - ii : ii;
                acc[i][j] = MfmaOp<DT>::run(fb[P][j], fa[P][i], acc[i][j]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // The two waves of a SIMD run the same code in step; at different priorities one leads and the other
    // fills in while the leader fetches, instead of both fetching and both multiplying at the same moments
    // (+0.7 % on random operands, nothing on all-zero ones).
    if (wave & 4) __builtin_amdgcn_s_setprio(3);
    if (my_tiles > 0) {
        // prologue: the first two bodies' quarters, then the fragments of k-step 0
        loader_open_tile();
        issue_pair(std::integral_constant<int, 0>{}, 0u, (uint32_t)QB);
        issue_pair(std::integral_constant<int, 1>{}, 0u, (uint32_t)QB);
        issue_pair(std::integral_constant<int, 2>{}, 0u, (uint32_t)QB);
        issue_pair(std::integral_constant<int, 3>{}, 0u, (uint32_t)QB);
        loader_advance();
        issue_pair(std::integral_constant<int, 0>{}, (uint32_t)(2 * QB), (uint32_t)(3 * QB));
        issue_pair(std::integral_constant<int, 1>{}, (uint32_t)(2 * QB), (uint32_t)(3 * QB));
        issue_pair(std::integral_constant<int, 2>{}, (uint32_t)(2 * QB), (uint32_t)(3 * QB));
        issue_pair(std::integral_constant<int, 3>{}, (uint32_t)(2 * QB), (uint32_t)(3 * QB));
        loader_advance();
        wait_vmcnt_imm<LPB>();
        wg_barrier();
#pragma unroll
        for (int i = 0; i < WTR; ++i) fa[0][i] = *(const CK_LDS u32x4*)(uintptr_t)(a_lane + (uint32_t)(i * 16 * RB));
#pragma unroll
        for (int j = 0; j < WTC; ++j) fb[0][j] = *(const CK_LDS u32x4*)(uintptr_t)(b_lane + (uint32_t)(j * 16 * RB));

        // K slices reduced in the kernel, without any wave waiting for another. Each wave handles its own wave tile of
        // D, of which S waves (one per slice, in S workgroups) hold a partial sum. Every one of them stores its partial to
        // scratch memory in the accumulators' own layout (1 KiB per store) and then counts itself on the wave tile's
        // counter; the one that finds itself the last adds the partials in slice order - ((p0 + p1) + p2) + ...
        // whichever wave comes last, so the result does not depend on the order of arrival and equals the reduction
        // pass's bit for bit - and runs the ordinary epilogue; the others are done with the tile. Nothing spins: the workgroups of a
        // launch need not be resident together, and other kernels may compete for the device's CUs.
        // Returns whether this wave is the one that writes the wave tile to D.
        auto reduce_slices = [&](int64_t tc, int slice) __attribute__((always_inline)) {
            // The partials cross from one XCD's CU to another's, and the L2s of different XCDs do not see each other's
            // lines. Fences would make that safe by writing back and invalidating whole L2s, once per wave (measured:
            // 45 us per launch); instead the partials are stored and loaded with system-scope accesses (sc0 sc1:
            // written through to memory, read past both caches), a wave counts itself only after its stores have
            // completed, and no cache is touched as a whole.
            constexpr int ROW_BYTES = WTC * 1024;          // one block row of a wave tile: 16 bytes per lane and block
            constexpr int SYSTEM_SCOPE = 1 | 16;           // sc0 | sc1 of a buffer access
            const int unit = __builtin_amdgcn_readfirstlane((int)(tc - T1) * 8 + wave);
            // (one counter per 128-byte line: counters that share a line share a memory channel)
            unsigned int* arrived = g.fix_state + (size_t)unit * (FIX_STATE_STRIDE_BYTES / 4);
            // per (tile, wave): [slice][block row]
            const int unit_bytes = S * WTR * ROW_BYTES;
            const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc((char*)g.fix_partials + (size_t)unit * (size_t)unit_bytes, 0,
                                                                                  unit_bytes, 0x00020000);
            const int ln16 = lane * 16;
            const int mine = __builtin_amdgcn_readfirstlane(slice * WTR * ROW_BYTES);
#pragma unroll
            for (int i = 0; i < WTR; ++i)
#pragma unroll
                for (int j = 0; j < WTC; ++j)
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i][j]), rows, ln16, mine + i * ROW_BYTES + j * 1024, SYSTEM_SCOPE);
            // the stores are complete (in memory) before the wave counts itself
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            unsigned int before = 0;
            if (lane == 0) before = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            before = __builtin_amdgcn_readfirstlane(before);
            asm volatile("" ::: "memory");
            if ((int)before != S - 1) return false;   // another wave will come last
            // Slice order without a second set of accumulators: p0 + p1 is p1 + p0, so the wave of slice 0 or 1 starts
            // from its registers and adds the other of the two; a wave of a later slice starts from p0 and takes its own
            // partial from memory like the others, in its place. Then p2, p3, ... (A partial sum starts from +0 and is
            // never -0, so starting from the first partial and starting from 0 + the first partial are the same.)
            const bool from_registers = slice <= 1;
            const int first = from_registers ? 1 - slice : 0, next = from_registers ? 2 : 1;
#pragma unroll
            for (int i = 0; i < WTR; ++i) {
                {
                    const int at = __builtin_amdgcn_readfirstlane((first * WTR + i) * ROW_BYTES);
                    u32x4 x[WTC];
#pragma unroll
                    for (int j = 0; j < WTC; ++j) x[j] = __builtin_amdgcn_raw_buffer_load_b128(rows, ln16, at + j * 1024, SYSTEM_SCOPE);
#pragma unroll
                    for (int j = 0; j < WTC; ++j) {
                        f32x4 start;
#pragma unroll
                        for (int e = 0; e < 4; ++e) start[e] = from_registers ? acc[i][j][e] : 0.f;
                        acc[i][j] = start + __builtin_bit_cast(f32x4, x[j]);
                    }
                }
                for (int c = next; c < S; ++c) {
                    const int at = __builtin_amdgcn_readfirstlane((c * WTR + i) * ROW_BYTES);
                    u32x4 x[WTC];
#pragma unroll
                    for (int j = 0; j < WTC; ++j) x[j] = __builtin_amdgcn_raw_buffer_load_b128(rows, ln16, at + j * 1024, SYSTEM_SCOPE);
#pragma unroll
                    for (int j = 0; j < WTC; ++j) acc[i][j] += __builtin_bit_cast(f32x4, x[j]);
                }
            }
            return true;
        };
        // D = alpha * acc + beta * C for this wave's wave tile, straight from the accumulators;
        // returns whether the tile is an interior one (every wave then issues exactly the stores the next body's landing wait counts)
        auto write_tile = [&](int64_t tc, int slice) __attribute__((always_inline)) {
            // Every value of C fetched ahead of its use passes through here at the point of use, on every path. The
            // compiler waits for a load where its result is used; when it moves the use under a condition (a row past the
            // edge, beta == 0), the paths that skip the use leave the load in flight as far as it can tell, all the way
            // round to the main loop. There it then waits for ALL loads (vmcnt(0): it knows nothing of the ring's, which
            // are issued from asm) in front of the first LDS read that reuses the register, and the load queue runs
            // empty once per k-step (measured on 16384^3: 7 % of the launch). The empty asm is a use no path can skip.
            auto landed = [](auto& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };
            const bool sliced = slice >= 0;
            const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
            GemmArgs go = g;  // without the reduction in the kernel a K slice writes its own plane of the workspace D points at
            if (sliced && g.fix_partials == nullptr) go.D = g.D + (size_t)slice * ((size_t)g.M * g.N);
            const int m_base = rc.row * TILE + R * WTR * 16 + (int)(threadIdx.x & 15);
            const int n_base = rc.col * TILE_N + Cc * WTC * 16 + (int)((threadIdx.x >> 4) & 3) * 4;
            // vec_cols: every column of the tile is inside the matrix, one vector access per block (rows past M are
            // skipped lane by lane); interior: every row as well, so every wave issues exactly the stores that the next
            // body's landing wait counts
            const bool vec_cols = g.vec_store && (rc.col + 1) * TILE_N <= g.N;
            const bool interior = vec_cols && (rc.row + 1) * TILE <= g.M;
            // rows of D on 128-byte lines: the stores below fill whole lines and bypass L2 retention; otherwise every
            // 128-byte run of a row straddles two lines, and ordinary stores let the halves meet in L2 (N = 4097,
            // 408 tiles: 138 us against 164 with non-temporal stores)
            const bool nt_store = g.nt_store != 0;
            if (vec_cols && !g.out16) {
                // Whole 128-byte lines per store: an accumulator block gives a row 64 bytes (4 lanes x 16),
                // and the write path's cost is per request, not per byte. Two neighbouring blocks are
                // exchanged between lanes so that 8 lanes hold the 32 consecutive floats of one row:
                // store t (0, 1) of a pair writes rows 8t .. 8t+7, lane L the piece L % 8 of row L / 8,
                // which sits in lane (8t + L / 8) + 16 * (piece % 4) of block piece / 4.
                const int piece = lane & 7;
                const int src0 = ((lane >> 3) + 16 * (piece & 3)) * 4;  // byte address of the source lane, t = 0
                const bool second = piece >= 4;
                const int64_t row0 = (int64_t)(rc.row * TILE + R * WTR * 16 + (lane >> 3));
                const int col0 = rc.col * TILE_N + Cc * WTC * 16 + piece * 4;
                const float alpha = g.alpha, beta = g.beta;
                // store s of the epilogue: block row i, group of two block columns j, half tt
                constexpr int GROUPS = WTC / F32_GROUP;
                auto exchanged = [&](int i, int j, int tt) __attribute__((always_inline)) {
                    f32x4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float x0 = acc[i][j][e], x1 = acc[i][j + 1][e];
                        const int a0 = __builtin_amdgcn_ds_bpermute(src0 + tt * 32, __float_as_int(x0));
                        const int a1 = __builtin_amdgcn_ds_bpermute(src0 + tt * 32, __float_as_int(x1));
                        v[e] = __int_as_float(second ? a1 : a0) * alpha;
                    }
                    return v;
                };
                auto put = [&](int64_t off, f32x4 v) __attribute__((always_inline)) {
                    if (nt_store) store_b128_nt(go.D + off, __builtin_bit_cast(u32x4, v));
                    else *(f32x4_u*)(go.D + off) = v;
                };
                if (beta == 0.f) {
#pragma unroll
                    for (int i = 0; i < WTR; ++i) {
#pragma unroll
                        for (int j = 0; j < WTC; j += F32_GROUP) {
#pragma unroll
                            for (int tt = 0; tt < STORES_PER_GROUP; ++tt) {
                                const f32x4 v = exchanged(i, j, tt);
                                const int64_t row = row0 + i * 16 + tt * 8;
                                if (row < g.M) put(row * g.N + (col0 + j * 16), v);
                            }
                        }
                    }
                } else {
                    // C is read C_DEPTH stores ahead of its use: the loads of a wave would otherwise wait for memory one
                    // by one between the stores (a load may not pass the store in front of it)
                    constexpr int C_DEPTH = 4;
                    f32x4 cv[C_DEPTH];
                    auto row_of = [&](int st) { return row0 + (st / (GROUPS * STORES_PER_GROUP)) * 16 + (st % STORES_PER_GROUP) * 8; };
                    auto off_of = [&](int st) { return row_of(st) * g.N + (col0 + ((st / STORES_PER_GROUP) % GROUPS) * F32_GROUP * 16); };
                    auto fetch = [&](int st) __attribute__((always_inline)) {
                        return row_of(st) < g.M ? (f32x4)*(const f32x4_u*)(go.C + off_of(st)) : f32x4{0.f, 0.f, 0.f, 0.f};
                    };
#pragma unroll
                    for (int st = 0; st < C_DEPTH; ++st) cv[st] = fetch(st);
#pragma unroll
                    for (int st = 0; st < EPILOGUE_STORES; ++st) {
                        f32x4 v = exchanged(st / (GROUPS * STORES_PER_GROUP), ((st / STORES_PER_GROUP) % GROUPS) * F32_GROUP, st % STORES_PER_GROUP);
                        landed(cv[st % C_DEPTH]);
                        v += cv[st % C_DEPTH] * beta;
                        if (row_of(st) < g.M) put(off_of(st), v);
                        if (st + C_DEPTH < EPILOGUE_STORES) cv[st % C_DEPTH] = fetch(st + C_DEPTH);
                    }
                }
            } else if (H16_WHOLE_LINES && interior && g.out16 && d16_misaligned == 0) {
                if constexpr (H16_WHOLE_LINES) {
                // 16-bit output in whole 128-byte lines, 16 bytes per lane. A lane's 4 results of a block are
                // 8 bytes, so two neighbouring blocks swap their odd and even 16-lane rows
                // (v_permlane16_swap): lane group G = lane / 16 then holds the 8 columns 8 (G / 2) .. of block
                // j + G % 2, and the 4 lanes of a row 64 consecutive bytes. Two such pairs make a line: the
                // lanes of rows 8 .. 15 hand the second pair's piece to rows 0 .. 7 and take theirs (a
                // rotation by 8 inside each 16-lane row, a DPP move), so that store t writes rows
                // 8t .. 8t+7, first pair from the lanes that own those rows, second pair from the others.
                unsigned short* d16 = (unsigned short*)go.D;
                const bool low_rows = lr < 8;
                const int unit = ((lg & 1) * 2 + (lg >> 1)) * 8;   // column of the lane's piece inside a pair's 32
                const int64_t row0 = (int64_t)(rc.row * TILE + R * WTR * 16 + (lr & 7));
                const int col0 = rc.col * TILE_N + Cc * WTC * 16 + unit;
                const float alpha = g.alpha, beta = g.beta;
                // C (beta not zero) is read in the accumulators' own layout, 8 bytes per lane and block (columns 4 lg ..
                // of row lr), one group of four blocks ahead of its use, and added in fp32 before the one rounding
                const bool with_c = beta != 0.f;
                const unsigned short* c16 = (const unsigned short*)go.C;
                const int64_t c_lane = (int64_t)(rc.row * TILE + R * WTR * 16 + lr) * g.N + (rc.col * TILE_N + Cc * WTC * 16 + lg * 4);
                typedef uint32_t pair_u32 __attribute__((ext_vector_type(2)));
                auto fetch_c = [&](int i, int j, pair_u32 (&c)[H16_GROUP]) __attribute__((always_inline)) {
#pragma unroll
                    for (int b = 0; b < H16_GROUP; ++b)
                        c[b] = with_c ? *(const pair_u32*)(c16 + c_lane + (int64_t)(i * 16) * g.N + (j + b) * 16) : pair_u32{0u, 0u};
                };
                auto scaled = [&](f32x4 x, pair_u32 c) __attribute__((always_inline)) {
                    f32x4 v = x * alpha;
                    if (with_c) {
                        v[0] += Out16<DT>::load((unsigned short)(c[0] & 0xffffu)) * beta;
                        v[1] += Out16<DT>::load((unsigned short)(c[0] >> 16)) * beta;
                        v[2] += Out16<DT>::load((unsigned short)(c[1] & 0xffffu)) * beta;
                        v[3] += Out16<DT>::load((unsigned short)(c[1] >> 16)) * beta;
                    }
                    return v;
                };
                auto packed_pair = [&](f32x4 v0, f32x4 v1) __attribute__((always_inline)) {
                    const uint32_t p00 = (uint32_t)Out16<DT>::store(v0[0]) | ((uint32_t)Out16<DT>::store(v0[1]) << 16);
                    const uint32_t p01 = (uint32_t)Out16<DT>::store(v0[2]) | ((uint32_t)Out16<DT>::store(v0[3]) << 16);
                    const uint32_t p10 = (uint32_t)Out16<DT>::store(v1[0]) | ((uint32_t)Out16<DT>::store(v1[1]) << 16);
                    const uint32_t p11 = (uint32_t)Out16<DT>::store(v1[2]) | ((uint32_t)Out16<DT>::store(v1[3]) << 16);
                    const pair_u32 s0 = __builtin_amdgcn_permlane16_swap(p00, p10, false, false);
                    const pair_u32 s1 = __builtin_amdgcn_permlane16_swap(p01, p11, false, false);
                    return u32x4{s0[0], s1[0], s0[1], s1[1]};
                };
                constexpr int GROUPS16 = WTC / H16_GROUP;
                pair_u32 cq[2][H16_GROUP];
                fetch_c(0, 0, cq[0]);
#pragma unroll
                for (int i = 0; i < WTR; ++i) {
#pragma unroll
                    for (int j = 0; j < WTC; j += H16_GROUP) {
                        const int gi = i * GROUPS16 + j / H16_GROUP;   // this group; the next one's C goes into the other buffer
                        if (gi + 1 < WTR * GROUPS16) fetch_c((gi + 1) / GROUPS16, ((gi + 1) % GROUPS16) * H16_GROUP, cq[(gi + 1) % 2]);
                        landed(cq[gi % 2][0]); landed(cq[gi % 2][1]); landed(cq[gi % 2][2]); landed(cq[gi % 2][3]);
                        const u32x4 first = packed_pair(scaled(acc[i][j], cq[gi % 2][0]), scaled(acc[i][j + 1], cq[gi % 2][1]));
                        const u32x4 second = packed_pair(scaled(acc[i][j + 2], cq[gi % 2][2]), scaled(acc[i][j + 3], cq[gi % 2][3]));
                        u32x4 other;  // the second pair's piece of the row 8 away
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            other[e] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)second[e], 0x128 /* row_ror:8 */, 0xf, 0xf, false);
#pragma unroll
                        for (int tt = 0; tt < STORES_PER_GROUP; ++tt) {
                            const bool own = low_rows == (tt == 0);  // this lane's row is among the store's 8 rows
                            u32x4 o;
#pragma unroll
                            for (int e = 0; e < 4; ++e) o[e] = own ? first[e] : other[e];
                            const int64_t off = (row0 + i * 16 + tt * 8) * g.N + (col0 + j * 16 + (own ? 0 : 32));
                            if (nt_store) store_b128_nt(d16 + off, o);
                            else *(u32x4*)(d16 + off) = o;
                        }
                    }
                }
                }
            } else {
#pragma unroll
                for (int i = 0; i < WTR; ++i)
#pragma unroll
                    for (int j = 0; j < WTC; ++j)
                        epilogue_block<DT>(go, m_base + i * 16, n_base + j * 16, acc[i][j], vec_cols);
            }
            return interior;
        };
        for (int t = 0; t < my_tiles; ++t) {
            int slice = 0;
            const int64_t tc = item_tile(slot + (int64_t)t * grid, slice);
            const bool sliced = slice >= 0;
            const int nb = sliced ? nb_slice : nb_whole;
            for (int b = 0; b < nb; ++b) {
                kstep(std::integral_constant<int, 0>{}, q1);
                kstep(std::integral_constant<int, 1>{}, q2);
                loader_advance();
                asm volatile("s_mov_b32 %0, 0" : "=s"(stores_in_flight));
                // two quarters on: q0 <- q2, q1 <- q3 = q4 - QB (mod ring), q2 <- q4, q4 <- q1
                {
                    const uint32_t n0 = q2, n2 = q4, n4 = q1;
                    uint32_t n1 = q2 + QB;
                    if (n1 == (uint32_t)(NQ * QB)) n1 = 0;
                    q0 = n0; q1 = n1; q2 = n2; q4 = n4;
                }
            }
            // a sliced tile whose slices are added in the kernel is written by the wave that comes last
            const bool reduce_here = !KTAIL && sliced && g.fix_partials != nullptr;
            bool writes = true;
            if constexpr (!KTAIL) {
                if (reduce_here) writes = reduce_slices(tc, slice);
            }
            bool interior = false;
            if (writes) interior = write_tile(tc, slice) && !reduce_here;
#pragma unroll
            for (int i = 0; i < WTR; ++i)
#pragma unroll
                for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
            // (set through asm so that the flag stays one opaque scalar register: otherwise the compiler
            // peels the loop around its known values)
            asm volatile("s_mov_b32 %0, %1" : "=s"(stores_in_flight) : "s"(interior ? count_stores : 0u));
        }
        // the loads issued past the last tile fetch nothing, but they still write the ring
        wait_vmcnt_imm<0>();
    }

    if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
        const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
        g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
        g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
    }
}

}  // namespace ck
#endif  // CK_GEMM_STREAM_KERNEL_HIP_H

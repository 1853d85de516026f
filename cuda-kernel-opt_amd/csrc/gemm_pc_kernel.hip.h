// gemm_shmem_tc_async_opt_port for gfx950: D = alpha * A * Bt^T + beta * C.
//
// A is M x K row-major, Bt is N x K row-major (B passed transposed, as the reference does,
// matmul_shmem_tc_async_opt_port_2.cu:642), both 16-bit (fp16 or bf16); C and D are M x N fp32.
//
// One workgroup per CU, persistent over output tiles (reference kernel role: port_2:638-878).
// Waves [0, PA) stream A K-segments, waves [PA, PA+PB) stream Bt K-segments from HBM/L2 straight
// into a multi-stage LDS ring with buffer_load ... lds (16 B per lane, no VGPR staging); the
// remaining CW waves are consumers running v_mfma_f32_16x16x32 into a per-wave accumulator tile of
// WTR x WTC blocks (the reference's NUM_ACC knob). There is no workgroup barrier in the steady
// state: producers and consumers meet only through monotonically increasing LDS flag counters.
//
//   full  counter: +1 by every producer wave of that operand once its share of the covered rows has
//                  landed in LDS (s_waitcnt vmcnt(n) on its own in-order load queue, then ds_add).
//   empty counter: +1 by every consumer wave that has finished reading the covered rows.
//
// Counters never reset; the fill number f = global_segment / num_stages gives the expected value
// (arrivals_per_fill * (f + 1) for full, * f for empty), so the reference's per-tile balancing
// arrivals (port_2:359-404, :458-482) have no counterpart.
//
// Shift synchronisation (port_1 / port_2) maps to the granularity of those counters:
//   TILE : one full/empty pair per operand and stage.
//   WAVE : the first bar_steps_a wave-tile rows of A and bar_steps_b wave-tile columns of Bt have
//          their own counters; consumer waves in that upper-left rectangle start as soon as THEIR
//          rows and columns have landed. All other waves share one residual counter per operand,
//          signalled after the last row block.
//   ACC  : inside every wave tile the first bar_steps_a 16-row blocks of A and bar_steps_b 16-row
//          blocks of Bt have their own counters; the rest of the wave tile shares a residual one.
//          The consumer then runs accumulator-outer / k-inner for the early columns.
#ifndef CK_GEMM_PC_KERNEL_HIP_H
#define CK_GEMM_PC_KERNEL_HIP_H

#include <hip/hip_runtime.h>
#include "ck_common.h"

namespace ck {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Four fp32 results of one output row as ONE 16-byte access at an address that is only 4-byte aligned (rows of D
// start anywhere when N is not a multiple of 4): global dwordx4 accesses need dword alignment, not 16 bytes.
typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));

#define CK_LDS __attribute__((address_space(3)))

constexpr int RESIDENT_BT_FRAGS = 3;  // Bt fragments kept resident per k-step when a wave tile has more than four block columns

struct GemmArgs {
    const void* A;
    const void* Bt;
    const float* C;
    float* D;
    float alpha, beta;
    int M, N, K;
    int tiles_m, tiles_n;
    int nseg;  // ceil(K / segment_dim_k)
    int tile_group_m, num_stages;
    int pa, pb;  // producer waves on A and on Bt (arrivals per fill on each operand's "full" counters)
    int single_producer;  // one producer wave streams A and then Bt of every segment (port_0's single producer warp); pa = pb = 1
    int bar_steps_a, bar_steps_b;
    int swizzle;
    int num_xcd;
    int vec_store;  // C and D allow one vector access per accumulator block (fp32: always; 16-bit: N % 4 == 0, 8-byte aligned)
    int out16;      // C and D hold the operands' 16-bit element type instead of fp32 (accumulation stays fp32)
    int nt_store;   // D's rows start on 128-byte lines: vector stores of D are non-temporal (they fill whole lines and need not
                    // stay in L2); otherwise ordinary stores, so that the two parts of a line written by different stores meet in L2
    int split_k;    // straight-line kernel only: the tiles from whole_tiles on are cut into this many K slices (>= 1), one
                    // work item per (tile, slice). Without fix_partials slice s writes its partial products to
                    // D + s * M * N (a workspace; alpha 1, beta 0, fp32) and a second kernel adds the planes.
    int split_chunk;  // consecutive work items that belong to one slice (32 = one XCD round, or all sliced tiles if fewer)
    int whole_tiles;  // straight-line kernel only: tile counts [0, whole_tiles) are work items over all of K; the K-sliced
                      // items follow them in the item list (all tiles when split_k is 1)
    // Reduction of the K slices inside the kernel (straight-line kernel): every slice's wave stores its partial sums of a
    // wave tile to fix_partials ([sliced tile][wave][slice][block row], 1 KiB per accumulator block) and counts itself in
    // fix_state, one word per (sliced tile, wave), 128 bytes apart, that starts at zero; the wave that finds itself the
    // last adds the partials in slice order and writes the wave tile of D. Null: no reduction in the kernel.
    float* fix_partials;
    unsigned int* fix_state;
    uint32_t spin_limit;
    int prio_mode;      // 0: producers at raised priority; 1: also asymmetric consumer burst priorities per SIMD pair; 2: none
    int producer_nap;   // s_sleep argument class of the producers' flag polling: 0 -> 1, 1 -> 4, 2 -> 16
    int batched_empty_reads;  // wave-tile granularity: a producer wave reads all "empty" counters of its operand and stage once per segment
    unsigned int* status;  // device words: [0] OR of CK_STATUS_* bits, [2..3] shader cycles and [4..5] 100 MHz
                           // ticks workgroup 0 spent in the last launch (actual-clock evidence)
};

enum : unsigned { CK_STATUS_PRODUCER_TIMEOUT = 1u, CK_STATUS_CONSUMER_TIMEOUT = 2u };

struct f16_tag {};
struct bf16_tag {};
template <typename T> struct MfmaOp;
template <> struct MfmaOp<f16_tag> {
    static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};
template <> struct MfmaOp<bf16_tag> {
    static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};

// ---- epilogue of one 16 x 16 accumulator block: D = alpha * acc + beta * C. With the Bt fragment as the
// first MFMA operand a lane holds 4 consecutive columns (n .. n+3) of one row m. C and D are fp32, or
// (out16) the operands' 16-bit type: the sum is formed in fp32 and rounded to nearest even once.
template <typename T> struct Out16;
template <> struct Out16<f16_tag> {
    static __device__ __forceinline__ float load(unsigned short b) { return (float)__builtin_bit_cast(_Float16, b); }
    static __device__ __forceinline__ unsigned short store(float x) { return __builtin_bit_cast(unsigned short, (_Float16)x); }
};
template <> struct Out16<bf16_tag> {
    static __device__ __forceinline__ float load(unsigned short b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }
    static __device__ __forceinline__ unsigned short store(float x) {
        uint32_t u = __builtin_bit_cast(uint32_t, x);
        if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40u);  // NaN stays NaN
        u += 0x7fffu + ((u >> 16) & 1u);
        return (unsigned short)(u >> 16);
    }
};
// Non-temporal vector stores, written as asm: as a compiler builtin in one branch of a run-time switch with an ordinary
// store of the same value in the other, the two are merged into one ordinary store and the hint is lost. (Addresses
// need 4-byte alignment only. The stores are not waited for anywhere; waits the compiler places for its own loads
// only become stronger by stores it does not know of, since vector memory operations complete in issue order.)
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store_b128_nt(void* p, u32x4 v) { asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(p), "v"(v) : "memory"); }
__device__ __forceinline__ void store_b64_nt(void* p, u32x2 v) { asm volatile("global_store_dwordx2 %0, %1, off nt" ::"v"(p), "v"(v) : "memory"); }

// vec_cols: the tile's columns all lie inside the matrix and C / D allow one vector access per block (fp32: always;
// 16-bit: N % 4 == 0 and 8-byte aligned pointers); rows past M are skipped. Otherwise element by element.
template <typename DT>
__device__ __forceinline__ void epilogue_block(const GemmArgs& g, int m, int n, f32x4 acc, bool vec_cols) {
    const int64_t off = (int64_t)m * g.N + n;
    const float alpha = g.alpha, beta = g.beta;
    f32x4 v = acc * alpha;
    if (m >= g.M) return;
    if (!g.out16) {
        if (vec_cols) {
            if (beta != 0.f) v += *(const f32x4_u*)(g.C + off) * beta;
            // D is written once and not read again: non-temporal, so that it does not displace the operands in L2
            // (rows off the 128-byte lines: ordinary stores, whose partial lines are merged in L2 before they reach memory)
            if (g.nt_store) store_b128_nt(g.D + off, __builtin_bit_cast(u32x4, v));
            else *(f32x4_u*)(g.D + off) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e < g.N) {
                    float x = v[e];
                    if (beta != 0.f) x += g.C[off + e] * beta;
                    g.D[off + e] = x;
                }
            }
        }
    } else {
        const unsigned short* c16 = (const unsigned short*)g.C;
        unsigned short* d16 = (unsigned short*)g.D;
        if (vec_cols) {
            if (beta != 0.f) {
                const uint2 c = *(const uint2*)(c16 + off);
                v[0] += Out16<DT>::load((unsigned short)(c.x & 0xffffu)) * beta;
                v[1] += Out16<DT>::load((unsigned short)(c.x >> 16)) * beta;
                v[2] += Out16<DT>::load((unsigned short)(c.y & 0xffffu)) * beta;
                v[3] += Out16<DT>::load((unsigned short)(c.y >> 16)) * beta;
            }
            uint2 o;
            o.x = (uint32_t)Out16<DT>::store(v[0]) | ((uint32_t)Out16<DT>::store(v[1]) << 16);
            o.y = (uint32_t)Out16<DT>::store(v[2]) | ((uint32_t)Out16<DT>::store(v[3]) << 16);
            if (g.nt_store) store_b64_nt(d16 + off, u32x2{o.x, o.y});
            else *(u32x2*)(d16 + off) = u32x2{o.x, o.y};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e < g.N) {
                    float x = v[e];
                    if (beta != 0.f) x += Out16<DT>::load(c16[off + e]) * beta;
                    d16[off + e] = Out16<DT>::store(x);
                }
            }
        }
    }
}

// ---- LDS flag primitives (inline asm so the compiler's wait-count pass does not tie them to the
// outstanding direct-to-LDS loads and force vmcnt(0) before every flag access) -------------------
__device__ __forceinline__ uint32_t flag_load(uint32_t lds_addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_addr) : "memory");
    return __builtin_amdgcn_readfirstlane(v);
}
// Counters move by exactly 1 per wave: the LDS atomic is issued with only lane 0 enabled. The
// EXEC mask is narrowed and restored inside one asm block; every caller runs with all 64 lanes
// active (no lane-divergent control flow in producers or consumers), so restoring to all ones is
// restoring the caller's mask.
// all earlier LDS reads of this wave have returned before the counter moves
__device__ __forceinline__ void flag_add_after_reads(uint32_t lds_addr) {
    uint32_t one = 1;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_mov_b64 exec, 1\n\tds_add_u32 %0, %1\n\ts_mov_b64 exec, -1" ::"v"(lds_addr), "v"(one) : "memory");
}
__device__ __forceinline__ void flag_add(uint32_t lds_addr) {
    uint32_t one = 1;
    asm volatile("s_mov_b64 exec, 1\n\tds_add_u32 %0, %1\n\ts_mov_b64 exec, -1" ::"v"(lds_addr), "v"(one) : "memory");
}

// Up to five adjacent counters in one round trip to the LDS (the reads are issued back to back and waited for once):
// what a producer wave of the wave-tile granularity looks at once per segment instead of polling every row block's
// counter on its own.
__device__ __forceinline__ void flag_load5(uint32_t lds_addr, int n, uint32_t (&out)[5]) {
    uint32_t v0, v1, v2, v3, v4;
    const uint32_t a1 = lds_addr + (n > 1 ? 4u : 0u), a2 = lds_addr + (n > 2 ? 8u : 0u), a3 = lds_addr + (n > 3 ? 12u : 0u),
                   a4 = lds_addr + (n > 4 ? 16u : 0u);
    asm volatile("ds_read_b32 %0, %5\n\tds_read_b32 %1, %6\n\tds_read_b32 %2, %7\n\tds_read_b32 %3, %8\n\tds_read_b32 %4, %9\n\ts_waitcnt lgkmcnt(0)"
                 : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4)
                 : "v"(lds_addr), "v"(a1), "v"(a2), "v"(a3), "v"(a4)
                 : "memory");
    out[0] = __builtin_amdgcn_readfirstlane(v0); out[1] = __builtin_amdgcn_readfirstlane(v1); out[2] = __builtin_amdgcn_readfirstlane(v2);
    out[3] = __builtin_amdgcn_readfirstlane(v3); out[4] = __builtin_amdgcn_readfirstlane(v4);
}

// Counter read whose answer is needed later: a relaxed workgroup-scope atomic load compiles to a
// plain ds_read_b32 that the compiler's wait-count pass tracks, so the wave keeps issuing and the
// (counted) wait lands at the first use of the value. The read must stay visible to the compiler:
// an inline-asm read would leave it free to copy or spill the destination register before the
// data has arrived.
__device__ __forceinline__ uint32_t flag_peek(uint32_t lds_addr) {
    return __hip_atomic_load((const CK_LDS uint32_t*)(uintptr_t)lds_addr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

template <int N> __device__ __forceinline__ void wait_vmcnt_imm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// wait until at most n of this wave's vector-memory loads are outstanding (n is wave-uniform);
// the immediate is the largest rung not above n, so the wait is exact or slightly early-safe
__device__ __forceinline__ void wait_vmcnt_le(uint32_t n) {
    if (n >= 48) wait_vmcnt_imm<48>();
    else if (n >= 32) wait_vmcnt_imm<32>();
    else if (n >= 24) wait_vmcnt_imm<24>();
    else if (n >= 16) wait_vmcnt_imm<16>();
    else if (n >= 12) wait_vmcnt_imm<12>();
    else if (n >= 8) wait_vmcnt_imm<8>();
    else if (n >= 6) wait_vmcnt_imm<6>();
    else if (n >= 4) wait_vmcnt_imm<4>();
    else if (n == 3) wait_vmcnt_imm<3>();
    else if (n == 2) wait_vmcnt_imm<2>();
    else if (n == 1) wait_vmcnt_imm<1>();
    else wait_vmcnt_imm<0>();
}

// Bounded polling: a wave that exceeds the spin limit records a status bit and stops waiting for
// the rest of the kernel, so every wave reaches the end of the grid whatever goes wrong.
struct Spin {
    uint32_t limit;
    unsigned int* status;
    unsigned bit;
    bool dead;
};
__device__ __forceinline__ bool flag_ready(uint32_t addr, uint32_t target) { return (int32_t)(flag_load(addr) - target) >= 0; }
__device__ __forceinline__ void wait_flag_ge(uint32_t addr, uint32_t target, Spin& sp) {
    if (sp.dead) return;
    uint32_t n = 0;
    while (!flag_ready(addr, target)) {
        if (++n > sp.limit) {
            sp.dead = true;
            if ((threadIdx.x & 63) == 0) atomicOr(sp.status, sp.bit);
            break;
        }
        if (n > 4) __builtin_amdgcn_s_sleep(1);
    }
}

// ---- producer --------------------------------------------------------------------------------------
// Pending "rows landed" signals of one producer wave: a short in-order queue of (counter address,
// number of loads issued when the covered rows were complete). Popping entry e needs at most
// issued_now - e.at loads outstanding, because a wave's loads complete in issue order.
template <int DEPTH> struct SignalQueue {
    uint32_t addr[DEPTH];
    uint32_t at[DEPTH];
    uint32_t issued;
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) { addr[i] = 0; at[i] = 0; }
        issued = 0;
    }
    __device__ __forceinline__ void pop_front() {
        if (addr[0]) {
            wait_vmcnt_le(issued - at[0]);
            flag_add(addr[0] & 0x7fffffffu);
        }
#pragma unroll
        for (int i = 0; i + 1 < DEPTH; ++i) { addr[i] = addr[i + 1]; at[i] = at[i + 1]; }
        addr[DEPTH - 1] = 0;
    }
    __device__ __forceinline__ void push(uint32_t a) {
        pop_front();  // slot DEPTH-1 is free afterwards
        addr[DEPTH - 1] = a | 0x80000000u;  // top bit marks the slot as occupied (LDS address 0 is legal)
        at[DEPTH - 1] = issued;
    }
    __device__ __forceinline__ bool pending() const {
        bool any = false;
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) any |= (addr[i] != 0);
        return any;
    }
    __device__ __forceinline__ void drain() {
        if (!pending()) return;
        wait_vmcnt_imm<0>();
#pragma unroll
        for (int i = 0; i < DEPTH; ++i) {
            if (addr[i]) flag_add(addr[i] & 0x7fffffffu);
            addr[i] = 0;
        }
    }
};

// Wait for an "empty" counter. While it is not there yet the wave keeps retiring its own pending
// "landed" signals oldest first (each needs only the loads up to that entry), so it never blocks
// while holding back a signal the consumers need to make progress.
template <int DEPTH>
__device__ __forceinline__ void producer_wait(uint32_t addr, uint32_t target, SignalQueue<DEPTH>& q, Spin& sp, int nap) {
    if (target == 0 || sp.dead) return;
    uint32_t n = 0;
    while (!flag_ready(addr, target)) {
        if (q.pending()) {
            q.pop_front();
            continue;
        }
        if (++n > sp.limit) {
            sp.dead = true;
            if ((threadIdx.x & 63) == 0) atomicOr(sp.status, sp.bit);
            break;
        }
        if (nap == 0) __builtin_amdgcn_s_sleep(1);
        else if (nap == 1) __builtin_amdgcn_s_sleep(4);
        else __builtin_amdgcn_s_sleep(16);
    }
}

// IS_A selects the operand: A producers walk wave-tile rows, Bt producers wave-tile columns.
// PX = producer waves on this operand; wave q issues the wave loads E with E % PX == q.
//
// Address generation is kept off the vector ALU. A wave load E covers rows [E*RPI, (E+1)*RPI) of
// the operand stage; lane (lane_row, lane_slot) fetches the 16-byte chunk that belongs at its
// linear LDS slot under the XOR swizzle. The swizzle key of a lane repeats with period VAR in E,
// so VAR per-lane byte offsets (row-in-load * pitch + chunk * 16) are computed once per kernel and
// everything that changes from load to load (E * RPI * pitch), from segment to segment (k0 * 2)
// and from tile to tile (the buffer base) is scalar: the load's soffset, M0 and the descriptor.
// The scalar offset is not range-checked by the buffer unit, so that fast path is taken only when
// all rows of the tile and all k of the segment exist; edge tiles and the K tail put the whole
// offset in the range-checked vector offset and push absent k out of range (zero fill).
template <int TILE, int SEGK, int CW, int MODE, bool IS_A, int PX>
__device__ __forceinline__ void produce(const GemmArgs& g, uint32_t flags_base, uint32_t ring_base, int q, int lane) {
    constexpr int WTR = TILE / (CW / 2) / MFMA_M, WTC = TILE / 2 / MFMA_N;
    constexpr int CPR = SEGK / CHUNK_ELEMS;      // 16-byte chunks per row
    constexpr int RB = SEGK * 2;                 // row bytes in LDS
    constexpr int RPI = WAVE / CPR;              // rows one wave load covers
    constexpr int OPB = TILE * RB;               // bytes of one operand stage
    constexpr int BLK_ROWS = MODE == CK_SYNC_TILE ? TILE : MODE == CK_SYNC_WAVE ? (IS_A ? WTR : WTC) * 16 : 16;
    constexpr int NBLK = TILE / BLK_ROWS;
    constexpr int NIB = BLK_ROWS / RPI;          // wave loads per row block
    constexpr int VAR = CPR == 4 ? 1 : CPR == 8 ? 2 : CPR == 16 ? 4 : 8;  // period of the swizzle key in E
    static_assert(BLK_ROWS % RPI == 0, "row block must be whole wave loads");

    const int sa = g.bar_steps_a, sb = g.bar_steps_b;
    const int S = g.num_stages;
    const int ua = units_a(MODE, CW, sa), ub = units_b(MODE, CW, sb);
    const int fps = 2 * ua + 2 * ub;
    // counters of this operand inside one stage's flag set
    const uint32_t full_off = IS_A ? 0 : 2 * ua;
    const uint32_t empty_off = IS_A ? ua : 2 * ua + ub;
    const int nres = CW - sa * sb;  // WAVE mode: consumer waves on the residual counters

    const char* base = (const char*)(IS_A ? g.A : g.Bt);
    const int rows_total = IS_A ? g.M : g.N;
    const int64_t pitch = (int64_t)g.K * 2;
    const uint32_t pitch32 = (uint32_t)pitch;

    const int lane_row = lane / CPR, lane_slot = lane % CPR;
    uint32_t lane_off[VAR];  // row-in-load * pitch + logical chunk * 16, per swizzle-key variant
    int lane_chunk[VAR];
#pragma unroll
    for (int v = 0; v < VAR; ++v) {
        lane_chunk[v] = swizzle_slot(v * RPI + lane_row, lane_slot, CPR, g.swizzle);
        lane_off[v] = (uint32_t)lane_row * pitch32 + (uint32_t)lane_chunk[v] * CHUNK_BYTES;
    }
    const uint32_t load_step = (uint32_t)RPI * pitch32;  // bytes between consecutive wave loads

    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    const int64_t total_tiles = (int64_t)g.tiles_m * g.tiles_n;

    Spin sp{g.spin_limit, g.status, CK_STATUS_PRODUCER_TIMEOUT, false};
    SignalQueue<MODE == CK_SYNC_TILE ? 3 : MODE == CK_SYNC_WAVE ? 4 : 8> sq;
    sq.init();

    int stage = 0;
    uint32_t fill = 0;
    for (int64_t tc = slot; tc < total_tiles; tc += grid) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
        const int row0 = __builtin_amdgcn_readfirstlane((IS_A ? rc.row : rc.col) * TILE);
        int rows_here = rows_total - row0;
        rows_here = rows_here < TILE ? rows_here : TILE;
        const uint32_t num_records = (uint32_t)((int64_t)rows_here * pitch);
        __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc((void*)(base + (int64_t)row0 * pitch), 0, (int)num_records, 0x00020000);
        const bool all_rows = rows_here == TILE;

        for (int seg = 0; seg < g.nseg; ++seg) {
            // loop-carried scalars are pinned to SGPRs so that address and flag arithmetic stays scalar
            stage = __builtin_amdgcn_readfirstlane(stage);
            fill = __builtin_amdgcn_readfirstlane(fill);
            const uint32_t fl = flags_base + (uint32_t)stage * fps * 4;
            const uint32_t st_base = ring_base + (uint32_t)stage * (2 * OPB) + (IS_A ? 0 : OPB);
            const int k0 = seg * SEGK;
            const bool fast = all_rows && k0 + SEGK <= g.K;
            // wave-tile granularity: all "empty" counters of this operand and stage in one look (g.batched_empty_reads);
            // a row block whose counter was already there is not polled again
            uint32_t seen[5] = {0, 0, 0, 0, 0};
            const bool batched = MODE == CK_SYNC_WAVE && g.batched_empty_reads && fill > 0;
            if (MODE == CK_SYNC_WAVE) {
                if (batched) flag_load5(fl + empty_off * 4, (IS_A ? sa : sb) + 1, seen);
            }
            auto wave_wait = [&](int idx, uint32_t target) __attribute__((always_inline)) {
                if (batched && (int32_t)(seen[idx] - target) >= 0) return;
                producer_wait(fl + (empty_off + idx) * 4, target, sq, sp, g.producer_nap);
            };
#pragma unroll
            for (int blk = 0; blk < NBLK; ++blk) {
                // ---- wait until the consumers of the previous fill have released these rows
                if (MODE == CK_SYNC_TILE) {
                    producer_wait(fl + (empty_off + 0) * 4, CW * fill, sq, sp, g.producer_nap);
                } else if (MODE == CK_SYNC_WAVE) {
                    const int s_own = IS_A ? sa : sb, s_oth = IS_A ? sb : sa;
                    const int oth_max = IS_A ? 2 : CW / 2;
                    const bool first_has_res = (s_own == 0 || s_oth < oth_max);
                    if (blk == 0 && first_has_res && nres > 0) wave_wait(s_own, nres * fill);
                    if (blk < s_own && s_oth > 0) {
                        wave_wait(blk, s_oth * fill);
                    } else if (blk == s_own && !first_has_res && nres > 0) {
                        wave_wait(s_own, nres * fill);
                    }
                } else {
                    constexpr int WT = IS_A ? WTR : WTC;
                    const int s_own = IS_A ? sa : sb;
                    const int unit = blk / WT, sub = blk % WT;
                    const int readers = IS_A ? 2 : CW / 2;
                    if (sub <= s_own) producer_wait(fl + (empty_off + unit * (s_own + 1) + sub) * 4, readers * fill, sq, sp, g.producer_nap);
                }
                // ---- this wave's share of the row block, straight into LDS
                if (fast) {
                    const uint32_t soff0 = (uint32_t)k0 * 2u;
#pragma unroll
                    for (int e = 0; e < NIB; ++e) {
                        const int E = blk * NIB + e;
                        if (PX > 1 && E % PX != q) continue;
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (CK_LDS void*)(uintptr_t)(st_base + (uint32_t)E * 1024u), 16,
                                                                 lane_off[E % VAR], soff0 + (uint32_t)E * load_step, 0, 0);
                        sq.issued++;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < NIB; ++e) {
                        const int E = blk * NIB + e;
                        if (PX > 1 && E % PX != q) continue;
                        uint32_t voff = lane_off[E % VAR] + (uint32_t)E * load_step + (uint32_t)k0 * 2u;
                        if (k0 + lane_chunk[E % VAR] * CHUNK_ELEMS >= g.K) voff = num_records;  // absent k: zero fill
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (CK_LDS void*)(uintptr_t)(st_base + (uint32_t)E * 1024u), 16, voff, 0, 0, 0);
                        sq.issued++;
                    }
                }
                // ---- queue the "landed" signals this block completes
                if (MODE == CK_SYNC_TILE) {
                    sq.push(fl + (full_off + 0) * 4);
                } else if (MODE == CK_SYNC_WAVE) {
                    const int s_own = IS_A ? sa : sb;
                    if (blk < s_own) sq.push(fl + (full_off + blk) * 4);
                    if (blk == NBLK - 1) sq.push(fl + (full_off + s_own) * 4);
                } else {
                    constexpr int WT = IS_A ? WTR : WTC;
                    const int s_own = IS_A ? sa : sb;
                    const int unit = blk / WT, sub = blk % WT;
                    if (sub < s_own) sq.push(fl + (full_off + unit * (s_own + 1) + sub) * 4);
                    else if (sub == WT - 1) sq.push(fl + (full_off + unit * (s_own + 1) + s_own) * 4);
                }
            }
            if (++stage == S) { stage = 0; ++fill; }
        }
    }
    sq.drain();
}

// The single producer wave of the port_0 launcher (port_0.cu:106-147 with one producer warp): tile granularity, the one
// wave streams the A rows and then the Bt rows of every segment and is the one arrival on each operand's "full" counter.
template <int TILE, int SEGK, int CW>
__device__ __forceinline__ void produce_both(const GemmArgs& g, uint32_t flags_base, uint32_t ring_base, int lane) {
    constexpr int CPR = SEGK / CHUNK_ELEMS, RB = SEGK * 2, RPI = WAVE / CPR, OPB = TILE * RB;
    constexpr int NI = TILE / RPI;               // wave loads per operand stage
    constexpr int VAR = CPR == 4 ? 1 : CPR == 8 ? 2 : CPR == 16 ? 4 : 8;
    constexpr int FPS = 4;                        // counters per stage: full A, empty A, full Bt, empty Bt
    const int S = g.num_stages;
    const int64_t pitch = (int64_t)g.K * 2;
    const uint32_t pitch32 = (uint32_t)pitch;
    const int lane_row = lane / CPR, lane_slot = lane % CPR;
    uint32_t lane_off[VAR];
    int lane_chunk[VAR];
#pragma unroll
    for (int v = 0; v < VAR; ++v) {
        lane_chunk[v] = swizzle_slot(v * RPI + lane_row, lane_slot, CPR, g.swizzle);
        lane_off[v] = (uint32_t)lane_row * pitch32 + (uint32_t)lane_chunk[v] * CHUNK_BYTES;
    }
    const uint32_t load_step = (uint32_t)RPI * pitch32;
    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    const int64_t total_tiles = (int64_t)g.tiles_m * g.tiles_n;
    Spin sp{g.spin_limit, g.status, CK_STATUS_PRODUCER_TIMEOUT, false};
    SignalQueue<3> sq;
    sq.init();
    int stage = 0;
    uint32_t fill = 0;
    for (int64_t tc = slot; tc < total_tiles; tc += grid) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
        for (int seg = 0; seg < g.nseg; ++seg) {
            stage = __builtin_amdgcn_readfirstlane(stage);
            fill = __builtin_amdgcn_readfirstlane(fill);
            const uint32_t fl = flags_base + (uint32_t)stage * FPS * 4;
            const int k0 = seg * SEGK;
#pragma unroll
            for (int op = 0; op < 2; ++op) {
                const int row0 = __builtin_amdgcn_readfirstlane((op == 0 ? rc.row : rc.col) * TILE);
                int rows_here = (op == 0 ? g.M : g.N) - row0;
                rows_here = rows_here < TILE ? rows_here : TILE;
                const uint32_t num_records = (uint32_t)((int64_t)rows_here * pitch);
                __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                    (void*)((const char*)(op == 0 ? g.A : g.Bt) + (int64_t)row0 * pitch), 0, (int)num_records, 0x00020000);
                const uint32_t st_base = ring_base + (uint32_t)stage * (2 * OPB) + (op == 0 ? 0 : OPB);
                producer_wait(fl + (op == 0 ? 1 : 3) * 4, CW * fill, sq, sp, g.producer_nap);
                if (rows_here == TILE && k0 + SEGK <= g.K) {
#pragma unroll
                    for (int E = 0; E < NI; ++E) {
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (CK_LDS void*)(uintptr_t)(st_base + (uint32_t)E * 1024u), 16,
                                                                 lane_off[E % VAR], (uint32_t)k0 * 2u + (uint32_t)E * load_step, 0, 0);
                        sq.issued++;
                    }
                } else {
#pragma unroll
                    for (int E = 0; E < NI; ++E) {
                        uint32_t voff = lane_off[E % VAR] + (uint32_t)E * load_step + (uint32_t)k0 * 2u;
                        if (k0 + lane_chunk[E % VAR] * CHUNK_ELEMS >= g.K) voff = num_records;  // absent k: zero fill
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (CK_LDS void*)(uintptr_t)(st_base + (uint32_t)E * 1024u), 16, voff, 0, 0, 0);
                        sq.issued++;
                    }
                }
                sq.push(fl + (op == 0 ? 0 : 2) * 4);
            }
            if (++stage == S) { stage = 0; ++fill; }
        }
    }
    sq.drain();
}

template <int TILE, int SEGK, int CW, int MODE, bool IS_A>
__device__ __forceinline__ void produce_px(const GemmArgs& g, uint32_t flags_base, uint32_t ring_base, int q, int px, int lane) {
    if (px == 1) produce<TILE, SEGK, CW, MODE, IS_A, 1>(g, flags_base, ring_base, q, lane);
    else if (px == 2) produce<TILE, SEGK, CW, MODE, IS_A, 2>(g, flags_base, ring_base, q, lane);
    else produce<TILE, SEGK, CW, MODE, IS_A, 4>(g, flags_base, ring_base, q, lane);
}

// ---- consumer ----------------------------------------------------------------------------------------
template <typename DT, int TILE, int SEGK, int CW, int MODE>
__device__ __forceinline__ void consume(const GemmArgs& g, uint32_t flags_base, uint32_t ring_base, int cw, int lane) {
    constexpr int WTR = TILE / (CW / 2) / MFMA_M, WTC = TILE / 2 / MFMA_N;
    constexpr int CPR = SEGK / CHUNK_ELEMS;
    constexpr int RB = SEGK * 2;
    constexpr int OPB = TILE * RB;
    constexpr int KSTEPS = SEGK / MFMA_K;

    const int sa = g.bar_steps_a, sb = g.bar_steps_b;
    const int S = g.num_stages;
    const int ua = units_a(MODE, CW, sa), ub = units_b(MODE, CW, sb);
    const int fps = 2 * ua + 2 * ub;
    const int R = cw / 2, Cc = cw % 2;  // wave-tile row / column of this wave
    const uint32_t pa = g.pa, pb = g.pb;

    // lane -> fragment element: row (lane % 16) of a 16-row block, logical chunk kstep*4 + lane/16
    const int lr = lane & 15, lg = lane >> 4;
    const int key = g.swizzle ? swizzle_key(lr, CPR) : 0;  // same for every 16-row block
    // Per-lane LDS offset of the k-step-0 fragment chunk. Row offsets are multiples of the row size
    // and stage bases multiples of 1 KiB, so the chunk of k-step ks is reached by XOR with ks * 64:
    // ((ks*4 + lg) ^ key) * 16 == ((lg ^ key) * 16) ^ (ks * 64).
    const uint32_t a_lane = (uint32_t)(R * WTR * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);
    const uint32_t b_lane = (uint32_t)OPB + (uint32_t)(Cc * WTC * 16 + lr) * RB + (uint32_t)((lg ^ key) * CHUNK_BYTES);

    const int grid = gridDim.x;
    const int slot = xcd_slot(blockIdx.x, grid, g.num_xcd);
    const int64_t total_tiles = (int64_t)g.tiles_m * g.tiles_n;
    Spin sp{g.spin_limit, g.status, CK_STATUS_CONSUMER_TIMEOUT, false};

    // waves are dealt to the four SIMDs round-robin, so consumer cw shares its SIMD with cw +- 4
    const bool burst_hi = (cw & 4) == 0;
    // WAVE mode: which counters this wave uses
    const bool individual = (MODE == CK_SYNC_WAVE) && R < sa && Cc < sb;
    int fa_idx = 0, fb_idx = 0;
    if (MODE == CK_SYNC_WAVE) { fa_idx = individual ? R : sa; fb_idx = individual ? Cc : sb; }

    int stage = 0;
    uint32_t fill = 0;
    uint32_t pre_a = 0, pre_b = 0;  // "full" counters of the upcoming segment, read ahead of time
    for (int64_t tc = slot; tc < total_tiles; tc += grid) {
        const TileRC rc = tile_order(g.tiles_m, g.tiles_n, g.tile_group_m, tc);
        f32x4 acc[WTR][WTC];
#pragma unroll
        for (int i = 0; i < WTR; ++i)
#pragma unroll
            for (int j = 0; j < WTC; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

        for (int seg = 0; seg < g.nseg; ++seg) {
            const uint32_t fl = flags_base + (uint32_t)stage * fps * 4;
            const uint32_t st = ring_base + (uint32_t)stage * (2 * OPB);
            const uint32_t fullA = fl, emptyA = fl + ua * 4, fullB = fl + 2 * ua * 4, emptyB = fl + (2 * ua + ub) * 4;

            if (MODE != CK_SYNC_ACC) {
                // The two "full" counters of this segment were read one segment ahead (behind the
                // previous segment's fragment reads); poll only if they were not there yet.
                const uint32_t seen_a = __builtin_amdgcn_readfirstlane(pre_a);
                const uint32_t seen_b = __builtin_amdgcn_readfirstlane(pre_b);
                if ((int32_t)(seen_a - pa * (fill + 1)) < 0) wait_flag_ge(fullA + fa_idx * 4, pa * (fill + 1), sp);
                if ((int32_t)(seen_b - pb * (fill + 1)) < 0) wait_flag_ge(fullB + fb_idx * 4, pb * (fill + 1), sp);
                asm volatile("" ::: "memory");
                {
                    const int nstage = stage + 1 == S ? 0 : stage + 1;
                    const uint32_t nfl = flags_base + (uint32_t)nstage * fps * 4;
                    pre_a = flag_peek(nfl + fa_idx * 4);
                    pre_b = flag_peek(nfl + 2 * ua * 4 + fb_idx * 4);
                }
#pragma unroll
                for (int ks = 0; ks < KSTEPS; ++ks) {
                    const uint32_t pa_k = (st + a_lane) ^ (uint32_t)(ks * 64), pb_k = (st + b_lane) ^ (uint32_t)(ks * 64);
                    // At most JB Bt fragments are resident; fragment j + JB replaces fragment j
                    // right after its last use, so a 4 x 8 wave tile needs 32 fragment registers
                    // next to its 128 accumulator registers.
                    constexpr int JB = WTC > 4 ? RESIDENT_BT_FRAGS : WTC;
                    u32x4 a[WTR], b[JB];
                    // Fragment-load phase at low priority, MFMA burst at a raised one. The two consumer
                    // waves that share a SIMD raise to DIFFERENT levels: when both have MFMAs ready one
                    // of them wins the matrix core outright, finishes its burst first and loads its next
                    // fragments while the other bursts, so the pair settles into ping-pong instead of
                    // stalling on LDS latency in lockstep.
                    if (g.prio_mode == 1) __builtin_amdgcn_s_setprio(0);
#pragma unroll
                    for (int i = 0; i < WTR; ++i) a[i] = *(const CK_LDS u32x4*)(uintptr_t)(pa_k + i * 16 * RB);
#pragma unroll
                    for (int j = 0; j < JB; ++j) b[j] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + j * 16 * RB);
                    __builtin_amdgcn_sched_barrier(0);
                    if (g.prio_mode == 1) {
                        if (burst_hi) __builtin_amdgcn_s_setprio(2);
                        else __builtin_amdgcn_s_setprio(1);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                    if (ks == KSTEPS - 1 && JB == WTC) {
                        flag_add_after_reads(emptyA + fa_idx * 4);
                        flag_add(emptyB + fb_idx * 4);
                    }
#pragma unroll
                    for (int j = 0; j < WTC; ++j) {
                        if (ks == KSTEPS - 1 && JB != WTC && j == WTC - 1) {
                            flag_add_after_reads(emptyA + fa_idx * 4);
                            flag_add(emptyB + fb_idx * 4);
                        }
#pragma unroll
                        for (int i = 0; i < WTR; ++i) {
                            acc[i][j] = MfmaOp<DT>::run(b[j % JB], a[i], acc[i][j]);
                        }
                        if (j + JB < WTC) {
                            __builtin_amdgcn_sched_barrier(0);
                            b[j % JB] = *(const CK_LDS u32x4*)(uintptr_t)(pb_k + (j + JB) * 16 * RB);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
            } else {
                // accumulator granularity: counters per (wave-tile row, 16-row block) and per
                // (wave-tile column, 16-row block); early columns run accumulator-outer, k-inner
                const uint32_t fa = fullA + R * (sa + 1) * 4, ea = emptyA + R * (sa + 1) * 4;
                const uint32_t fb = fullB + Cc * (sb + 1) * 4, eb = emptyB + Cc * (sb + 1) * 4;
                int a_waited = -1;  // highest A counter index already waited for in this segment
                // phase 1: every row against the first sb columns
#pragma unroll
                for (int i = 0; i < WTR; ++i) {
#pragma unroll
                    for (int j = 0; j < WTC; ++j) {
                        if (j < sb) {
                            const int ai = i < sa ? i : sa;
                            if (ai > a_waited) { wait_flag_ge(fa + ai * 4, pa * (fill + 1), sp); a_waited = ai; }
                            if (i == 0) wait_flag_ge(fb + j * 4, pb * (fill + 1), sp);
#pragma unroll
                            for (int ks = 0; ks < KSTEPS; ++ks) {
                                const u32x4 av = *(const CK_LDS u32x4*)(uintptr_t)(((st + a_lane) ^ (uint32_t)(ks * 64)) + i * 16 * RB);
                                const u32x4 bv = *(const CK_LDS u32x4*)(uintptr_t)(((st + b_lane) ^ (uint32_t)(ks * 64)) + j * 16 * RB);
                                acc[i][j] = MfmaOp<DT>::run(bv, av, acc[i][j]);
                            }
                            if (i == WTR - 1) flag_add_after_reads(eb + j * 4);
                        }
                    }
                }
                // phase 2: every row against the residual columns
                wait_flag_ge(fb + sb * 4, pb * (fill + 1), sp);
#pragma unroll
                for (int i = 0; i < WTR; ++i) {
                    const int ai = i < sa ? i : sa;
                    if (ai > a_waited) { wait_flag_ge(fa + ai * 4, pa * (fill + 1), sp); a_waited = ai; }
                    u32x4 a[KSTEPS];
#pragma unroll
                    for (int ks = 0; ks < KSTEPS; ++ks) {
                        a[ks] = *(const CK_LDS u32x4*)(uintptr_t)(((st + a_lane) ^ (uint32_t)(ks * 64)) + i * 16 * RB);
                    }
#pragma unroll
                    for (int j = 0; j < WTC; ++j) {
                        if (j >= sb) {
#pragma unroll
                            for (int ks = 0; ks < KSTEPS; ++ks) {
                                const u32x4 bv = *(const CK_LDS u32x4*)(uintptr_t)(((st + b_lane) ^ (uint32_t)(ks * 64)) + j * 16 * RB);
                                acc[i][j] = MfmaOp<DT>::run(bv, a[ks], acc[i][j]);
                            }
                        }
                    }
                    if (i < sa) flag_add_after_reads(ea + i * 4);
                    if (i == WTR - 1) {
                        flag_add_after_reads(ea + sa * 4);
                        flag_add(eb + sb * 4);
                    }
                }
            }
            if (++stage == S) { stage = 0; ++fill; }
        }

        // ---- epilogue: D = alpha * acc + beta * C straight from the accumulators. With the Bt
        // fragment as the first MFMA operand a lane holds 4 consecutive columns of one row.
        const int m_base = rc.row * TILE + R * WTR * 16 + (int)(threadIdx.x & 15);
        const int n_base = rc.col * TILE + Cc * WTC * 16 + (int)((threadIdx.x >> 4) & 3) * 4;
        const bool vec_cols = g.vec_store && (rc.col + 1) * TILE <= g.N;
#pragma unroll
        for (int i = 0; i < WTR; ++i) {
#pragma unroll
            for (int j = 0; j < WTC; ++j) epilogue_block<DT>(g, m_base + i * 16, n_base + j * 16, acc[i][j], vec_cols);
        }
    }
}

template <typename DT, int TILE, int SEGK, int CW, int MODE, int MAXW>
__global__ __launch_bounds__(MAXW * 64) void gemm_pc_kernel(const GemmArgs g) {
    extern __shared__ __attribute__((aligned(1024))) char ck_smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(CK_LDS char*)ck_smem;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;

    const unsigned long long clk0 = clock64(), wall0 = wall_clock64();
    const int fregion = flag_region_bytes(MODE, CW, g.bar_steps_a, g.bar_steps_b, g.num_stages);
    for (int i = threadIdx.x; i < fregion / 4; i += blockDim.x) ((CK_LDS uint32_t*)ck_smem)[i] = 0;
    __syncthreads();

    const uint32_t flags_base = lds0, ring_base = lds0 + fregion;
    // producers are rarely runnable and must issue their loads promptly when they are
    if (MODE == CK_SYNC_TILE && g.single_producer) {
        if constexpr (MODE == CK_SYNC_TILE) {
            if (wave == 0) {
                if (g.prio_mode != 2) __builtin_amdgcn_s_setprio(3);
                produce_both<TILE, SEGK, CW>(g, flags_base, ring_base, lane);
            } else if (wave < 1 + CW) {
                consume<DT, TILE, SEGK, CW, MODE>(g, flags_base, ring_base, wave - 1, lane);
                if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
                    const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
                    g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
                    g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
                }
            }
        }
        return;
    }
    if (wave < g.pa + g.pb && g.prio_mode != 2) __builtin_amdgcn_s_setprio(3);
    if (wave < g.pa) {
        produce_px<TILE, SEGK, CW, MODE, true>(g, flags_base, ring_base, wave, g.pa, lane);
    } else if (wave < g.pa + g.pb) {
        produce_px<TILE, SEGK, CW, MODE, false>(g, flags_base, ring_base, wave - g.pa, g.pb, lane);
    } else if (wave < g.pa + g.pb + CW) {
        consume<DT, TILE, SEGK, CW, MODE>(g, flags_base, ring_base, wave - g.pa - g.pb, lane);
        // the last consumer wave of workgroup 0 records how long the workgroup ran
        if (blockIdx.x == 0 && threadIdx.x == blockDim.x - 1) {
            const unsigned long long dc = clock64() - clk0, dw = wall_clock64() - wall0;
            g.status[2] = (unsigned)dc; g.status[3] = (unsigned)(dc >> 32);
            g.status[4] = (unsigned)dw; g.status[5] = (unsigned)(dw >> 32);
        }
    }
}

}  // namespace ck
#endif  // CK_GEMM_PC_KERNEL_HIP_H

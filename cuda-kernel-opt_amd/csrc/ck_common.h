// Pure index arithmetic shared by the host launch layer, the gfx950 kernels and the CPU unit tests.
//
// Everything here is a constexpr/inline integer function with no HIP dependency, so the same code
// is compiled by hipcc into the kernels and by g++ into the host-only test helper.
//
// Reference functions these follow (semantics, not code):
//   get_num_acc / get_warp_tile_rows      matmul_shmem_tc_async_opt_port_2.cu:158-169
//   get_tile_offset_cd                    matmul_shmem_tc_async_opt_port_2.cu:605-614
//   launcher parameter legality           matmul_shmem_tc_async_opt_port_2.cu:1110-1123
//   get_shmem_req (role only)             matmul_shmem_tc_async_opt_port_2.cu:1057-1086
#ifndef CK_COMMON_H
#define CK_COMMON_H

#include <stdint.h>

#if defined(__HIPCC__)
#define CK_HD __host__ __device__ inline
#else
#define CK_HD inline
#endif

namespace ck {

// ---- error codes returned by every extern "C" entry point -------------------------------------
enum : int {
    CK_OK = 0,
    CK_ERR_BAD_PARAM = -1,      // a tuning or shape parameter is outside the legal set
    CK_ERR_LDS_BUDGET = -2,     // the requested ring does not fit the 160 KiB LDS of one CU
    CK_ERR_NO_INSTANCE = -3,    // legal in principle, but no kernel instance is compiled for it
    CK_ERR_HIP = -4,            // a HIP runtime call failed
    CK_ERR_ALIGNMENT = -5,      // pointer or row pitch not aligned as the kernel requires
    CK_ERR_NULL = -6,           // a required pointer is null
    CK_ERR_TOO_LARGE = -7,      // a size exceeds what an entry point supports
};

enum : int { CK_DT_F16 = 0, CK_DT_BF16 = 1, CK_DT_F32 = 2, CK_DT_I32 = 3 };

// Granularity at which producers signal "rows landed" and consumers release them.
enum : int { CK_SYNC_TILE = 0, CK_SYNC_WAVE = 1, CK_SYNC_ACC = 2 };

constexpr int MFMA_M = 16;       // rows of one accumulator block
constexpr int MFMA_N = 16;       // columns of one accumulator block
constexpr int MFMA_K = 32;       // K depth of v_mfma_f32_16x16x32_{f16,bf16}
constexpr int WAVE = 64;
constexpr int LDS_BYTES_PER_CU = 160 * 1024;
constexpr int CHUNK_BYTES = 16;  // one lane of a dwordx4 direct-to-LDS load
constexpr int CHUNK_ELEMS = 8;   // 16-bit elements per chunk
constexpr int FLAG_REGION_ALIGN = 1024;
constexpr int MAX_STAGES = 16;

CK_HD int align_up(int x, int a) { return (x + a - 1) / a * a; }
CK_HD int64_t ceil_div64(int64_t x, int64_t a) { return (x + a - 1) / a; }

// Consumer waves are arranged (C/2) x 2 over the tile, as the reference arranges its warps
// (port_2:804-806). One wave owns wave_tile_rows x wave_tile_cols accumulator blocks of 16x16.
CK_HD int wave_tile_rows(int tile_dim, int consumer_waves) { return tile_dim / (consumer_waves / 2) / MFMA_M; }
CK_HD int wave_tile_cols(int tile_dim, int /*consumer_waves*/) { return tile_dim / 2 / MFMA_N; }

// Accumulator blocks (16x16) per consumer wave. Agrees with the reference's closed form
// (4>>(t==64)) * ((4>>(t==64))>>(C==8)) on its domain t in {64,128}, C in {4,8}, and extends it
// to t = 256.
CK_HD int get_num_acc(int tile_dim, int consumer_waves) {
    return wave_tile_rows(tile_dim, consumer_waves) * wave_tile_cols(tile_dim, consumer_waves);
}
CK_HD int get_warp_tile_rows(int tile_dim, int consumer_waves) { return wave_tile_rows(tile_dim, consumer_waves); }

// Grouped tile order: groups of tile_group_m tile-rows, column-major inside a group, the last group
// may be short. Returns the tile's (row, col) in units of tiles. tiles_m/tiles_n are ceil-divided
// tile counts, so ragged problems use the same order.
struct TileRC { int row, col; };
CK_HD TileRC tile_order(int tiles_m, int tiles_n, int tile_group_m, int64_t tile_count) {
    const int64_t group_tile_count = (int64_t)tile_group_m * tiles_n;
    const int group_first_row = (int)(tile_count / group_tile_count) * tile_group_m;
    const int rem_rows = tiles_m - group_first_row;
    const int group_rows = rem_rows < tile_group_m ? rem_rows : tile_group_m;
    const int in_group = (int)(tile_count % group_tile_count);
    TileRC rc;
    rc.row = group_first_row + in_group % group_rows;
    rc.col = in_group / group_rows;
    return rc;
}

// Element offset of a tile in C/D, 64-bit (the reference's int version overflows past 46K^2).
CK_HD int64_t get_tile_offset_cd(int M, int N, int tile_dim, int tile_group_m, int64_t tile_count) {
    const int tiles_m = (M + tile_dim - 1) / tile_dim, tiles_n = (N + tile_dim - 1) / tile_dim;
    const TileRC rc = tile_order(tiles_m, tiles_n, tile_group_m, tile_count);
    return (int64_t)rc.row * tile_dim * N + (int64_t)rc.col * tile_dim;
}

// Persistent workgroup b of a grid of G workgroups takes tile counts n*G + slot(b). Workgroups are
// dealt round-robin to the 8 XCDs (each with a private L2), so the slot puts the G/8 workgroups of
// one XCD on consecutive tile counts: under the grouped order those form one compact block of
// tiles sharing A row-panels and B column-panels in that XCD's L2.
CK_HD int xcd_slot(int block, int grid, int num_xcd) {
    if (num_xcd <= 1 || grid % num_xcd != 0) return block;
    return (block % num_xcd) * (grid / num_xcd) + block / num_xcd;
}

// ---- LDS ring layout ----------------------------------------------------------------------------
// One stage of one operand is tile_dim rows of segment_dim_k 16-bit elements, stored row-major with
// NO padding (a direct-to-LDS wave load writes 64 lanes x 16 B linearly), and the 16-byte chunks of
// each row XOR-swizzled so that the 16 lanes of one ds_read_b128 phase (16 consecutive rows, same
// logical chunk) fall into 16 distinct 4-bank groups of the 64-bank LDS.
CK_HD int chunks_per_row(int segment_dim_k) { return segment_dim_k / CHUNK_ELEMS; }
CK_HD int swizzle_key(int row, int cpr) {
    // Found conflict-free for ds_read_b128 on gfx950 by measurement (64 banks, 256 B/clk): rows of
    // 64 and 128 bytes rotate with every second row, rows of 256 bytes with every row.
    // (rows of 512 bytes: as rows of 256 - the key moves a chunk inside its 256-byte half)
    return cpr >= 16 ? row % 16 : (row >> 1) % cpr;
}
// slot (physical chunk index inside the row) that holds logical chunk c of row `row`
CK_HD int swizzle_slot(int row, int c, int cpr, int swizzle_on) { return swizzle_on ? (c ^ swizzle_key(row, cpr)) : c; }

CK_HD int stage_bytes_one_operand(int tile_dim, int segment_dim_k) { return tile_dim * segment_dim_k * 2; }

// ---- flag counters --------------------------------------------------------------------------------
// Flags are monotonically increasing uint32 counters in LDS. Per stage and per operand there is a
// set of "full" counters (producer waves add 1 when their share of the rows a counter covers has
// landed) and a set of "empty" counters (consumer waves add 1 when they have read those rows).
//   TILE : 1 unit per operand and stage
//   WAVE : bar_steps individually signalled upper-left wave-tile rows (A) / columns (B) + 1 residual
//   ACC  : per wave-tile row (A) / column (B): bar_steps individual 16-row blocks + 1 residual
CK_HD int sync_mode_of(int tile_dim, int consumer_waves, int bar_step_rows_a, int bar_step_rows_b) {
    const int wtr = wave_tile_rows(tile_dim, consumer_waves), wtc = wave_tile_cols(tile_dim, consumer_waves);
    if (bar_step_rows_a == tile_dim && bar_step_rows_b == tile_dim) return CK_SYNC_TILE;
    if (bar_step_rows_a == wtr * MFMA_M && bar_step_rows_b == wtc * MFMA_N) return CK_SYNC_WAVE;
    if (bar_step_rows_a == MFMA_M && bar_step_rows_b == MFMA_N) return CK_SYNC_ACC;
    return -1;
}
CK_HD int units_a(int mode, int consumer_waves, int bar_steps_a) {
    return mode == CK_SYNC_TILE ? 1 : mode == CK_SYNC_WAVE ? bar_steps_a + 1 : (consumer_waves / 2) * (bar_steps_a + 1);
}
CK_HD int units_b(int mode, int /*consumer_waves*/, int bar_steps_b) {
    return mode == CK_SYNC_TILE ? 1 : mode == CK_SYNC_WAVE ? bar_steps_b + 1 : 2 * (bar_steps_b + 1);
}
// counters per stage: full A, empty A, full B, empty B
CK_HD int flags_per_stage(int mode, int consumer_waves, int bar_steps_a, int bar_steps_b) {
    return 2 * units_a(mode, consumer_waves, bar_steps_a) + 2 * units_b(mode, consumer_waves, bar_steps_b);
}
CK_HD int flag_region_bytes(int mode, int consumer_waves, int bar_steps_a, int bar_steps_b, int num_stages) {
    return align_up(flags_per_stage(mode, consumer_waves, bar_steps_a, bar_steps_b) * num_stages * 4, FLAG_REGION_ALIGN);
}

// Total dynamic LDS the kernel needs: flag region + num_stages x (A stage + B stage). The D tile
// is written straight from the accumulators (no staging), so unlike the reference's
// max(size_ab, size_cd) there is no C/D term.
CK_HD int get_lds_req(int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                      int bar_step_rows_b, int num_stages, int consumer_waves) {
    const int mode = sync_mode_of(tile_dim, consumer_waves, bar_step_rows_a, bar_step_rows_b);
    if (mode < 0) return -1;
    return flag_region_bytes(mode, consumer_waves, bar_steps_a, bar_steps_b, num_stages) +
           num_stages * 2 * stage_bytes_one_operand(tile_dim, segment_dim_k);
}

// ---- parameter legality -----------------------------------------------------------------------------
struct GemmTuning {
    int tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b;
    int tile_group_m, num_stages, num_producer_waves, num_consumer_waves, num_cus;
    int port_0_rules;  // the legal set of the port_0 launcher: also one producer wave (port_0.cu:538)
};

// Largest total wave count (producers + consumers) a kernel instance is compiled for. It fixes the
// per-wave register budget: all waves of a kernel get the same allocation out of 512 per SIMD lane.
CK_HD int max_waves_for(int tile_dim, int /*consumer_waves*/) { return tile_dim == 256 ? 12 : 16; }

// Dynamic LDS of a launch. The fused variant keeps no counters in LDS: the whole allocation is ring.
CK_HD int gemm_lds_bytes(const GemmTuning& t) {
    if (t.num_producer_waves == 0) return t.num_stages * 2 * stage_bytes_one_operand(t.tile_dim, t.segment_dim_k);
    return get_lds_req(t.tile_dim, t.segment_dim_k, t.bar_steps_a, t.bar_steps_b, t.bar_step_rows_a, t.bar_step_rows_b,
                       t.num_stages, t.num_consumer_waves);
}

CK_HD int check_gemm_tuning(const GemmTuning& t) {
    if (!(t.tile_dim == 64 || t.tile_dim == 128 || t.tile_dim == 256)) return CK_ERR_BAD_PARAM;
    // the reference takes every multiple of 64 (port_2.cu:1113; port_0: of tile_dim / 2, port_0.cu:534); one MFMA eats 32 of K
    if (t.segment_dim_k < MFMA_K || t.segment_dim_k % MFMA_K != 0) return CK_ERR_BAD_PARAM;
    if (!(t.num_consumer_waves == 4 || t.num_consumer_waves == 8)) return CK_ERR_BAD_PARAM;
    // 0 producer waves: every consumer wave also streams its share of the segments (fused variant); 1: port_0 only
    if (!(t.num_producer_waves == 0 || t.num_producer_waves == 2 || t.num_producer_waves == 4 || t.num_producer_waves == 8 ||
          (t.num_producer_waves == 1 && t.port_0_rules)))
        return CK_ERR_BAD_PARAM;
    if (t.num_stages < 1 || t.num_stages > MAX_STAGES) return CK_ERR_BAD_PARAM;
    if (t.tile_group_m < 1 || t.num_cus < 1) return CK_ERR_BAD_PARAM;
    const int wtr = wave_tile_rows(t.tile_dim, t.num_consumer_waves), wtc = wave_tile_cols(t.tile_dim, t.num_consumer_waves);
    const int mode = sync_mode_of(t.tile_dim, t.num_consumer_waves, t.bar_step_rows_a, t.bar_step_rows_b);
    if (mode < 0) return CK_ERR_BAD_PARAM;
    if (mode == CK_SYNC_WAVE) {
        if (t.bar_steps_a < 0 || t.bar_steps_a > t.num_consumer_waves / 2) return CK_ERR_BAD_PARAM;
        if (t.bar_steps_b < 0 || t.bar_steps_b > 2) return CK_ERR_BAD_PARAM;
    } else if (mode == CK_SYNC_ACC) {
        if (t.bar_steps_a < 0 || t.bar_steps_a >= wtr) return CK_ERR_BAD_PARAM;
        if (t.bar_steps_b < 0 || t.bar_steps_b >= wtc) return CK_ERR_BAD_PARAM;
    }
    // no producer waves: the waves meet at the workgroup barrier (no finer granularity). Two or more stages:
    // the fused variant (a stage is refilled while the next one is multiplied); one stage: the synchronous
    // load / barrier / multiply / barrier kernel
    if (t.num_producer_waves == 0 && mode != CK_SYNC_TILE) return CK_ERR_NO_INSTANCE;
    // 64 accumulator blocks (256 registers) leave no room for a second wave on the SIMD
    if (get_num_acc(t.tile_dim, t.num_consumer_waves) > 32) return CK_ERR_NO_INSTANCE;
    if (t.num_producer_waves + t.num_consumer_waves > max_waves_for(t.tile_dim, t.num_consumer_waves)) return CK_ERR_NO_INSTANCE;
    const int64_t lds = t.segment_dim_k > 4096 ? (int64_t)LDS_BYTES_PER_CU + 1 : (int64_t)gemm_lds_bytes(t);
    if (lds > LDS_BYTES_PER_CU) return CK_ERR_LDS_BUDGET;
    // kernel instances: 32, 64 and 128 deep segments everywhere; 256 deep ones in the producer/consumer kernel on 64 and
    // 128 tiles (the depths the reference's drivers sweep, port_2.cu:1520-1564); every other legal depth has none
    const bool deep = t.segment_dim_k == 256 && t.num_producer_waves > 0 && t.tile_dim <= 128;
    if (!(t.segment_dim_k == 32 || t.segment_dim_k == 64 || t.segment_dim_k == 128 || deep)) return CK_ERR_NO_INSTANCE;
    return CK_OK;
}

// ---- matmul_shmem (SIMT) ------------------------------------------------------------------------------
// Public knobs stay tile_dim and block_rows (accumulators per thread = tile_dim / block_rows,
// matmul_shmem.cu:151-160). The accumulators of one thread form a 2-D micro-tile rm x rn.
struct MicroTile { int rm, rn; };
CK_HD MicroTile simt_micro_tile(int accs) {
    MicroTile m{0, 0};
    switch (accs) {
        case 1: m = {1, 1}; break;
        case 2: m = {2, 1}; break;
        case 4: m = {2, 2}; break;
        case 8: m = {4, 2}; break;
        case 16: m = {4, 4}; break;
        case 32: m = {8, 4}; break;
        case 64: m = {8, 8}; break;
        default: break;
    }
    return m;
}
// Row pitch of the k-major LDS slices beyond tile_dim. (Pitches of tile_dim + 8, 12, 16, 20 and 36 measured the same as
// this one on fp32 4096^3, 90 to 93 TFLOP/s: the two-dword LDS writes of a fetched chunk collide in half of the banks at
// every one of them, and cost nothing that shows - the kernel is bound by the vector ALUs' clock under load.)
constexpr int SIMT_PAD = 4;
constexpr int SIMT_KT = 16;  // K depth of one LDS tile of the SIMT kernel
CK_HD int simt_lds_req(int tile_dim, int elem_bytes) {
    // two operands x two buffers x KT x (tile_dim + pad) elements
    return 2 * 2 * SIMT_KT * (tile_dim + SIMT_PAD) * elem_bytes;
}
CK_HD int check_simt_tuning(int tile_dim, int block_rows) {
    if (!(tile_dim == 32 || tile_dim == 64 || tile_dim == 128)) return CK_ERR_BAD_PARAM;
    if (block_rows < 1 || tile_dim % block_rows) return CK_ERR_BAD_PARAM;
    const int accs = tile_dim / block_rows;
    if (simt_micro_tile(accs).rm == 0) return CK_ERR_BAD_PARAM;
    const int threads = tile_dim * block_rows;
    if (threads > 1024 || threads < 64) return CK_ERR_NO_INSTANCE;
    return CK_OK;
}

}  // namespace ck
#endif  // CK_COMMON_H

/* C ABI of the MI355X (gfx950) GEMM hot path: the drop-in boundary.
 *
 * The reference has no FFI; its boundary is one C++ host launcher template per translation unit.
 * Each entry point below replaces one of those launchers and keeps its parameter order and
 * meaning. Differences that hold for every entry point:
 *   - element types are selected by an int (CKOPT_DT_*) instead of template arguments;
 *   - the return value is 0 or a negative CKOPT_ERR_* code where the reference asserts or swallows
 *     the error (matmul_shmem_tc_async_opt_port_2.cu:76-85, :1112-1123);
 *   - a trailing `stream` (a hipStream_t passed as void*, NULL = default stream) is added;
 *   - "warps" are 64-lane wavefronts and "SMs" are compute units.
 * All pointers are device memory owned by the caller. Nothing is synchronised; launches are asynchronous on `stream`.
 * Device memory beyond the operands is needed in two cases only (zero-padded operand copies when K % 8 != 0 or an
 * operand is off a 16-byte boundary; partial planes when the straight-line kernel cuts K into slices). The reference's
 * launcher needs none and allocates nothing (port_2.cu:1088-1168; its drivers own all memory, :1200-1203). Here the
 * plain entry points take it from stream-ordered allocations on `stream`, out of a memory pool the library keeps per
 * device (freed blocks stay in the pool for the next launch; ckopt_trim_scratch_pool hands them back);
 * ckopt_gemm_shmem_tc_async_opt_port_2_ws takes it from a workspace the caller owns and allocates nothing;
 * ckopt_gemm_shmem_tc_async_opt_port_2_noalloc takes it from a static array inside the library.
 */
#ifndef CKOPT_H
#define CKOPT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { CKOPT_DT_F16 = 0, CKOPT_DT_BF16 = 1, CKOPT_DT_F32 = 2, CKOPT_DT_I32 = 3 };

enum {
    CKOPT_OK = 0,
    CKOPT_ERR_BAD_PARAM = -1,   /* tuning or shape parameter outside the legal set */
    CKOPT_ERR_LDS_BUDGET = -2,  /* ring does not fit 160 KiB of LDS */
    CKOPT_ERR_NO_INSTANCE = -3, /* legal, but no kernel instance is compiled for the tuple */
    CKOPT_ERR_HIP = -4,         /* a HIP runtime call failed */
    CKOPT_ERR_ALIGNMENT = -5,   /* pointer or row pitch not aligned as required */
    CKOPT_ERR_NULL = -6,        /* required pointer is NULL */
    CKOPT_ERR_TOO_LARGE = -7    /* size beyond what the entry point supports */
};

/* Replaces gemm_shmem_tc_async_opt_port<DT,DT_ACC>() of matmul_shmem_tc_async_opt_port_2.cu:1088-1168.
 * D = alpha * A * Bt^T + beta * C (textbook form; C is not read when beta == 0).
 * A: M x K row-major, Bt: N x K row-major (B transposed), dtype CKOPT_DT_F16 or CKOPT_DT_BF16;
 * C, D: M x N row-major fp32, distinct buffers (C may be NULL when beta == 0).
 * tile_dim in {64,128,256}; segment_dim_k a multiple of 32 (the reference: of 64, port_2.cu:1113; port_0: of tile_dim / 2,
 * port_0.cu:534), with kernel instances for 32, 64, 128 and - producer/consumer kernels on 64 and 128 tiles - 256; any other
 * multiple is CKOPT_ERR_NO_INSTANCE (or CKOPT_ERR_LDS_BUDGET when one stage of it exceeds the LDS); bar_step_rows_{a,b} select the
 * synchronisation granularity exactly as in the reference: (tile_dim, tile_dim), or
 * (wave_tile_rows*16, wave_tile_cols*16) with bar_steps_a <= C/2 and bar_steps_b <= 2, or (16, 16)
 * with bar_steps_a < wave_tile_rows and bar_steps_b < wave_tile_cols; num_producer_waves in
 * {2,4,8} (half stream A, half stream Bt) or 0 (no dedicated producers: every consumer wave also
 * streams its share of each segment and the waves meet at the workgroup barrier once per segment;
 * tile granularity only; with num_stages 1 nothing overlaps: load, barrier, multiply, barrier, the schedule of the
 * reference's first tensor-core kernel, matmul_shmem_tc.cu:105-231); num_consumer_waves in {4,8}; num_cus = persistent grid.
 * M, N need not be multiples of tile_dim and K need not be a multiple of segment_dim_k (edges are
 * zero-filled / masked). The kernels read operand rows that start on 16-byte boundaries: when K is
 * not a multiple of 8, or A / Bt is not 16-byte aligned (2-byte alignment is required), the call first copies both
 * operands into zero-padded rows in a stream-ordered temporary (hipMallocAsync / hipFreeAsync on `stream`,
 * (M + N) * Kp * 2 bytes with Kp = round_up(K, 8), or round_up(K, 64) for the tuple tile_dim 256, segment_dim_k 32,
 * num_stages 5, no producer waves, whose straight-line kernel works in loop bodies of 64). */
int ckopt_gemm_shmem_tc_async_opt_port_2(int dtype, const void* A, const void* Bt, const float* C, float* D,
                                         float alpha, float beta, int M, int N, int K, int tile_dim,
                                         int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                                         int bar_step_rows_b, int tile_group_m, int num_stages,
                                         int num_producer_waves, int num_consumer_waves, int num_cus, void* stream);

/* The <half, half> role of the same launcher (the reference instantiates DT_ACC = half next to float,
 * matmul_shmem_tc_async_opt_port_2.cu:968-1055): C and D hold the operands' 16-bit element type (fp16 for
 * CKOPT_DT_F16, bf16 for CKOPT_DT_BF16; 2-byte aligned). Accumulation stays fp32; alpha * A * Bt^T + beta * C
 * is rounded to nearest even once, so the result is at least as accurate as a 16-bit accumulator's. */
int ckopt_gemm_shmem_tc_async_opt_port_2_lp(int dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim,
                                            int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                                            int bar_step_rows_b, int tile_group_m, int num_stages,
                                            int num_producer_waves, int num_consumer_waves, int num_cus, void* stream);

/* The port_2 launcher (both C / D forms) on caller-owned scratch memory: the reference's ownership rule (the launcher
 * works on the caller's device memory only, port_2.cu:1088-1168, :1200-1203) for the launches that need memory beyond
 * the operands. cd_dtype is CKOPT_DT_F32 (the port_2 entry) or equal to dtype (the _lp entry). `workspace` is device
 * memory of `workspace_bytes` bytes, any alignment, used only during the call's work on `stream`; it may be NULL when
 * the launch needs none. ckopt_gemm_workspace_bytes returns how much the launch with these sizes and this tuning
 * needs under the process's current options (0: none; negative: the error the launch would give);
 * operands_aligned != 0 promises A and Bt on 16-byte boundaries. A workspace that is too small gives
 * CKOPT_ERR_TOO_LARGE and D is not written; nothing is allocated in any case. */
int64_t ckopt_gemm_workspace_bytes(int M, int N, int K, int operands_aligned, int tile_dim, int segment_dim_k, int bar_steps_a,
                                   int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                                   int num_producer_waves, int num_consumer_waves, int num_cus);

/* What a launch with these sizes and this tuning will run under the process's current options, without launching:
 * plan_out[0] = 1 if it takes the straight-line kernel (gemm_stream_kernel), 0 for the other designs;
 * plan_out[1] = width of its tiles in columns of D (256 or 128 for the straight-line kernel, else tile_dim);
 * plan_out[2] = number of K slices (1: no split-K); plan_out[3] = 1 if A and Bt are first copied into zero-padded rows;
 * plan_out[4] = number of tiles that are cut into those slices (all of them when there are fewer tiles than num_cus; the
 * tiles of the partly filled last round otherwise; 0 without slices); plan_out[5] = 1 if the slices are added inside the
 * kernel, 0 if by a second kernel; plan_out[6] = workgroups of the straight-line kernel's grid. plan_out points at 7 ints.
 * Returns CKOPT_OK or the error the launch would give. No reference counterpart (its launcher has one kernel form). */
int ckopt_gemm_launch_plan(int M, int N, int K, int operands_aligned, int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b,
                           int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages, int num_producer_waves,
                           int num_consumer_waves, int num_cus, int* plan_out);
int ckopt_gemm_shmem_tc_async_opt_port_2_ws(int dtype, int cd_dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim, int segment_dim_k,
                                            int bar_steps_a, int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b,
                                            int tile_group_m, int num_stages, int num_producer_waves, int num_consumer_waves,
                                            int num_cus, void* workspace, size_t workspace_bytes, void* stream);

/* The port_2 launcher above for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference, whose launcher needs no
 * memory beyond its operands. Same parameters and results as ckopt_gemm_shmem_tc_async_opt_port_2 (the same kernels
 * in the same order), but the zero-padded operand copies (K % 8 != 0 or operands off a 16-byte boundary:
 * (M + N) * round_up(K, 8 or 64) * 2 bytes) and the split-K planes (slices * M * N * 4 bytes) live in a static device array
 * of CKOPT_NOALLOC_SCRATCH_BYTES inside the library instead of stream-ordered allocations: no hipMalloc, hipFree or
 * allocating library routine is called. A launch that needs more than the array holds (both pieces, each rounded up
 * to 256 bytes) returns CKOPT_ERR_TOO_LARGE and D is not written; ckopt_set_option(7, 0) makes such a launch
 * fit by not cutting K. Every device holds one array and every call on a device uses it: calls that overlap on one
 * device (different streams, different threads) race on it. Nothing in it needs to start at zero (the counters of
 * a reduction inside the kernel are cleared by a small kernel of the same launch, not by a memset).
 * Before a launch is recorded into a HIP graph, one eager call with the same element type, shape class (K a
 * multiple of 64 or not, the tile width the plan query reports) and options must have run on the device: the first
 * call on a device resolves the array's address and the first use of each kernel instance sets its LDS-size
 * attribute, neither of which may happen under capture. The array is resident on every device the process uses the
 * library on, whether or not this entry point is ever called. */
#define CKOPT_NOALLOC_SCRATCH_BYTES (64u << 20)
int ckopt_gemm_shmem_tc_async_opt_port_2_noalloc(int dtype, const void* A, const void* Bt, const float* C, float* D,
                                                 float alpha, float beta, int M, int N, int K, int tile_dim,
                                                 int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                                                 int bar_step_rows_b, int tile_group_m, int num_stages,
                                                 int num_producer_waves, int num_consumer_waves, int num_cus, void* stream);

/* Launch options as a per-call argument. In the reference every knob is a launcher parameter (port_2.cu:1088-1109);
 * the knobs this implementation adds (kernel form, tile width, K slices, store policy, ...) are one struct here, so
 * that a size query and the launch that follows it see the same values whatever other threads do, and two threads can
 * launch with different settings at the same time. Each field has the meaning and range of the ckopt_set_option key
 * named beside it; ckopt_launch_options_init fills the struct with the process-wide defaults (what ckopt_set_option
 * last set), which are also what every entry point without an options argument uses - read once, at its start. */
typedef struct ckopt_launch_options {
    int struct_bytes;         /* sizeof(ckopt_launch_options): set by ckopt_launch_options_init, checked by the callee */
    int lds_swizzle;          /* key 0 */
    int spin_limit;           /* key 1 */
    int num_xcd;              /* key 2 */
    int prio_mode;            /* key 3 */
    int producer_nap;         /* key 4 */
    int tile_sync_barrier;    /* key 5 */
    int straight_line;        /* key 6 */
    int split_k;              /* key 7 */
    int barrier_every_kstep;  /* key 8 */
    int even_rounds;          /* key 9 */
    int d_store_policy;       /* key 10 */
    int half_width;           /* key 11 */
    int tail_round;           /* key 12 */
    int fused_reduction;      /* key 13 */
    int batched_empty_reads;  /* key 14 */
} ckopt_launch_options;
int ckopt_launch_options_init(ckopt_launch_options* options);

/* The port_2 launcher (both C / D forms: cd_dtype CKOPT_DT_F32 or equal to dtype) with its options as an argument.
 * options == NULL: the process-wide defaults. workspace == NULL: memory beyond the operands comes from stream-ordered
 * allocations, as in ckopt_gemm_shmem_tc_async_opt_port_2; otherwise from [workspace, workspace + workspace_bytes), as
 * in the _ws entry point, and nothing is allocated. ckopt_gemm_workspace_bytes_ex and ckopt_gemm_launch_plan_ex are
 * the queries for the same arguments: query and launch are pure functions of what they are given (plus the device's
 * compute-unit count, which the cost model reads once per device). No reference counterpart beyond port_2.cu:1088-1109. */
int ckopt_gemm_shmem_tc_async_opt_port_2_ex(int dtype, int cd_dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim, int segment_dim_k,
                                            int bar_steps_a, int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b,
                                            int tile_group_m, int num_stages, int num_producer_waves, int num_consumer_waves,
                                            int num_cus, const ckopt_launch_options* options, void* workspace,
                                            size_t workspace_bytes, void* stream);
int64_t ckopt_gemm_workspace_bytes_ex(int M, int N, int K, int operands_aligned, int tile_dim, int segment_dim_k, int bar_steps_a,
                                      int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                                      int num_producer_waves, int num_consumer_waves, int num_cus,
                                      const ckopt_launch_options* options);
int ckopt_gemm_launch_plan_ex(int M, int N, int K, int operands_aligned, int tile_dim, int segment_dim_k, int bar_steps_a,
                              int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                              int num_producer_waves, int num_consumer_waves, int num_cus, const ckopt_launch_options* options,
                              int* plan_out);

/* Replaces gemm_shmem_tc_async_opt_port<DT,DT_ACC>() of matmul_shmem_tc_async_opt_port_1.cu:889-965:
 * every wave tile (or every 16-row block) has its own signal, i.e. port_2 with maximal bar_steps. */
int ckopt_gemm_shmem_tc_async_opt_port_1(int dtype, const void* A, const void* Bt, const float* C, float* D,
                                         float alpha, float beta, int M, int N, int K, int tile_dim,
                                         int segment_dim_k, int bar_step_rows_a, int bar_step_rows_b,
                                         int tile_group_m, int num_stages, int num_producer_waves,
                                         int num_consumer_waves, int num_cus, void* stream);
/* Its <half, half> instance (port_1.cu:1292, :1332): C and D in the operands' 16-bit type, as in the _2_lp entry point. */
int ckopt_gemm_shmem_tc_async_opt_port_1_lp(int dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim,
                                            int segment_dim_k, int bar_step_rows_a, int bar_step_rows_b,
                                            int tile_group_m, int num_stages, int num_producer_waves,
                                            int num_consumer_waves, int num_cus, void* stream);

/* Replaces gemm_shmem_tc_async_opt_port<DT,DT_ACC>() of matmul_shmem_tc_async_opt_port_0.cu:515-579:
 * one full/empty signal pair per operand and stage. num_producer_waves may also be 1 (port_0.cu:538): the one wave
 * streams the A rows and then the Bt rows of every segment (port_0.cu:106-147). */
int ckopt_gemm_shmem_tc_async_opt_port_0(int dtype, const void* A, const void* Bt, const float* C, float* D,
                                         float alpha, float beta, int M, int N, int K, int tile_dim,
                                         int segment_dim_k, int tile_group_m, int num_stages,
                                         int num_producer_waves, int num_consumer_waves, int num_cus, void* stream);
/* Its <half, half> instance (port_0.cu:866, :906). */
int ckopt_gemm_shmem_tc_async_opt_port_0_lp(int dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim,
                                            int segment_dim_k, int tile_group_m, int num_stages,
                                            int num_producer_waves, int num_consumer_waves, int num_cus, void* stream);

/* Role of get_shmem_req<DT,DT_ACC>() (port_2.cu:1057-1086): dynamic LDS bytes of the launch, or a
 * negative error code. The caller may compare it with 160 KiB; the launcher does so itself. */
int ckopt_get_lds_req(int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                      int bar_step_rows_b, int num_stages, int num_consumer_waves);

/* get_num_acc / get_warp_tile_rows (port_2.cu:158-169), extended to tile_dim 256. */
int ckopt_get_num_acc(int tile_dim, int num_consumer_waves);
int ckopt_get_warp_tile_rows(int tile_dim, int num_consumer_waves);

/* get_tile_offset_cd (port_2.cu:605-614) with 64-bit offsets and ceil-divided tile counts. */
int64_t ckopt_get_tile_offset_cd(int M, int N, int tile_dim, int tile_group_m, int64_t tile_count);

/* Validates a port_2 tuning tuple without launching (the reference's asserts, port_2.cu:1112-1123,
 * plus the LDS budget and the instance table). Returns CKOPT_OK or the error the launch would give. */
int ckopt_check_gemm_tuning(int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b,
                            int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                            int num_producer_waves, int num_consumer_waves, int num_cus);

/* A tuning tuple for a problem size, from the measurements on MI355X (no counterpart in the reference, whose
 * drivers sweep the tuples by hand, port_2.cu:1463-1480): tuning_out receives {tile_dim, segment_dim_k,
 * bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
 * num_consumer_warps} in the launcher's parameter order. Enough 256 x 256 tiles for half the CUs (or a K deep
 * enough to be cut into at least four slices): the straight-line kernel's tuple; else 128 x 128 tiles if those
 * occupy half the CUs; else 64 x 64 tiles. */
int ckopt_suggest_gemm_tuning(int M, int N, int K, int num_cus, int* tuning_out);

/* Replaces matmul_shmem<DT,DT_ACC>() of matmul_shmem.cu:143-174: C = A * B without matrix cores.
 * dtype CKOPT_DT_F32 (fp32 in, fp32 accumulate), CKOPT_DT_F16 (fp16 in/out, fp32 accumulate) or
 * CKOPT_DT_I32 (exact). A: M x K, C: M x N row-major. b_transposed == 0: B is K x N row-major as in
 * the reference; b_transposed != 0: B is given as N x K row-major.
 * tile_dim in {32,64,128}, tile_dim % block_rows == 0, accumulators per thread
 * tile_dim/block_rows in {1,2,4,8,16,32,64}, 64 <= tile_dim*block_rows <= 1024.
 * M, N must be multiples of tile_dim and K a multiple of 16. */
int ckopt_matmul_shmem(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int tile_dim,
                       int block_rows, int b_transposed, void* stream);

/* Role of get_shmem_req<DT>(tile_dim) (matmul_shmem.cu:138-141). */
int ckopt_matmul_shmem_lds_req(int dtype, int tile_dim);
int ckopt_check_matmul_shmem_tuning(int tile_dim, int block_rows);

/* Releases what the library's stream-ordered scratch pool of the current device holds beyond keep_bytes (0: everything
 * that is not in use). The pool keeps the largest scratch a launch of the allocating entry points has used on the device,
 * so that the next launch does not pay for a fresh allocation. No reference counterpart. */
int ckopt_trim_scratch_pool(size_t keep_bytes);

/* Waits for `stream`, then returns the device status word of the current device and clears it:
 * 0 = all flag waits inside the GEMM kernels completed; bit 0 / bit 1 = a producer / consumer wave
 * gave up a bounded wait (results are then invalid). Negative = HIP error. No reference counterpart
 * (cuda::barrier waits are unbounded). */
int ckopt_device_status(void* stream);

/* Waits for `stream`, then reports how long workgroup 0 of the last GEMM launch on the current device
 * ran: shader-clock cycles and ticks of the constant 100 MHz reference clock. Their ratio is the clock
 * the compute units actually ran at (it drops under matrix-core load), which turns a duration into a
 * matrix-core utilisation. No reference counterpart. */
int ckopt_last_launch_clocks(void* stream, uint64_t* shader_cycles, uint64_t* ref_ticks);

/* Process-wide defaults of the tuning switches that are not launcher parameters in the reference (ckopt_launch_options
 * carries the same switches per call). An entry point without an options argument reads all of them once, when it
 * starts: a switch changed by one thread while another launches takes effect for all or none of that launch. Two
 * threads that need different settings at the same time use the _ex entry points.
 * key 0: LDS XOR swizzle on/off (default 1); key 1: spin limit of bounded waits (default 1<<22);
 * key 2: number of XCDs assumed by the workgroup->tile remap (default 8; 1 disables the remap);
 * key 3: wave priorities of the counter-synchronised kernel (0 producers raised (default), 1 also asymmetric
 *        consumer bursts per SIMD pair, 2 none); key 4: producers' polling nap (0, 1, 2 = s_sleep 1, 4, 16);
 * key 5: tile granularity with dedicated producers synchronises through the hardware workgroup barrier
 *        (gemm_pcb_kernel, needs num_stages >= 2) instead of LDS counters (default 0).
 * key 6: launches with num_producer_warps 0, tile_dim 256, segment_dim_k 32, num_stages 5, 8 consumer warps (any M, N, K)
 *        take the straight-line kernel written for exactly that shape (gemm_stream_kernel; default 1); 0 sends them
 *        through the general fused kernel.
 * key 7: split-K of the straight-line kernel. 1 (default): with fewer tiles than num_sms, K is cut into the number of
 *        slices (at most 16, each a multiple of 64 and at least 1024 deep) for which a cost model of the device gives
 *        the shortest time - loop bodies at the rate the active CUs sustain, the store burst of every round, the
 *        reduction pass (e.g. 64 tiles, K 32768: 4 slices; 128 tiles, K 16384: 2; 128 tiles, K 4096: none); the
 *        slices' partial products go to scratch memory (slices * M * N * 4 bytes) and a second kernel adds them in
 *        slice order and applies alpha, beta and the output type. 0: never. 2..16: that many slices whenever legal.
 * key 8: schedule of the straight-line kernel. 1 (default): a workgroup barrier in every k-step, the loads of a loop
 *        body spread over both (three k-steps to land); 0: one barrier per two k-steps, all loads behind it (two
 *        k-steps to land) - at 8192^3 on random operand values 1.5 % faster on one device and 0.7 % slower on another,
 *        slower wherever memory latency is higher (16384^3: 7 %, split-K: 6 to 12 %) or the clock is free (3 %).
 * key 9: even rounds (default 1). A launch with more tiles than num_sms runs ceil(tiles / num_sms) rounds; with 1 the
 *        persistent grid is the smallest number of workgroups (a multiple of the XCD count, at most num_sms) that
 *        needs no more rounds, so that no round is partly empty (408 tiles on 256 CUs: 208 workgroups x 2 rounds
 *        instead of 256 + 152; 5.7 % faster where the clock is power-limited); 0: always min(tiles, num_sms).
 * key 10: how the GEMM kernels store D. 0 (default): non-temporal vector stores where every row of D starts on a 128-byte
 *        line (D on a 128-byte boundary and N * element size a multiple of 128), ordinary stores otherwise: rows that
 *        start anywhere make every 128-byte run of a row straddle two lines, and only ordinary stores let the parts
 *        meet in L2 before they reach memory (bf16 6143 x 4097 x 3072: 138 us against 164). 1: always non-temporal;
 *        2: never.
 * key 11: tile width of the straight-line kernel. 1 (default): 256 x 192 tiles (wave tiles of 64 x 96, 0.88 of the rate of
 *        256 x 256 tiles on a full device) or 256 x 128 tiles (wave tiles of 64 x 64, 0.86) where the launcher's cost model
 *        gives them at least 5 % less time than 256 x 256 tiles - tile counts that fill the last round badly or leave
 *        much of the device idle (6144^3: 576 tiles in 2.25 rounds -> 768 tiles of 256 x 192 in exactly 3, 395 us ->
 *        362 us; 3072^3: 65 us -> 57 us; 2560^3: 100 tiles, 53 us -> 37 us with 200 tiles of 256 x 128);
 *        0: always 256 x 256; 2: always 256 x 128; 3: always 256 x 192. tile_dim stays 256 in the launcher's parameters.
 * key 12: the partly filled last round of the straight-line kernel (default 1). With more tiles than num_sms the last
 *        round leaves CUs idle (6144^3: 576 tiles = 2 x 256 + 64); with 1 its tiles are cut into 2 to 4 K slices that
 *        run as work items of the same launch behind the whole tiles, where the cost model gives that at least 3 % less
 *        time than evenly filled rounds of whole tiles (key 9); needs key 7 at 1 and key 13 not 0. 0: never.
 * key 13: where K slices are added. Inside the straight-line kernel: every slice's wave stores its partial sums of a
 *        wave tile to scratch memory (slices x tile bytes and 1 KiB of counters per cut tile) and counts itself on the
 *        wave tile's counter; the wave that finds itself the last adds the partials in slice order - the same order
 *        whichever comes last, so the result is deterministic and equal to the second kernel's bit for bit - and writes
 *        D; no second kernel, and no wave waits for another (launches may overlap with anything). Or by a second
 *        kernel over slices x M x N x 4 bytes of planes. 1 (default): inside the kernel where the cost model gives it
 *        less time (measured: two slices of 128 tiles 27 us against 22 for the second kernel, four of 64 tiles 47
 *        against 19 - the last wave's chain of memory round trips - so on a 256-CU device the second kernel is what
 *        runs); 2: always inside the kernel; 0: never.
 * key 14: wave-tile granularity of the counter-synchronised kernel (default 1). 1: a producer wave reads all "released"
 *        counters of its operand and stage in one look per segment and polls a row block's counter only if that look
 *        found it short; 0: it polls every row block's counter on its own, as the reference's producers wait on every
 *        barrier in turn (port_2.cu:212-232).
 * Returns the previous value or CKOPT_ERR_BAD_PARAM. */
int ckopt_set_option(int key, int value);

/* Seeded host-side input generation (role of MatmulTest*::Rerand / SetConstant, matmul_test.h:160-168,
 * :328-351). Element i of stream `stream_id` depends only on (seed, stream_id, i): value i is the
 * (i+1)-th output of SplitMix64 started at seed + stream_id * 0xD1342543DE82EF95, reduced to a
 * 24-bit uniform in [0,1). `out` is HOST memory of n elements of `dtype`. */
int ckopt_fill_uniform(int dtype, void* out, int64_t n, uint64_t seed, uint64_t stream_id, float lo, float hi);
int ckopt_fill_normal(int dtype, void* out, int64_t n, uint64_t seed, uint64_t stream_id, float mean, float stddev);
int ckopt_fill_int(int dtype, void* out, int64_t n, uint64_t seed, uint64_t stream_id, int lo, int hi_inclusive);
int ckopt_fill_constant(int dtype, void* out, int64_t n, float value);

const char* ckopt_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* CKOPT_H */

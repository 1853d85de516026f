// C++ face of libckopt.so: the reference's launcher templates, same names and parameter order, as thin
// wrappers over the C ABI of ckopt.h. A failed call throws ckopt::Error where the reference asserts.
//
//   gemm_shmem_tc_async_opt_port<DT,DT_ACC>   matmul_shmem_tc_async_opt_port_2.cu:1088-1109 (port_1:889-908 and
//                                             port_0:515-532 are the overloads with fewer parameters)
//   matmul_shmem<DT,DT_ACC>                   matmul_shmem.cu:143-152
//   get_shmem_req<DT,DT_ACC>                  port_2.cu:1057-1066        get_num_acc / get_warp_tile_rows  :158-169
//   get_shmem_req<DT>(tile_dim)               matmul_shmem.cu:138-141
//
// DT is one of ckopt::half_t (IEEE fp16; layout-compatible with __half), ckopt::bfloat16_t, float, int;
// DT_ACC is float (GEMM) or equals DT (matmul_shmem). Pointers are device memory owned by the caller.
#ifndef CKOPT_HPP
#define CKOPT_HPP

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "ckopt.h"

namespace ckopt {

using half_t = _Float16;
struct bfloat16_t { std::uint16_t bits; };

struct Error : std::runtime_error {
    int code;
    Error(int c, const char* where) : std::runtime_error(std::string(where) + ": " + ckopt_error_string(c)), code(c) {}
};
inline void check(int rc, const char* where) { if (rc != CKOPT_OK) throw Error(rc, where); }

// The kernels' flag waits are bounded: a wave that gives one up sets a status bit and the launch's D is then invalid
// (cuda::barrier waits in the reference are unbounded and would hang instead). The launcher templates below do not
// synchronise, so they cannot report it; a caller that wants the check calls this after its launches: it waits for
// `stream`, reads and clears the device's status word and throws if a wait was given up.
struct DeviceStatusError : std::runtime_error {
    int status;
    explicit DeviceStatusError(int s)
        : std::runtime_error("a bounded flag wait was given up (device status " + std::to_string(s) + "): results are invalid"), status(s) {}
};
inline void synchronize_and_check(void* stream = nullptr) {
    const int st = ckopt_device_status(stream);
    if (st < 0) throw Error(st, "device_status");
    if (st != 0) throw DeviceStatusError(st);
}

// A launcher call followed by that check, for callers that want the reference's blocking behaviour (its drivers
// synchronise right behind every launch, port_2.cu:1241-1242) together with an error instead of a silently wrong D:
//     ckopt::checked(stream, [&] { ckopt::gemm_shmem_tc_async_opt_port<DT, float>(A, B, C, D, ...); });
template <typename Launch>
inline void checked(void* stream, Launch&& launch) {
    launch();
    synchronize_and_check(stream);
}

inline float to_float(float x) { return x; }
inline float to_float(half_t x) { return (float)x; }
inline float to_float(bfloat16_t x) {
    const std::uint32_t u = (std::uint32_t)x.bits << 16;
    float f;
    static_assert(sizeof f == sizeof u, "");
    __builtin_memcpy(&f, &u, sizeof f);
    return f;
}

template <typename DT> struct dtype_of;
template <> struct dtype_of<half_t> { static constexpr int value = CKOPT_DT_F16; };
template <> struct dtype_of<bfloat16_t> { static constexpr int value = CKOPT_DT_BF16; };
template <> struct dtype_of<float> { static constexpr int value = CKOPT_DT_F32; };
template <> struct dtype_of<int> { static constexpr int value = CKOPT_DT_I32; };

// port_2: individually signalled upper-left units (bar_steps) + granularity (bar_step_rows)
template <typename DT, typename DT_ACC>
void gemm_shmem_tc_async_opt_port(const DT* A, const DT* B /* transposed: N x K */, const DT_ACC* C, DT_ACC* D, DT_ACC alpha,
                                  DT_ACC beta, int M, int N, int K, int tile_dim, int segment_dim_k, int bar_steps_a,
                                  int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                                  int num_producer_warps, int num_consumer_warps, int num_sms, void* stream = nullptr) {
    static_assert(std::is_same<DT_ACC, float>::value || std::is_same<DT_ACC, DT>::value, "C / D are fp32 or the operand type");
    if constexpr (std::is_same<DT_ACC, float>::value) {
        check(ckopt_gemm_shmem_tc_async_opt_port_2(dtype_of<DT>::value, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k,
                                                   bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m,
                                                   num_stages, num_producer_warps, num_consumer_warps, num_sms, stream),
              "gemm_shmem_tc_async_opt_port");
    } else {  // the <half, half> instance: 16-bit C and D, alpha / beta given in that type
        check(ckopt_gemm_shmem_tc_async_opt_port_2_lp(dtype_of<DT>::value, A, B, C, D, to_float(alpha), to_float(beta), M, N, K,
                                                      tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
                                                      bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
                                                      num_consumer_warps, num_sms, stream),
              "gemm_shmem_tc_async_opt_port <DT, DT>");
    }
}
// port_2 on caller-owned scratch memory (ckopt_gemm_workspace_bytes says how much): nothing is allocated
template <typename DT, typename DT_ACC>
void gemm_shmem_tc_async_opt_port(const DT* A, const DT* B, const DT_ACC* C, DT_ACC* D, DT_ACC alpha, DT_ACC beta, int M, int N, int K,
                                  int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                                  int bar_step_rows_b, int tile_group_m, int num_stages, int num_producer_warps, int num_consumer_warps,
                                  int num_sms, void* workspace, std::size_t workspace_bytes, void* stream) {
    static_assert(std::is_same<DT_ACC, float>::value || std::is_same<DT_ACC, DT>::value, "C / D are fp32 or the operand type");
    check(ckopt_gemm_shmem_tc_async_opt_port_2_ws(dtype_of<DT>::value, dtype_of<DT_ACC>::value, A, B, C, D, to_float(alpha), to_float(beta), M, N,
                                                  K, tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b,
                                                  tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, workspace,
                                                  workspace_bytes, stream),
          "gemm_shmem_tc_async_opt_port (workspace)");
}
// port_1: granularity only
template <typename DT, typename DT_ACC>
void gemm_shmem_tc_async_opt_port(const DT* A, const DT* B, const DT_ACC* C, DT_ACC* D, DT_ACC alpha, DT_ACC beta, int M, int N,
                                  int K, int tile_dim, int segment_dim_k, int bar_step_rows_a, int bar_step_rows_b,
                                  int tile_group_m, int num_stages, int num_producer_warps, int num_consumer_warps, int num_sms,
                                  void* stream = nullptr) {
    static_assert(std::is_same<DT_ACC, float>::value || std::is_same<DT_ACC, DT>::value, "C / D are fp32 or the operand type");
    if constexpr (std::is_same<DT_ACC, float>::value) {
        check(ckopt_gemm_shmem_tc_async_opt_port_1(dtype_of<DT>::value, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k,
                                                   bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages, num_producer_warps,
                                                   num_consumer_warps, num_sms, stream),
              "gemm_shmem_tc_async_opt_port (port_1)");
    } else {  // the <half, half> instance (port_1.cu:1292, :1332)
        check(ckopt_gemm_shmem_tc_async_opt_port_1_lp(dtype_of<DT>::value, A, B, C, D, to_float(alpha), to_float(beta), M, N, K, tile_dim,
                                                      segment_dim_k, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
                                                      num_producer_warps, num_consumer_warps, num_sms, stream),
              "gemm_shmem_tc_async_opt_port (port_1) <DT, DT>");
    }
}
// port_0: one signal pair per stage
template <typename DT, typename DT_ACC>
void gemm_shmem_tc_async_opt_port(const DT* A, const DT* B, const DT_ACC* C, DT_ACC* D, DT_ACC alpha, DT_ACC beta, int M, int N,
                                  int K, int tile_dim, int segment_dim_k, int tile_group_m, int num_stages,
                                  int num_producer_warps, int num_consumer_warps, int num_sms, void* stream = nullptr) {
    static_assert(std::is_same<DT_ACC, float>::value || std::is_same<DT_ACC, DT>::value, "C / D are fp32 or the operand type");
    if constexpr (std::is_same<DT_ACC, float>::value) {
        check(ckopt_gemm_shmem_tc_async_opt_port_0(dtype_of<DT>::value, A, B, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k,
                                                   tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, stream),
              "gemm_shmem_tc_async_opt_port (port_0)");
    } else {  // the <half, half> instance (port_0.cu:866, :906)
        check(ckopt_gemm_shmem_tc_async_opt_port_0_lp(dtype_of<DT>::value, A, B, C, D, to_float(alpha), to_float(beta), M, N, K, tile_dim,
                                                      segment_dim_k, tile_group_m, num_stages, num_producer_warps, num_consumer_warps,
                                                      num_sms, stream),
              "gemm_shmem_tc_async_opt_port (port_0) <DT, DT>");
    }
}
// port_2 with the launch options as an argument (ckopt_launch_options; nullptr: the process-wide defaults) and, optionally,
// caller-owned scratch memory (nullptr: stream-ordered allocations)
template <typename DT, typename DT_ACC>
void gemm_shmem_tc_async_opt_port(const DT* A, const DT* B, const DT_ACC* C, DT_ACC* D, DT_ACC alpha, DT_ACC beta, int M, int N, int K,
                                  int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                                  int bar_step_rows_b, int tile_group_m, int num_stages, int num_producer_warps, int num_consumer_warps,
                                  int num_sms, const ckopt_launch_options* options, void* workspace, std::size_t workspace_bytes,
                                  void* stream) {
    static_assert(std::is_same<DT_ACC, float>::value || std::is_same<DT_ACC, DT>::value, "C / D are fp32 or the operand type");
    check(ckopt_gemm_shmem_tc_async_opt_port_2_ex(dtype_of<DT>::value, dtype_of<DT_ACC>::value, A, B, C, D, to_float(alpha), to_float(beta), M, N,
                                                  K, tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b,
                                                  tile_group_m, num_stages, num_producer_warps, num_consumer_warps, num_sms, options,
                                                  workspace, workspace_bytes, stream),
          "gemm_shmem_tc_async_opt_port (options)");
}
inline ckopt_launch_options default_launch_options() {
    ckopt_launch_options o;
    check(ckopt_launch_options_init(&o), "launch_options_init");
    return o;
}

template <typename DT, typename DT_ACC>
void matmul_shmem(const DT* A, const DT* B, DT* C, int M, int N, int K, int tile_dim, int block_rows, bool b_transposed = false,
                  void* stream = nullptr) {
    check(ckopt_matmul_shmem(dtype_of<DT>::value, A, B, C, M, N, K, tile_dim, block_rows, b_transposed ? 1 : 0, stream), "matmul_shmem");
}

template <typename DT, typename DT_ACC>
int get_shmem_req(int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b,
                  int num_stages, int num_consumer_warps) {
    const int r = ckopt_get_lds_req(tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, num_stages,
                                    num_consumer_warps);
    if (r < 0) throw Error(r, "get_shmem_req");
    return r;
}
// get_shmem_req<DT>(tile_dim) of matmul_shmem.cu:138-141: dynamic LDS bytes of a matmul_shmem launch
template <typename DT>
int get_shmem_req(int tile_dim) {
    const int r = ckopt_matmul_shmem_lds_req(dtype_of<DT>::value, tile_dim);
    if (r < 0) throw Error(r, "get_shmem_req");
    return r;
}
// tuning tuple for a problem size in the launcher's parameter order (no counterpart in the reference)
struct Tuning {
    int tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, num_stages,
        num_producer_warps, num_consumer_warps;
};
inline Tuning suggest_gemm_tuning(int M, int N, int K, int num_sms) {
    int v[10];
    const int r = ckopt_suggest_gemm_tuning(M, N, K, num_sms, v);
    if (r < 0) throw Error(r, "suggest_gemm_tuning");
    return Tuning{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7], v[8], v[9]};
}

// what a launch of `t` on these sizes will run (ckopt_gemm_launch_plan)
struct LaunchPlan {
    bool straight_line;
    int tile_cols, k_slices;
    bool operand_copies;
    int sliced_tiles;          // tiles cut into k_slices (0: none)
    bool reduced_in_kernel;    // the slices are added inside the kernel (no second kernel)
    int grid;                  // workgroups of the straight-line kernel
};
inline LaunchPlan gemm_launch_plan(int M, int N, int K, bool operands_aligned, const Tuning& t, int num_sms,
                                   const ckopt_launch_options* options = nullptr) {
    int v[7];
    check(ckopt_gemm_launch_plan_ex(M, N, K, operands_aligned ? 1 : 0, t.tile_dim, t.segment_dim_k, t.bar_steps_a, t.bar_steps_b,
                                    t.bar_step_rows_a, t.bar_step_rows_b, t.tile_group_m, t.num_stages, t.num_producer_warps,
                                    t.num_consumer_warps, num_sms, options, v),
          "gemm_launch_plan");
    return LaunchPlan{v[0] != 0, v[1], v[2], v[3] != 0, v[4], v[5] != 0, v[6]};
}

inline int get_num_acc(int tile_dim, int num_consumer_warps) {
    const int r = ckopt_get_num_acc(tile_dim, num_consumer_warps);
    if (r < 0) throw Error(r, "get_num_acc");
    return r;
}
inline int get_warp_tile_rows(int tile_dim, int num_consumer_warps) {
    const int r = ckopt_get_warp_tile_rows(tile_dim, num_consumer_warps);
    if (r < 0) throw Error(r, "get_warp_tile_rows");
    return r;
}

}  // namespace ckopt
#endif  // CKOPT_HPP

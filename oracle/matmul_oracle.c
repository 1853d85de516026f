/* CPU ORACLE - TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C restatement of the CPU side of alfin3/cuda-kernel-opt that the GPU results are checked
 * against. Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this file's
 * library; nothing under cuda-kernel-opt_amd/ links or calls it.
 *
 * What each function follows in the reference (/root/reference):
 *   oracle_gemm_rows / oracle_gemm            matmul_test.h:289-302, :307-326 (MatmulTestGemmSquare::
 *                                            IsCorrect / GetNumIncorrect): temp = 0; for k ascending:
 *                                            temp += float(a[i*K+k]) * float(bt[j*K+k]); value =
 *                                            alpha*temp + beta*c. The reference writes the Bt stride as
 *                                            dim.n, equal to K only for its square tests; K is used here.
 *   oracle_gemm_blocked                       same arithmetic per element (one accumulator, ascending
 *                                            k, separately rounded multiply and add), vectorised ACROSS
 *                                            output columns only; pinned bit-for-bit to oracle_gemm.
 *   oracle_matmul                             matmul_test.h:121-137 (MatmulTestSquare): b[k*N+j], the
 *                                            sum is cast to DT before comparing. `fused` selects one
 *                                            fmaf per k instead of multiply-then-add: what the
 *                                            reference's GPU kernel computes (matmul_shmem.cu:87 under
 *                                            the device compiler's default contraction).
 *   oracle_get_num_acc / _warp_tile_rows      matmul_shmem_tc_async_opt_port_2.cu:158-169 (closed forms
 *                                            as written there, domain tile in {64,128}, C in {4,8}).
 *   oracle_get_tile_offset_cd                 port_2.cu:605-614 (int arithmetic as written there).
 *   oracle_get_shmem_req                      port_2.cu:1057-1086 incl. the "+ size % 32" quirk; the
 *                                            product's LDS layout differs by design, this restatement
 *                                            only documents the reference's numbers.
 *   oracle_count_incorrect                    matmul_test.h:320 (|expected - res| > atol counting).
 *
 * Pinning (see tests/test_oracle.py): constant matrices against the closed form alpha*a*b*K+beta*c
 * (matmul_test.h:279-288); small-integer inputs against exact int64 numpy; fp16/bf16 decode against
 * numpy/torch; blocked vs scalar bit-for-bit; identity and one-hot operands; index helpers against the
 * README table (2/4/8/16), bijection of the tile order, and the reference's smem figures.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

enum { DT_F16 = 0, DT_BF16 = 1, DT_F32 = 2, DT_I32 = 3 };

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

float oracle_half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1f) return bits_to_f32(sign | 0x7f800000u | (m << 13));
    if (e != 0) return bits_to_f32(sign | ((e + 112u) << 23) | (m << 13));
    /* zero or subnormal: m * 2^-24, exact in float */
    const float v = ldexpf((float)m, -24);
    return sign ? -v : v;
}

float oracle_bf16_to_float(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

static inline float elem16(int dtype, const uint16_t* p, int64_t idx) {
    return dtype == DT_F16 ? oracle_half_to_float(p[idx]) : oracle_bf16_to_float(p[idx]);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Rows [row_begin, row_end) of alpha * A * Bt^T + beta * C into out (row-major, N columns,
 * out row 0 = row_begin). dtype: DT_F16 or DT_BF16. c may be NULL when beta == 0. */
int oracle_gemm_rows(int dtype, const uint16_t* a, const uint16_t* bt, const float* c, float* out, float alpha,
                     float beta, int M, int N, int K, int row_begin, int row_end, int threads) {
    if (!(dtype == DT_F16 || dtype == DT_BF16) || row_begin < 0 || row_end > M || row_begin > row_end) return -1;
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 0 ? threads : omp_get_max_threads())
#endif
    for (int i = row_begin; i < row_end; ++i) {
        for (int j = 0; j < N; ++j) {
            float temp = 0.0f;
            for (int k = 0; k < K; ++k) {
                temp += elem16(dtype, a, (int64_t)i * K + k) * elem16(dtype, bt, (int64_t)j * K + k);
            }
            float v = alpha * temp;
            if (beta != 0.0f) v = alpha * temp + beta * c[(int64_t)i * N + j];
            out[(int64_t)(i - row_begin) * N + j] = v;
        }
    }
    return 0;
}

int oracle_gemm(int dtype, const uint16_t* a, const uint16_t* bt, const float* c, float* out, float alpha, float beta,
                int M, int N, int K, int threads) {
    return oracle_gemm_rows(dtype, a, bt, c, out, alpha, beta, M, N, K, 0, M, threads);
}

/* Same values as oracle_gemm_rows, computed IB rows x JB columns at a time so that the inner loop
 * runs over independent output columns and vectorises. Each output still owns one accumulator that
 * sees k = 0, 1, 2, ... in order with a separately rounded multiply and add. */
#define IB 4
#define JB 128
__attribute__((target_clones("default", "avx2", "avx512f")))
static void gemm_panel(const float* af, const float* bpanel /* K x JB */, float* acc /* IB x JB */, int K, int ib) {
    for (int k = 0; k < K; ++k) {
        const float* brow = bpanel + (int64_t)k * JB;
        for (int ii = 0; ii < ib; ++ii) {
            const float av = af[(int64_t)ii * K + k];
            float* arow = acc + ii * JB;
            for (int jj = 0; jj < JB; ++jj) {
                const float p = av * brow[jj];
                arow[jj] = arow[jj] + p;
            }
        }
    }
}

int oracle_gemm_blocked(int dtype, const uint16_t* a, const uint16_t* bt, const float* c, float* out, float alpha,
                        float beta, int M, int N, int K, int row_begin, int row_end, int threads) {
    if (!(dtype == DT_F16 || dtype == DT_BF16) || row_begin < 0 || row_end > M || row_begin > row_end) return -1;
    const int rows = row_end - row_begin;
    if (rows == 0) return 0;
    float* af = (float*)malloc((size_t)rows * K * sizeof(float));
    if (!af) return -2;
    for (int64_t i = 0; i < (int64_t)rows * K; ++i) af[i] = elem16(dtype, a, (int64_t)row_begin * K + i);
    const int npanels = (N + JB - 1) / JB;
    int fail = 0;
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel num_threads(threads > 0 ? threads : omp_get_max_threads())
#endif
    {
        float* bpanel = (float*)malloc((size_t)K * JB * sizeof(float));
        float acc[IB * JB];
        if (!bpanel) {
#ifdef _OPENMP
#pragma omp atomic write
#endif
            fail = 1;
        }
#ifdef _OPENMP
#pragma omp for schedule(dynamic, 1)
#endif
        for (int p = 0; p < npanels; ++p) {
            if (!bpanel) continue;
            const int j0 = p * JB;
            const int jn = N - j0 < JB ? N - j0 : JB;
            for (int k = 0; k < K; ++k)
                for (int jj = 0; jj < JB; ++jj)
                    bpanel[(int64_t)k * JB + jj] = jj < jn ? elem16(dtype, bt, (int64_t)(j0 + jj) * K + k) : 0.0f;
            for (int i0 = 0; i0 < rows; i0 += IB) {
                const int ib = rows - i0 < IB ? rows - i0 : IB;
                memset(acc, 0, sizeof(acc));
                gemm_panel(af + (int64_t)i0 * K, bpanel, acc, K, ib);
                for (int ii = 0; ii < ib; ++ii)
                    for (int jj = 0; jj < jn; ++jj) {
                        const float temp = acc[ii * JB + jj];
                        float v = alpha * temp;
                        if (beta != 0.0f) v = alpha * temp + beta * c[(int64_t)(row_begin + i0 + ii) * N + j0 + jj];
                        out[(int64_t)(i0 + ii) * N + j0 + jj] = v;
                    }
            }
        }
        free(bpanel);
    }
    free(af);
    return fail ? -2 : 0;
}

/* matmul_shmem check: C = A * B, A M x K, B K x N (or N x K when b_transposed), element type dtype
 * in {DT_F32, DT_F16, DT_I32}; accumulate in float (int for DT_I32), ascending k; the result is
 * converted to the element type (DT_F16 results are returned as float values already rounded to
 * half by the caller-provided rounding in the tests, so `out` is float for F32/F16 and int32 for I32).
 * fused != 0: one fmaf per k. Rows [row_begin, row_end). */
int oracle_matmul(int dtype, const void* a, const void* b, void* out, int M, int N, int K, int b_transposed, int fused,
                  int row_begin, int row_end, int threads) {
    if (row_begin < 0 || row_end > M || row_begin > row_end) return -1;
    if (!(dtype == DT_F32 || dtype == DT_F16 || dtype == DT_I32)) return -1;
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 0 ? threads : omp_get_max_threads())
#endif
    for (int i = row_begin; i < row_end; ++i) {
        for (int j = 0; j < N; ++j) {
            if (dtype == DT_I32) {
                const int32_t* ai = (const int32_t*)a;
                const int32_t* bi = (const int32_t*)b;
                int32_t temp = 0;
                for (int k = 0; k < K; ++k)
                    temp += ai[(int64_t)i * K + k] * (b_transposed ? bi[(int64_t)j * K + k] : bi[(int64_t)k * N + j]);
                ((int32_t*)out)[(int64_t)(i - row_begin) * N + j] = temp;
            } else {
                float temp = 0.0f;
                for (int k = 0; k < K; ++k) {
                    float x, y;
                    if (dtype == DT_F32) {
                        x = ((const float*)a)[(int64_t)i * K + k];
                        y = b_transposed ? ((const float*)b)[(int64_t)j * K + k] : ((const float*)b)[(int64_t)k * N + j];
                    } else {
                        x = oracle_half_to_float(((const uint16_t*)a)[(int64_t)i * K + k]);
                        y = oracle_half_to_float(b_transposed ? ((const uint16_t*)b)[(int64_t)j * K + k]
                                                              : ((const uint16_t*)b)[(int64_t)k * N + j]);
                    }
                    if (fused) temp = fmaf(x, y, temp);
                    else { const float p = x * y; temp = temp + p; }
                }
                ((float*)out)[(int64_t)(i - row_begin) * N + j] = temp;
            }
        }
    }
    return 0;
}

/* matmul_test.h:320 - number of elements with |expected - res| > atol */
int64_t oracle_count_incorrect(const float* expected, const float* res, int64_t n, float atol) {
    int64_t count = 0;
    for (int64_t i = 0; i < n; ++i) {
        const float d = fabsf(expected[i] - res[i]);
        if (d > atol || d != d) ++count;
    }
    return count;
}

/* Number of elements violating |res - ref| <= rtol * (|ref| + 1); *worst gets max |res-ref|/(|ref|+1). */
int64_t oracle_count_outside_rel(const float* ref, const float* res, int64_t n, float rtol, float* worst) {
    int64_t count = 0;
    float w = 0.0f;
    for (int64_t i = 0; i < n; ++i) {
        const float d = fabsf(res[i] - ref[i]) / (fabsf(ref[i]) + 1.0f);
        if (!(d <= rtol)) ++count;
        if (d > w || d != d) w = d;
    }
    if (worst) *worst = w;
    return count;
}

/* ---- index helpers, as written in the reference -------------------------------------------------- */
int oracle_get_num_acc(int tile_dim, int num_consumer_warps) {
    return (4 >> (tile_dim == 64)) * ((4 >> (tile_dim == 64)) >> (num_consumer_warps == 8));
}

int oracle_get_warp_tile_rows(int tile_dim, int num_consumer_warps) {
    const int num_acc = oracle_get_num_acc(tile_dim, num_consumer_warps);
    return num_acc < 8 ? num_acc / 2 : num_acc / 4;
}

int oracle_get_tile_offset_cd(int M, int N, int tile_dim, int tile_group_m, int tile_count) {
    const int group_tile_count = tile_group_m * N / tile_dim;
    const int group_first_row = (tile_count / group_tile_count) * tile_group_m;
    const int rem = M / tile_dim - group_first_row;
    const int group_rows = rem < tile_group_m ? rem : tile_group_m;
    const int tile_row = group_first_row + (tile_count % group_tile_count) % group_rows;
    const int tile_col = (tile_count % group_tile_count) / group_rows;
    return tile_row * tile_dim * N + tile_col * tile_dim;
}

int oracle_get_shmem_req(int sizeof_dt, int sizeof_dt_acc, int tile_dim, int segment_k_dim, int bar_steps_a,
                         int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b, int num_stages,
                         int num_consumer_warps) {
    const int WMMA = 16, SKEW_HALF = 16, SHMEM_ALIGNMENT = 32, SIZEOF_BARRIER = 8;
    const int wtr = oracle_get_warp_tile_rows(tile_dim, num_consumer_warps);
    const int wtc = oracle_get_num_acc(tile_dim, num_consumer_warps) / wtr;
    int na = 0, nb = 0;
    if (bar_step_rows_a == tile_dim && bar_step_rows_b == tile_dim) {
        na = num_stages; nb = num_stages;
    } else if (bar_step_rows_a == wtr * WMMA && bar_step_rows_b == wtc * WMMA) {
        na = num_stages * (bar_steps_a * bar_steps_b + 1); nb = na;
    } else if (bar_step_rows_a == WMMA && bar_step_rows_b == WMMA) {
        na = num_stages * num_consumer_warps * (bar_steps_a + 1);
        nb = num_stages * num_consumer_warps * (bar_steps_b + 1);
    } else {
        return -1;
    }
    const int bar = (1 + 2 * (na + nb)) * SIZEOF_BARRIER;
    const int bar_al = bar + bar % SHMEM_ALIGNMENT;
    const int size_ab = num_stages * (2 * tile_dim * (segment_k_dim + SKEW_HALF) * sizeof_dt) + bar_al;
    const int size_cd = tile_dim * tile_dim * sizeof_dt_acc + bar_al;
    return size_ab > size_cd ? size_ab : size_cd;
}

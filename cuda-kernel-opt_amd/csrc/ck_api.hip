// extern "C" launch layer: parameter validation, instance dispatch, device status word.
// Declarations and the reference launcher each entry point replaces are in include/ckopt.h.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <cmath>
#include <mutex>
#include <type_traits>

#include "../../include/ckopt.h"
#include "ck_common.h"
#include "gemm_pc_kernel.hip.h"
#include "simt_kernel.hip.h"

namespace ck {
#define CK_DECL_GEMM(NAME) \
    hipError_t NAME(int tile, int segk, int cw, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const GemmArgs& a);
CK_DECL_GEMM(launch_gemm_pc_f16_m0) CK_DECL_GEMM(launch_gemm_pc_f16_m1) CK_DECL_GEMM(launch_gemm_pc_f16_m2)
CK_DECL_GEMM(launch_gemm_pc_bf16_m0) CK_DECL_GEMM(launch_gemm_pc_bf16_m1) CK_DECL_GEMM(launch_gemm_pc_bf16_m2)
#undef CK_DECL_GEMM
hipError_t launch_gemm_pcb_f16(int tile, int segk, int cw, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const GemmArgs& a);
hipError_t launch_gemm_pcb_bf16(int tile, int segk, int cw, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const GemmArgs& a);
hipError_t launch_gemm_stream_f16(dim3 grid, hipStream_t stream, const GemmArgs& a, bool barrier_every_kstep, int tile_n);
hipError_t launch_gemm_stream_bf16(dim3 grid, hipStream_t stream, const GemmArgs& a, bool barrier_every_kstep, int tile_n);
bool gemm_stream_applies(const GemmArgs& a, int tile_dim, int segment_dim_k, int num_stages, int producer_waves, int consumer_waves);
constexpr int STREAM_K_MULTIPLE_HOST = 64;  // K extent of one loop body of the straight-line kernel
hipError_t launch_gemm_fused_f16(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a);
hipError_t launch_gemm_fused_bf16(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a);
hipError_t launch_gemm_sync_f16(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a);
hipError_t launch_gemm_sync_bf16(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a);
hipError_t launch_matmul_shmem(int dtype, int tile, int accs, bool bt, dim3 grid, hipStream_t s, const SimtArgs& a);
}  // namespace ck

// One status word per device; the kernels OR a bit into it when a bounded flag wait gives up.
__device__ unsigned int ck_status_word[8] = {};  // [0]: status bits, [2..5]: cycles and reference ticks of the last launch

// Scratch memory of the entry point that allocates nothing (ckopt_gemm_shmem_tc_async_opt_port_2_noalloc): the
// zero-padded operand copies and the split-K planes of one launch. Every device the library runs on holds its own
// copy of the array, at its own address, until the process ends. Host code never uses the array's name as an
// address: the per-device address comes from hipGetSymbolAddress (static_scratch_for_current_device below). That
// host-side use is what makes the compiler emit the array into the code object under a global symbol the runtime can
// look up; marked __attribute__((used)) it would stay a local symbol and the lookup would abort the process.
static __device__ __align__(256) unsigned char scratch[CKOPT_NOALLOC_SCRATCH_BYTES];

namespace {

// The knobs that are not launcher parameters in the reference. A launch works on one Options value: the caller's
// ckopt_launch_options, or a snapshot of the process-wide defaults taken once when the entry point starts.
enum { OPT_SWIZZLE, OPT_SPIN_LIMIT, OPT_NUM_XCD, OPT_PRIO_MODE, OPT_PRODUCER_NAP, OPT_TILE_SYNC_BARRIER, OPT_STRAIGHT_LINE, OPT_SPLIT_K,
       OPT_BARRIER_EVERY_KSTEP, OPT_EVEN_ROUNDS, OPT_D_STORE_POLICY, OPT_HALF_WIDTH, OPT_TAIL_ROUND, OPT_FUSED_REDUCTION, OPT_BATCHED_EMPTY_READS,
       NUM_OPTIONS };
struct OptionRule { int initial, lo, hi; };
constexpr OptionRule OPTION_RULES[NUM_OPTIONS] = {
    {1, 0, 1}, {1 << 22, 1, 0x7fffffff}, {8, 1, 64}, {0, 0, 2}, {0, 0, 2}, {0, 0, 1}, {1, 0, 1}, {1, 0, 16},
    {1, 0, 1}, {1, 0, 1}, {0, 0, 2}, {1, 0, 3}, {1, 0, 1}, {1, 0, 2}, {1, 0, 1}};
std::atomic<int> g_option[NUM_OPTIONS] = {{1}, {1 << 22}, {8}, {0}, {0}, {0}, {1}, {1}, {1}, {1}, {0}, {1}, {1}, {1}, {1}};
struct Options {
    int v[NUM_OPTIONS];
    int operator[](int key) const { return v[key]; }
};
Options default_options() {
    Options o;
    for (int k = 0; k < NUM_OPTIONS; ++k) o.v[k] = g_option[k].load();
    return o;
}
// the public struct's fields follow struct_bytes in key order
int options_from_public(const ckopt_launch_options* p, Options* out) {
    if (!p) { *out = default_options(); return ck::CK_OK; }
    if (p->struct_bytes != (int)sizeof(ckopt_launch_options)) return ck::CK_ERR_BAD_PARAM;
    const int* f = &p->lds_swizzle;
    for (int k = 0; k < NUM_OPTIONS; ++k) {
        if (f[k] < OPTION_RULES[k].lo || f[k] > OPTION_RULES[k].hi) return ck::CK_ERR_BAD_PARAM;
        out->v[k] = f[k];
    }
    return ck::CK_OK;
}
static_assert(sizeof(ckopt_launch_options) == (NUM_OPTIONS + 1) * sizeof(int), "one int per key behind struct_bytes");
constexpr int LINE_BYTES = 128;         // cache line of the vector memory path
constexpr int TAIL_ROUND_MAX_SLICES = 4;   // the partly filled last round is cut into at most this many slices
constexpr int SPLIT_K_MIN_SLICE = 1024;  // shortest K slice split-K will make (shorter ones lose more in the reduction pass than they gain)

constexpr int MAX_DEV = 64;
std::mutex g_status_mutex;
unsigned int* g_status_ptr[MAX_DEV] = {};

int status_ptr_for_current_device(unsigned int** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return ck::CK_ERR_HIP;
    if (dev < 0 || dev >= MAX_DEV) return ck::CK_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_status_mutex);
    if (!g_status_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(ck_status_word)) != hipSuccess || !p) return ck::CK_ERR_HIP;
        g_status_ptr[dev] = static_cast<unsigned int*>(p);
    }
    *out = g_status_ptr[dev];
    return ck::CK_OK;
}

unsigned char* g_scratch_ptr[MAX_DEV] = {};

// Compute units of the current device (what the cost model's measurements scale with), read once per device;
// 256, the device the model was calibrated on, where no device can be asked.
int g_device_cus[MAX_DEV] = {};
int device_cus() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) {
        (void)hipGetLastError();
        return 256;
    }
    std::lock_guard<std::mutex> lock(g_status_mutex);
    if (!g_device_cus[dev]) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = 256;
        }
        g_device_cus[dev] = n;
    }
    return g_device_cus[dev];
}

// Device address of this device's copy of `scratch`, looked up once per device with that device current.
int static_scratch_for_current_device(unsigned char** out) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return ck::CK_ERR_HIP;
    if (dev < 0 || dev >= MAX_DEV) return ck::CK_ERR_HIP;
    std::lock_guard<std::mutex> lock(g_status_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return ck::CK_ERR_HIP;
        g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
    }
    *out = g_scratch_ptr[dev];
    return ck::CK_OK;
}

// Copies `rows` rows of K 2-byte elements into rows of Kp >= K elements (Kp % 8 == 0), zero filling
// the tail: the form the direct-to-LDS loads need (every row starts on a 16-byte boundary). One
// thread produces one 16-byte chunk of the destination.
// Both operands go through one launch: chunks [0, rows_a * Kp / 8) belong to A, the rest to Bt.
__global__ void pad_rows_kernel(const unsigned short* __restrict__ src_a, unsigned short* __restrict__ dst_a, int rows_a,
                                const unsigned short* __restrict__ src_b, unsigned short* __restrict__ dst_b, int rows_b, int K, int Kp) {
    const int chunks_per_row = Kp / 8;
    const long long total_a = (long long)rows_a * chunks_per_row;
    const long long total = total_a + (long long)rows_b * chunks_per_row;
    for (long long cc = (long long)blockIdx.x * blockDim.x + threadIdx.x; cc < total; cc += (long long)gridDim.x * blockDim.x) {
        const bool second = cc >= total_a;
        const unsigned short* src = second ? src_b : src_a;
        unsigned short* dst = second ? dst_b : dst_a;
        const long long c = second ? cc - total_a : cc;
        const int r = (int)(c / chunks_per_row), k0 = (int)(c % chunks_per_row) * 8;
        if (k0 + 8 <= K) {
            // a whole chunk of the row: one 16-byte load (the vector memory path takes 2-byte-aligned addresses)
            typedef unsigned int u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
            const u32x4_a2 v = *reinterpret_cast<const u32x4_a2*>(src + (long long)r * K + k0);
            *reinterpret_cast<uint4*>(dst + (long long)r * Kp + k0) = uint4{v[0], v[1], v[2], v[3]};
            continue;
        }
        // The chunk that holds the end of the row (or lies past it). Its 16 source bytes start on a 2-byte boundary: five aligned 4-byte words cover them,
        // shifted by two bytes where the start is odd. A word that lies only half inside
        // [chunk start, row end) is read as that one element, so no byte outside the row is touched.
        const uintptr_t first = (uintptr_t)(src + (long long)r * K + k0);
        const uintptr_t row_end = (uintptr_t)(src + (long long)r * K + K);
        const uintptr_t w0 = first & ~(uintptr_t)3;
        const bool odd = (first & 2) != 0;
        unsigned d[5];
#pragma unroll
        for (int i = 0; i < 5; ++i) {
            const uintptr_t lo = w0 + 4 * i, hi = lo + 2;
            const bool lo_in = lo >= first && lo < row_end, hi_in = hi >= first && hi < row_end;
            if (lo_in && hi_in) d[i] = *reinterpret_cast<const unsigned*>(lo);
            else d[i] = (lo_in ? (unsigned)*reinterpret_cast<const unsigned short*>(lo) : 0u) |
                        (hi_in ? (unsigned)*reinterpret_cast<const unsigned short*>(hi) << 16 : 0u);
        }
        unsigned o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            o[i] = odd ? (d[i] >> 16) | (d[i + 1] << 16) : d[i];
            const int k = k0 + 2 * i;  // elements k, k + 1 of the row: zero where the row has ended
            if (k >= K) o[i] = 0u;
            else if (k + 1 >= K) o[i] &= 0xffffu;
        }
        *reinterpret_cast<uint4*>(dst + (long long)r * Kp + k0) = uint4{o[0], o[1], o[2], o[3]};
    }
}

// Second pass of a split-K product: D = alpha * (plane 0 + plane 1 + ...) + beta * C, the planes added in
// slice order (the result does not depend on how the first pass was scheduled). One thread per element;
// DT16 selects the 16-bit C/D forms.
template <int OUT16, bool BF16>
__global__ void splitk_reduce_kernel(const float* __restrict__ ws, int slices, long long count, const void* C, void* D, float alpha, float beta) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (long long)gridDim.x * blockDim.x) {
        float sum = ws[i];
        for (int s = 1; s < slices; ++s) sum += ws[(long long)s * count + i];
        float v = alpha * sum;
        if (OUT16) {
            using O = ck::Out16<typename std::conditional<BF16, ck::bf16_tag, ck::f16_tag>::type>;
            if (beta != 0.f) v += O::load(static_cast<const unsigned short*>(C)[i]) * beta;
            static_cast<unsigned short*>(D)[i] = O::store(v);
        } else {
            if (beta != 0.f) v += static_cast<const float*>(C)[i] * beta;
            static_cast<float*>(D)[i] = v;
        }
    }
}

// The fp32 form of the same pass with four elements per thread (16-byte loads and stores): same additions in
// the same order per element. For count % 4 == 0 and C, D on 16-byte boundaries.
typedef float f32x4 __attribute__((ext_vector_type(4)));
__global__ void splitk_reduce4_kernel(const f32x4* __restrict__ ws, int slices, long long count4, const f32x4* C, f32x4* D, float alpha, float beta) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count4; i += (long long)gridDim.x * blockDim.x) {
        f32x4 sum = __builtin_nontemporal_load(ws + i);
        for (int s = 1; s < slices; ++s) sum += __builtin_nontemporal_load(ws + (long long)s * count4 + i);
        f32x4 v = alpha * sum;
        if (beta != 0.f) v += C[i] * beta;
        D[i] = v;
    }
}

// Clears the arrival words of the reduction inside the straight-line kernel (a kernel, not a memset: callers may
// record the launch into a graph).
__global__ void zero_words_kernel(unsigned int* p, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) p[i] = 0u;
}

// Where a launch takes device memory beyond its operands from (the zero-padded operand copies, the split-K planes).
// ALLOCATE: stream-ordered allocations inside the call. PROVIDED: the buffer [ptr, ptr + bytes) that the caller or the
// library's static array supplies; pieces are carved off its front on 256-byte boundaries and nothing is allocated.
struct Scratch {
    enum Mode { ALLOCATE, PROVIDED } mode;
    char* ptr;
    size_t bytes;
};
constexpr size_t SCRATCH_ALIGN = 256;
size_t scratch_round(size_t n) { return (n + SCRATCH_ALIGN - 1) / SCRATCH_ALIGN * SCRATCH_ALIGN; }

// Stream-ordered allocations come from a memory pool of the library's own, one per device, that keeps freed blocks: the
// device's default pool hands its memory back to the system at every synchronisation, and the launch behind one then
// pays for a fresh allocation (config 4, 20 launches behind a synchronize: 247 us per launch against 229). What the pool
// holds is the largest scratch a launch on that device has used; ckopt_trim_scratch_pool gives it back.
hipMemPool_t g_scratch_pool[MAX_DEV] = {};
bool g_scratch_pool_tried[MAX_DEV] = {};
hipMemPool_t scratch_pool_for_current_device() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) return nullptr;
    std::lock_guard<std::mutex> lock(g_status_mutex);
    if (!g_scratch_pool_tried[dev]) {
        g_scratch_pool_tried[dev] = true;
        hipMemPoolProps props = {};
        props.allocType = hipMemAllocationTypePinned;
        props.handleTypes = hipMemHandleTypeNone;
        props.location.type = hipMemLocationTypeDevice;
        props.location.id = dev;
        hipMemPool_t pool = nullptr;
        if (hipMemPoolCreate(&pool, &props) == hipSuccess && pool) {
            uint64_t keep = UINT64_MAX;
            if (hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &keep) == hipSuccess) g_scratch_pool[dev] = pool;
            else (void)hipMemPoolDestroy(pool);
        }
        (void)hipGetLastError();   // without a pool of its own the library allocates from the device's default pool
    }
    return g_scratch_pool[dev];
}

// Takes `need` bytes: CK_OK with *out set, CK_ERR_HIP if the allocation failed, CK_ERR_TOO_LARGE if a provided buffer
// is too small. A piece of an ALLOCATE scratch is handed back with scratch_release().
int scratch_take(Scratch& sc, size_t need, hipStream_t s, void** out) {
    if (sc.mode == Scratch::ALLOCATE) {
        *out = nullptr;
        hipMemPool_t pool = scratch_pool_for_current_device();
        if ((pool ? hipMallocFromPoolAsync(out, need, pool, s) : hipMallocAsync(out, need, s)) != hipSuccess || !*out) {
            (void)hipGetLastError();  // the failure is reported through the return value, not left for the next HIP call
            return ck::CK_ERR_HIP;
        }
        return ck::CK_OK;
    }
    const uintptr_t base = (uintptr_t)sc.ptr;
    const uintptr_t aligned = (base + SCRATCH_ALIGN - 1) / SCRATCH_ALIGN * SCRATCH_ALIGN;
    const size_t skip = (size_t)(aligned - base);
    if (!sc.ptr || skip > sc.bytes || need > sc.bytes - skip) return ck::CK_ERR_TOO_LARGE;
    *out = (void*)aligned;
    const size_t used = skip + scratch_round(need);
    sc.ptr += used < sc.bytes ? used : sc.bytes;
    sc.bytes -= used < sc.bytes ? used : sc.bytes;
    return ck::CK_OK;
}
bool scratch_release(const Scratch& sc, void* piece, hipStream_t s) {
    return sc.mode != Scratch::ALLOCATE || hipFreeAsync(piece, s) == hipSuccess;
}

int gemm_launch(int dtype, const void* A, const void* Bt, const void* C, void* D, float alpha, float beta, int M,
                int N, int K, const ck::GemmTuning& t, const Options& opt, void* stream, int out16, Scratch sc);

// Estimated duration (microseconds) of the straight-line kernel on `tiles` tiles of 256 x tile_n (256, 192 or 128) of an
// M x N product with K cut into S slices, plus what adding the slices costs when S > 1. The constants
// are measurements of one MI355X (256 CUs) on random operands: a loop body (64 of K) of a 256 x 256 tile takes 1.05 us
// while at most half of the CUs multiply and the clock is free, and grows with the share of active CUs once the device is
// power-limited (1.42 us with all of them); a 256 x 128 tile's body has half the MFMAs and takes 0.585 of that time
// at the power-limited clock but no less than 0.69 us (one barrier per 16 MFMAs), a 256 x 192 tile's three quarters of
// the MFMAs and BODY_192 of the time, no less than BODY_192_MIN_US; a work item costs about 3 us of pipeline
// fill and drain; the items of a round store their tile at the 4.6 TB/s the write path sustains. The slices are added
// either by a reduction pass (reads S planes and writes D at 5.3 TB/s behind about 3 us of launch) or inside the kernel.
// device_cus is the device's real CU count: the power-limit knee lies at half of it. The model is calibrated for a
// 256-CU gfx950.
constexpr double HALF_WIDTH_BODY = 0.585, HALF_WIDTH_BODY_MIN_US = 0.69, BODY_192 = 0.80, BODY_192_MIN_US = 0.88;
double body_us_for(double active, int tile_n, int dev_cus) {
    const double full_body_us = 1.05 * std::max(1.0, std::pow(active / (0.5 * dev_cus), 0.43));
    if (tile_n == 128) return std::max(HALF_WIDTH_BODY_MIN_US, HALF_WIDTH_BODY * full_body_us);
    if (tile_n == 192) return std::max(BODY_192_MIN_US, BODY_192 * full_body_us);
    return full_body_us;
}
// one round of `active` work items of `bodies` loop bodies each, with the store burst that ends it
double round_us_for(double active, double bodies, int tile_n, int dev_cus) {
    const double store_us = active * (double)tile_n * 1024.0 / 4.6e6;
    return bodies * body_us_for(active, tile_n, dev_cus) + store_us + 3.0;
}
// what adding the slices costs: inside the kernel (every wave stores its partial sums and counts itself; the one that
// comes last reads the other S - 1 partials, a block row of 8 KiB at a time, and writes the tile alone - a chain of
// memory round trips at the end of the launch, once per sliced item of a workgroup; measured against the pass: two slices
// of 128 tiles 27 us against 22, three of 81 tiles 35 against 19, four of 64 tiles 47 against 19), or by the reduction pass
double fused_reduction_us(int S, double sliced_items_per_workgroup) { return (17.0 + 10.0 * (double)(S - 1)) * std::max(1.0, sliced_items_per_workgroup); }
double reduction_pass_us(int S, int64_t mn) { return 3.0 + (double)(S + 1) * (double)mn * 4.0 / 5.3e6; }
double split_k_estimate_us(int64_t tiles, int64_t mn, int K, int S, int num_cus, int tile_n, bool fused, int dev_cus) {
    const double items = (double)tiles * S;
    const double rounds = std::ceil(items / num_cus);
    const double active = items / rounds;   // workgroups (CUs) busy in a round
    const double bodies = (double)K / S / ck::STREAM_K_MULTIPLE_HOST;
    double t = rounds * round_us_for(active, bodies, tile_n, dev_cus);
    if (S > 1) t += fused ? fused_reduction_us(S, rounds) : reduction_pass_us(S, mn);
    return t;
}

// How the straight-line kernel runs an M x N x K product on num_cus workgroups.
struct StreamPlan {
    int tile_n;            // tile width: 256, 192 or 128 columns of D
    int64_t tiles;         // tiles of that width
    int64_t whole_tiles;   // tile counts [0, whole_tiles) run over all of K ...
    int slices;            // ... the others in this many K slices each (1: none are cut, whole_tiles == tiles)
    bool fused;            // the slices are added inside the kernel (else by a second pass over slices x M x N planes)
    int grid;              // workgroups
    double us;             // the estimate that decided
};

bool slices_legal(int K, int c) { return c >= 2 && K % (c * ck::STREAM_K_MULTIPLE_HOST) == 0 && K / c >= SPLIT_K_MIN_SLICE; }
// The slices are added inside the kernel where the option allows it and that is estimated cheaper than the reduction
// pass. (No wave waits for another there, so nothing has to be resident together: any number of sliced items per
// workgroup, any grid.)
bool reduces_in_kernel(const Options& opt, int slices, int64_t sliced_tiles, int64_t mn, int num_cus) {
    if (!opt[OPT_FUSED_REDUCTION] || slices < 2) return false;
    const double per_workgroup = std::ceil((double)sliced_tiles * slices / num_cus);
    return opt[OPT_FUSED_REDUCTION] == 2 || fused_reduction_us(slices, per_workgroup) < reduction_pass_us(slices, mn);
}

// Number of K slices for `tiles` tiles that all are cut (1: no split). policy 0: never; 1: automatic - with fewer tiles
// than CUs, the legal slice count whose estimated duration is shortest (a larger count must win by 3 %: it costs scratch
// memory); >= 2: that many slices if legal, else the next smaller legal count.
// Legal: slices of whole loop bodies and at least SPLIT_K_MIN_SLICE deep (any tile count, any N).
int split_k_slices(int64_t tiles, int64_t mn, int K, int num_cus, const Options& opt, int tile_n, int dev_cus) {
    const int policy = opt[OPT_SPLIT_K];
    if (policy == 0 || tiles <= 0) return 1;
    if (policy >= 2) {
        int cand = policy > 16 ? 16 : policy;
        while (cand >= 2 && !slices_legal(K, cand)) --cand;
        return cand < 2 ? 1 : cand;
    }
    if (tiles >= num_cus) return 1;
    int best = 1;
    double best_us = split_k_estimate_us(tiles, mn, K, 1, num_cus, tile_n, false, dev_cus);
    for (int c = 2; c <= 16; ++c) {
        if (!slices_legal(K, c)) continue;
        const double us = split_k_estimate_us(tiles, mn, K, c, num_cus, tile_n, reduces_in_kernel(opt, c, tiles, mn, num_cus), dev_cus);
        if (us < 0.97 * best_us) { best = c; best_us = us; }
    }
    return best;
}

// Workgroups of the persistent grid. With more tiles than CUs, num_cus workgroups run ceil(tiles / num_cus)
// rounds and the last one is partly empty: CUs idle at the end while the full rounds before it ran at the
// power-limited clock. The same number of rounds over fewer workgroups (whole XCDs' worth) keeps every round
// full and spreads the power budget over fewer CUs (bf16 6143 x 4097 x 3071, 408 tiles: 208 workgroups x 2
// rounds are 5.7 % faster than 256 + 152). Never more rounds than num_cus workgroups would take.
int persistent_grid(int64_t tiles, int num_cus, int num_xcd, bool even_rounds) {
    if (tiles <= num_cus) return (int)tiles;
    if (!even_rounds) return num_cus;
    const int64_t rounds = (tiles + num_cus - 1) / num_cus;
    int64_t g = (tiles + rounds - 1) / rounds;
    if (num_xcd > 1) g = (g + num_xcd - 1) / num_xcd * num_xcd;
    return (int)(g < num_cus ? g : num_cus);
}

// Tile width, K slices and grid of a launch. With fewer tiles than CUs every tile may be cut (split_k_slices). With more,
// the full rounds run whole tiles on all num_cus workgroups and the tiles of the partly filled last round are cut into 2
// to 4 slices reduced in the kernel, in the same launch, where that is estimated at least 5 % shorter than rounds of
// whole tiles (6144^3 measures the same either way, 391 us: 576 tiles as 2 x 256 whole tiles + 64 tiles in 2 slices, or as
// 3 rounds of 192 whole tiles; with the 5 % margin it takes the rounds). 256 x 192 or 256 x 128 tiles where they are
// estimated at least 5 % faster than 256 x 256 (they fill a device that the large tiles leave partly idle, at a lower rate
// per CU), or always / never by the option.
StreamPlan stream_plan(int M, int N, int K, int num_cus, const Options& opt) {
    const int64_t mn = (int64_t)M * N;
    const int width = opt[OPT_HALF_WIDTH], dev_cus = device_cus();
    const bool even = opt[OPT_EVEN_ROUNDS] != 0;
    auto plan = [&](int tile_n) {
        const int64_t tiles = (int64_t)((M + 255) / 256) * ((N + tile_n - 1) / tile_n);
        StreamPlan p{tile_n, tiles, tiles, 1, false, persistent_grid(tiles, num_cus, opt[OPT_NUM_XCD], even), 0.0};
        if (tiles <= num_cus) {
            p.slices = split_k_slices(tiles, mn, K, num_cus, opt, tile_n, dev_cus);
            p.fused = reduces_in_kernel(opt, p.slices, tiles, mn, num_cus);
            if (p.slices > 1) {
                p.whole_tiles = 0;
                p.grid = (int)std::min<int64_t>(tiles * p.slices, num_cus);
            }
            p.us = split_k_estimate_us(tiles, mn, K, p.slices, num_cus, tile_n, p.fused, dev_cus);
            return p;
        }
        // rounds of whole tiles (as many rounds as num_cus workgroups need, evenly filled)
        const double rounds = std::ceil((double)tiles / num_cus), bodies = (double)K / ck::STREAM_K_MULTIPLE_HOST;
        p.us = rounds * round_us_for(even ? (double)tiles / rounds : (double)num_cus, bodies, tile_n, dev_cus);
        const int64_t full = tiles / num_cus * num_cus, rest = tiles - full;
        if (rest > 0 && opt[OPT_TAIL_ROUND] && opt[OPT_FUSED_REDUCTION] && opt[OPT_SPLIT_K] == 1) {
            const double head_us = (double)(full / num_cus) * round_us_for(num_cus, bodies, tile_n, dev_cus);
            for (int c = 2; c <= TAIL_ROUND_MAX_SLICES; ++c) {
                if (!slices_legal(K, c) || rest * c > num_cus) continue;
                const double us = head_us + split_k_estimate_us(rest, mn, K, c, num_cus, tile_n, true, dev_cus);
                if (us < 0.95 * p.us) {
                    p.us = us; p.slices = c; p.fused = true; p.whole_tiles = full; p.grid = num_cus;
                }
            }
        }
        return p;
    };
    // width option: 0 only 256 x 256 tiles; 1 the width estimated shortest (a narrower one must beat 256 x 256 by 5 %: per CU
    // it runs at a lower rate, and the estimate is coarse); 2 always 256 x 128; 3 always 256 x 192
    if (width == 2) return plan(128);
    if (width == 3) return plan(192);
    StreamPlan best = plan(256);
    if (width == 0) return best;
    const double bar = 0.95 * best.us;
    for (int tile_n : {192, 128}) {
        const StreamPlan p = plan(tile_n);
        if (p.us < bar && p.us < best.us) best = p;
    }
    return best;
}

// Scratch memory of the K slices of a plan. Reduced in the kernel: per sliced tile `slices` tiles of fp32 in the
// accumulators' layout (every slice's wave stores its partial sums), behind the arrival counters (one 128-byte line per
// sliced tile and wave, cleared by every launch). Reduced by the second pass: slices planes of M x N fp32.
constexpr size_t FIX_STATE_BYTES_PER_TILE = 8 * 128;   // eight waves, one counter per 128-byte line (FIX_STATE_STRIDE_BYTES of the kernel)
size_t fix_state_bytes(const StreamPlan& p) { return (size_t)(p.tiles - p.whole_tiles) * FIX_STATE_BYTES_PER_TILE; }
size_t fix_partial_bytes(const StreamPlan& p) {
    return (size_t)(p.tiles - p.whole_tiles) * (size_t)p.slices * 256 * p.tile_n * sizeof(float);
}

// The tuning tuple the straight-line kernel is written for (it also needs K in whole loop bodies of 64).
bool straight_line_tuple(const ck::GemmTuning& t, const Options& opt) {
    return opt[OPT_STRAIGHT_LINE] && opt[OPT_SWIZZLE] && t.num_producer_waves == 0 && t.num_consumer_waves == 8 && t.tile_dim == 256 &&
           t.segment_dim_k == 32 && t.num_stages == 5;
}
// Does a launch on these sizes first copy A and Bt into zero-padded rows, and with which K? The kernels read operand rows
// that start on 16-byte boundaries in whole 16-byte chunks: copies are made when K % 8 != 0 or an operand is off a
// 16-byte boundary, with K rounded up to whole chunks - for the straight-line tuple to whole loop bodies, so that the
// copies take that kernel's plain instance.
bool needs_copies(int K, bool operands_aligned) { return K % ck::CHUNK_ELEMS != 0 || !operands_aligned; }
int padded_k(int K, const ck::GemmTuning& t, const Options& opt) {
    const int unit = straight_line_tuple(t, opt) ? ck::STREAM_K_MULTIPLE_HOST : ck::CHUNK_ELEMS;
    return (K + unit - 1) / unit * unit;
}
// K the kernels of a launch work on (the one rule the launcher, the workspace query, the plan query and the tuning
// suggestion share)
int launch_k(int K, bool operands_aligned, const ck::GemmTuning& t, const Options& opt) {
    return needs_copies(K, operands_aligned) ? padded_k(K, t, opt) : K;
}

// Scratch bytes a launch takes from a provided buffer whose start is on a 256-byte boundary (the launcher's own
// rules, evaluated without launching): the zero-padded operand copies, then what the K slices need.
size_t scratch_need(int M, int N, int K, bool operands_aligned, const ck::GemmTuning& t, const Options& opt) {
    using namespace ck;
    size_t need = 0;
    const int k = launch_k(K, operands_aligned, t, opt);
    if (needs_copies(K, operands_aligned)) need += scratch_round(((size_t)M + (size_t)N) * k * 2);
    if (straight_line_tuple(t, opt)) {
        const StreamPlan p = stream_plan(M, N, k, t.num_cus, opt);
        if (p.slices > 1 && p.fused) need += scratch_round(fix_state_bytes(p)) + scratch_round(fix_partial_bytes(p));
        else if (p.slices > 1) need += scratch_round((size_t)p.slices * M * N * sizeof(float));
    }
    return need;
}

// K % 8 != 0 or operands off a 16-byte boundary: the product is computed from zero-padded,
// aligned copies of A and Bt in a stream-ordered temporary (zeros in the K tail add nothing).
int gemm_launch_repacked(int dtype, const void* A, const void* Bt, const void* C, void* D, float alpha, float beta,
                         int M, int N, int K, const ck::GemmTuning& t, const Options& opt, void* stream, int out16, Scratch sc) {
    using namespace ck;
    const int Kp = padded_k(K, t, opt);
    const size_t bytes_a = (size_t)M * Kp * 2, bytes_b = (size_t)N * Kp * 2;
    hipStream_t s = static_cast<hipStream_t>(stream);
    void* ws = nullptr;
    const int trc = scratch_take(sc, bytes_a + bytes_b, s, &ws);
    if (trc != CK_OK) return trc;
    unsigned short* pa = static_cast<unsigned short*>(ws);
    unsigned short* pb = pa + (size_t)M * Kp;
    const int threads = 256;
    auto blocks = [&](long long chunks) { long long b = (chunks + threads - 1) / threads; return (unsigned)(b < 65535 * 8 ? (b > 0 ? b : 1) : 65535 * 8); };
    hipLaunchKernelGGL(pad_rows_kernel, dim3(blocks(((long long)M + N) * (Kp / 8))), dim3(threads), 0, s, static_cast<const unsigned short*>(A), pa, M,
                       static_cast<const unsigned short*>(Bt), pb, N, K, Kp);
    int rc = hipGetLastError() == hipSuccess ? CK_OK : CK_ERR_HIP;
    if (rc == CK_OK) rc = gemm_launch(dtype, pa, pb, C, D, alpha, beta, M, N, Kp, t, opt, stream, out16, sc);
    if (!scratch_release(sc, ws, s) && rc == CK_OK) rc = CK_ERR_HIP;
    return rc;
}

int gemm_launch(int dtype, const void* A, const void* Bt, const void* C, void* D, float alpha, float beta, int M,
                int N, int K, const ck::GemmTuning& t, const Options& opt, void* stream, int out16, Scratch sc) {
    using namespace ck;
    if (!(dtype == CK_DT_F16 || dtype == CK_DT_BF16)) return CK_ERR_BAD_PARAM;
    if (M <= 0 || N <= 0 || K <= 0) return CK_ERR_BAD_PARAM;
    const int rc = check_gemm_tuning(t);
    if (rc != CK_OK) return rc;
    if (!A || !Bt || !D) return CK_ERR_NULL;
    if (beta != 0.f && !C) return CK_ERR_NULL;
    if (((uintptr_t)A & 1) || ((uintptr_t)Bt & 1)) return CK_ERR_ALIGNMENT;
    const uintptr_t elem_mask = out16 ? 1 : 3;
    if (((uintptr_t)D & elem_mask) || ((uintptr_t)C & elem_mask)) return CK_ERR_ALIGNMENT;
    // the kernels want every operand row on a 16-byte boundary
    if (needs_copies(K, !(((uintptr_t)A | (uintptr_t)Bt) & 15)))
        return gemm_launch_repacked(dtype, A, Bt, C, D, alpha, beta, M, N, K, t, opt, stream, out16, sc);
    // one tile's rows are addressed through a 32-bit buffer offset
    if ((int64_t)t.tile_dim * K * 2 >= (int64_t)1 << 31) return CK_ERR_TOO_LARGE;

    const int mode = sync_mode_of(t.tile_dim, t.num_consumer_waves, t.bar_step_rows_a, t.bar_step_rows_b);
    GemmArgs a{};
    a.A = A; a.Bt = Bt; a.C = static_cast<const float*>(C); a.D = static_cast<float*>(D);
    a.out16 = out16 ? 1 : 0;
    a.alpha = alpha; a.beta = beta;
    a.M = M; a.N = N; a.K = K;
    a.tiles_m = (M + t.tile_dim - 1) / t.tile_dim;
    a.tiles_n = (N + t.tile_dim - 1) / t.tile_dim;
    a.nseg = (K + t.segment_dim_k - 1) / t.segment_dim_k;
    a.tile_group_m = t.tile_group_m;
    a.num_stages = t.num_stages;
    // one producer wave (port_0 only): it streams A and then Bt of every segment, and counts as one arrival on each operand's counter
    a.single_producer = t.num_producer_waves == 1;
    a.pa = a.single_producer ? 1 : t.num_producer_waves / 2;
    a.pb = a.single_producer ? 1 : t.num_producer_waves - a.pa;
    a.bar_steps_a = mode == CK_SYNC_TILE ? 0 : t.bar_steps_a;
    a.bar_steps_b = mode == CK_SYNC_TILE ? 0 : t.bar_steps_b;
    a.swizzle = opt[OPT_SWIZZLE];
    a.num_xcd = opt[OPT_NUM_XCD];
    // one vector access per accumulator block: 16 bytes of fp32 need only the 4-byte alignment checked above
    // (any N); 8 bytes of 16-bit results need their own alignment
    a.vec_store = !out16 || ((N % 4 == 0) && !((uintptr_t)D & 7) && (beta == 0.f || !((uintptr_t)C & 7)));
    // Non-temporal stores of D pay where the stores of a row fill whole 128-byte lines; rows that start anywhere make
    // every 128-byte run straddle two lines, and only ordinary stores let the two parts meet in L2.
    const int store_policy = opt[OPT_D_STORE_POLICY];
    auto whole_lines = [](const void* base, int64_t row_bytes) { return (uintptr_t)base % LINE_BYTES == 0 && row_bytes % LINE_BYTES == 0; };
    a.nt_store = store_policy == 1 || (store_policy == 0 && whole_lines(D, (int64_t)N * (out16 ? 2 : 4)));
    a.spin_limit = (uint32_t)opt[OPT_SPIN_LIMIT];
    a.prio_mode = opt[OPT_PRIO_MODE];
    a.producer_nap = opt[OPT_PRODUCER_NAP];
    a.batched_empty_reads = opt[OPT_BATCHED_EMPTY_READS];
    const int src = status_ptr_for_current_device(&a.status);
    if (src != CK_OK) return src;

    const int64_t tiles = (int64_t)a.tiles_m * a.tiles_n;
    const int grid = persistent_grid(tiles, t.num_cus, a.num_xcd, opt[OPT_EVEN_ROUNDS] != 0);
    const dim3 block((t.num_producer_waves + t.num_consumer_waves) * WAVE);
    const size_t lds = (size_t)gemm_lds_bytes(t);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = hipErrorInvalidValue;
    a.split_k = 1;
    a.split_chunk = 32;
    a.whole_tiles = (int)tiles;
    a.fix_partials = nullptr;
    a.fix_state = nullptr;
    if (straight_line_tuple(t, opt) && gemm_stream_applies(a, t.tile_dim, t.segment_dim_k, t.num_stages, t.num_producer_waves, t.num_consumer_waves)) {
        // Tile width, K slices and grid from the cost model: few tiles and a deep K are cut into slices so that every CU
        // has an item; the partly filled last round of many tiles likewise; tile counts that leave much of the device idle
        // take 256 x 128 tiles.
        const bool bek = opt[OPT_BARRIER_EVERY_KSTEP] != 0;
        StreamPlan plan = stream_plan(M, N, K, t.num_cus, opt);
        const int tile_n = plan.tile_n;
        a.tiles_n = (N + tile_n - 1) / tile_n;
        const long long count = (long long)M * N;
        auto launch = [&](const GemmArgs& args, int wgs) {
            return dtype == CK_DT_F16 ? launch_gemm_stream_f16(dim3(wgs), s, args, bek, tile_n) : launch_gemm_stream_bf16(dim3(wgs), s, args, bek, tile_n);
        };
        // the K slices' scratch memory: a provided buffer that is too small is the caller's error; a failed allocation
        // is not - the launch of whole tiles computes the same product without any
        void* state = nullptr;
        float* ws = nullptr;
        if (plan.slices > 1) {
            int trc = CK_OK;
            if (plan.fused) {
                trc = scratch_take(sc, fix_state_bytes(plan), s, &state);
                if (trc == CK_OK) {
                    trc = scratch_take(sc, fix_partial_bytes(plan), s, (void**)&ws);
                    if (trc != CK_OK) (void)scratch_release(sc, state, s);
                }
            } else {
                trc = scratch_take(sc, (size_t)plan.slices * count * sizeof(float), s, (void**)&ws);
            }
            if (trc == CK_ERR_TOO_LARGE) return trc;
            if (trc != CK_OK) {
                plan.slices = 1; plan.whole_tiles = plan.tiles; plan.fused = false;
                plan.grid = persistent_grid(plan.tiles, t.num_cus, a.num_xcd, opt[OPT_EVEN_ROUNDS] != 0);
            }
        }
        const int64_t sliced_tiles = plan.tiles - plan.whole_tiles;
        if (plan.slices == 1) {
            e = launch(a, plan.grid);
        } else if (plan.fused) {
            // one launch: the whole tiles, then the (tile, slice) items; of a wave tile's slices the wave that arrives last adds them all
            GemmArgs p = a;
            p.split_k = plan.slices;
            p.whole_tiles = (int)plan.whole_tiles;
            // sliced items are dealt slice by slice in runs of split_chunk tiles: 32 (what an XCD runs at a time) when the
            // sliced tiles come in whole runs of 32, otherwise all of them in one run
            p.split_chunk = sliced_tiles % 32 == 0 ? 32 : (int)sliced_tiles;
            p.fix_state = static_cast<unsigned int*>(state);
            p.fix_partials = ws;
            const long long words = (long long)(fix_state_bytes(plan) / 4);
            hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)std::min<long long>((words + 255) / 256, 1024)), dim3(256), 0, s, p.fix_state, words);
            e = hipGetLastError();
            if (e == hipSuccess) e = launch(p, plan.grid);
            if (!scratch_release(sc, ws, s) && e == hipSuccess) e = hipErrorUnknown;
            if (!scratch_release(sc, state, s) && e == hipSuccess) e = hipErrorUnknown;
        } else {
            GemmArgs p = a;
            p.split_k = plan.slices;
            p.whole_tiles = 0;
            p.split_chunk = plan.tiles % 32 == 0 ? 32 : (int)plan.tiles;
            p.D = ws; p.C = nullptr; p.alpha = 1.f; p.beta = 0.f; p.out16 = 0; p.vec_store = 1;
            p.nt_store = store_policy == 1 || (store_policy == 0 && whole_lines(ws, (int64_t)N * 4) && count * 4 % LINE_BYTES == 0);
            e = launch(p, plan.grid);
            if (e == hipSuccess) {
                const unsigned blocks = (unsigned)((count + 255) / 256 < 65535 * 8 ? (count + 255) / 256 : 65535 * 8);
                const bool vec4 = !out16 && count % 4 == 0 && ((uintptr_t)D | (uintptr_t)(beta != 0.f ? C : nullptr)) % 16 == 0;
                const int slices = plan.slices;
                if (vec4) {
                    const long long count4 = count / 4;
                    const unsigned b4 = (unsigned)((count4 + 255) / 256 < 65535 * 8 ? (count4 + 255) / 256 : 65535 * 8);
                    hipLaunchKernelGGL(splitk_reduce4_kernel, dim3(b4), dim3(256), 0, s, reinterpret_cast<const f32x4*>(ws), slices, count4,
                                       static_cast<const f32x4*>(C), static_cast<f32x4*>(D), alpha, beta);
                } else if (!out16) hipLaunchKernelGGL((splitk_reduce_kernel<0, false>), dim3(blocks), dim3(256), 0, s, ws, slices, count, C, D, alpha, beta);
                else if (dtype == CK_DT_F16) hipLaunchKernelGGL((splitk_reduce_kernel<1, false>), dim3(blocks), dim3(256), 0, s, ws, slices, count, C, D, alpha, beta);
                else hipLaunchKernelGGL((splitk_reduce_kernel<1, true>), dim3(blocks), dim3(256), 0, s, ws, slices, count, C, D, alpha, beta);
                e = hipGetLastError();
            }
            if (!scratch_release(sc, ws, s) && e == hipSuccess) e = hipErrorUnknown;
        }
    } else if (t.num_producer_waves == 0 && t.num_stages == 1) {
        // one stage, no producers: load, barrier, multiply, barrier (the synchronous A/B partner)
        e = dtype == CK_DT_F16 ? launch_gemm_sync_f16(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), lds, s, a)
                               : launch_gemm_sync_bf16(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), lds, s, a);
    } else if (t.num_producer_waves == 0) {
        e = dtype == CK_DT_F16 ? launch_gemm_fused_f16(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), lds, s, a)
                               : launch_gemm_fused_bf16(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), lds, s, a);
    } else if (mode == CK_SYNC_TILE && t.num_stages >= 2 && opt[OPT_TILE_SYNC_BARRIER] && !a.single_producer && t.segment_dim_k <= 128) {
        // tile granularity through the workgroup barrier: the ring is the whole LDS allocation
        const size_t ring = (size_t)t.num_stages * 2 * stage_bytes_one_operand(t.tile_dim, t.segment_dim_k);
        e = dtype == CK_DT_F16 ? launch_gemm_pcb_f16(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, ring, s, a)
                               : launch_gemm_pcb_bf16(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, ring, s, a);
    } else if (dtype == CK_DT_F16) {
        if (mode == 0) e = launch_gemm_pc_f16_m0(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, lds, s, a);
        if (mode == 1) e = launch_gemm_pc_f16_m1(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, lds, s, a);
        if (mode == 2) e = launch_gemm_pc_f16_m2(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, lds, s, a);
    } else {
        if (mode == 0) e = launch_gemm_pc_bf16_m0(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, lds, s, a);
        if (mode == 1) e = launch_gemm_pc_bf16_m1(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, lds, s, a);
        if (mode == 2) e = launch_gemm_pc_bf16_m2(t.tile_dim, t.segment_dim_k, t.num_consumer_waves, dim3(grid), block, lds, s, a);
    }
    if (e == hipErrorInvalidValue) return CK_ERR_NO_INSTANCE;
    return e == hipSuccess ? CK_OK : CK_ERR_HIP;
}

}  // namespace

extern "C" {

#define CK_TUNING_PARAMS int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a, int bar_step_rows_b, \
                         int tile_group_m, int num_stages, int num_producer_waves, int num_consumer_waves, int num_cus
#define CK_TUNING_VALUE ck::GemmTuning{tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b, tile_group_m, \
                                       num_stages, num_producer_waves, num_consumer_waves, num_cus, 0}

int ckopt_launch_options_init(ckopt_launch_options* options) {
    if (!options) return ck::CK_ERR_NULL;
    const Options o = default_options();
    options->struct_bytes = (int)sizeof(ckopt_launch_options);
    int* f = &options->lds_swizzle;
    for (int k = 0; k < NUM_OPTIONS; ++k) f[k] = o.v[k];
    return ck::CK_OK;
}

int ckopt_gemm_shmem_tc_async_opt_port_2(int dtype, const void* A, const void* Bt, const float* C, float* D, float alpha, float beta,
                                         int M, int N, int K, CK_TUNING_PARAMS, void* stream) {
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, CK_TUNING_VALUE, default_options(), stream, 0, Scratch{Scratch::ALLOCATE, nullptr, 0});
}

int ckopt_gemm_shmem_tc_async_opt_port_2_lp(int dtype, const void* A, const void* Bt, const void* C, void* D, float alpha, float beta,
                                            int M, int N, int K, CK_TUNING_PARAMS, void* stream) {
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, CK_TUNING_VALUE, default_options(), stream, 1, Scratch{Scratch::ALLOCATE, nullptr, 0});
}

int ckopt_gemm_shmem_tc_async_opt_port_2_noalloc(int dtype, const void* A, const void* Bt, const float* C, float* D, float alpha, float beta,
                                                 int M, int N, int K, CK_TUNING_PARAMS, void* stream) {
    unsigned char* ptr = nullptr;
    const int rc = static_scratch_for_current_device(&ptr);
    if (rc != ck::CK_OK) return rc;
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, CK_TUNING_VALUE, default_options(), stream, 0,
                       Scratch{Scratch::PROVIDED, reinterpret_cast<char*>(ptr), (size_t)CKOPT_NOALLOC_SCRATCH_BYTES});
}

int ckopt_gemm_shmem_tc_async_opt_port_2_ex(int dtype, int cd_dtype, const void* A, const void* Bt, const void* C, void* D, float alpha,
                                            float beta, int M, int N, int K, CK_TUNING_PARAMS, const ckopt_launch_options* options,
                                            void* workspace, size_t workspace_bytes, void* stream) {
    Options opt;
    const int orc = options_from_public(options, &opt);
    if (orc != ck::CK_OK) return orc;
    if (!(cd_dtype == ck::CK_DT_F32 || cd_dtype == dtype)) return ck::CK_ERR_BAD_PARAM;
    const Scratch sc = workspace ? Scratch{Scratch::PROVIDED, static_cast<char*>(workspace), workspace_bytes} : Scratch{Scratch::ALLOCATE, nullptr, 0};
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, CK_TUNING_VALUE, opt, stream, cd_dtype == ck::CK_DT_F32 ? 0 : 1, sc);
}

int64_t ckopt_gemm_workspace_bytes_ex(int M, int N, int K, int operands_aligned, CK_TUNING_PARAMS, const ckopt_launch_options* options) {
    Options opt;
    const int orc = options_from_public(options, &opt);
    if (orc != ck::CK_OK) return orc;
    const ck::GemmTuning t = CK_TUNING_VALUE;
    if (M <= 0 || N <= 0 || K <= 0) return ck::CK_ERR_BAD_PARAM;
    const int rc = ck::check_gemm_tuning(t);
    if (rc != ck::CK_OK) return rc;
    const size_t need = scratch_need(M, N, K, operands_aligned != 0, t, opt);
    return need ? (int64_t)(need + SCRATCH_ALIGN) : 0;  // room to start on a 256-byte boundary inside any buffer
}
int64_t ckopt_gemm_workspace_bytes(int M, int N, int K, int operands_aligned, CK_TUNING_PARAMS) {
    return ckopt_gemm_workspace_bytes_ex(M, N, K, operands_aligned, tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
                                         bar_step_rows_b, tile_group_m, num_stages, num_producer_waves, num_consumer_waves, num_cus, nullptr);
}

int ckopt_gemm_launch_plan_ex(int M, int N, int K, int operands_aligned, CK_TUNING_PARAMS, const ckopt_launch_options* options, int* plan_out) {
    Options opt;
    const int orc = options_from_public(options, &opt);
    if (orc != ck::CK_OK) return orc;
    const ck::GemmTuning t = CK_TUNING_VALUE;
    if (!plan_out) return ck::CK_ERR_NULL;
    if (M <= 0 || N <= 0 || K <= 0) return ck::CK_ERR_BAD_PARAM;
    const int rc = ck::check_gemm_tuning(t);
    if (rc != ck::CK_OK) return rc;
    const bool copies = needs_copies(K, operands_aligned != 0);
    plan_out[0] = 0; plan_out[1] = t.tile_dim; plan_out[2] = 1; plan_out[3] = copies ? 1 : 0;
    plan_out[4] = 0; plan_out[5] = 0; plan_out[6] = 0;
    if (straight_line_tuple(t, opt)) {
        const StreamPlan plan = stream_plan(M, N, launch_k(K, operands_aligned != 0, t, opt), t.num_cus, opt);
        plan_out[0] = 1;
        plan_out[1] = plan.tile_n;
        plan_out[2] = plan.slices;
        plan_out[4] = (int)(plan.tiles - plan.whole_tiles);
        plan_out[5] = plan.slices > 1 && plan.fused ? 1 : 0;
        plan_out[6] = plan.grid;
    }
    return ck::CK_OK;
}
int ckopt_gemm_launch_plan(int M, int N, int K, int operands_aligned, CK_TUNING_PARAMS, int* plan_out) {
    return ckopt_gemm_launch_plan_ex(M, N, K, operands_aligned, tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a,
                                     bar_step_rows_b, tile_group_m, num_stages, num_producer_waves, num_consumer_waves, num_cus, nullptr, plan_out);
}

int ckopt_gemm_shmem_tc_async_opt_port_2_ws(int dtype, int cd_dtype, const void* A, const void* Bt, const void* C, void* D, float alpha,
                                            float beta, int M, int N, int K, CK_TUNING_PARAMS, void* workspace, size_t workspace_bytes,
                                            void* stream) {
    if (!(cd_dtype == ck::CK_DT_F32 || cd_dtype == dtype)) return ck::CK_ERR_BAD_PARAM;
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, CK_TUNING_VALUE, default_options(), stream, cd_dtype == ck::CK_DT_F32 ? 0 : 1,
                       Scratch{Scratch::PROVIDED, static_cast<char*>(workspace), workspace ? workspace_bytes : 0});
}

// port_1: every wave tile (or every 16-row block) has its own signal = port_2 with maximal bar_steps
static int launch_port_1(int dtype, const void* A, const void* Bt, const void* C, void* D, float alpha, float beta, int M, int N, int K,
                         int tile_dim, int segment_dim_k, int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                         int num_producer_waves, int num_consumer_waves, int num_cus, void* stream, int out16) {
    if (!(num_consumer_waves == 4 || num_consumer_waves == 8) || !(tile_dim == 64 || tile_dim == 128 || tile_dim == 256))
        return ck::CK_ERR_BAD_PARAM;
    const int mode = ck::sync_mode_of(tile_dim, num_consumer_waves, bar_step_rows_a, bar_step_rows_b);
    int sa = 0, sb = 0;
    if (mode == ck::CK_SYNC_WAVE) { sa = num_consumer_waves / 2; sb = 2; }
    if (mode == ck::CK_SYNC_ACC) {
        sa = ck::wave_tile_rows(tile_dim, num_consumer_waves) - 1;
        sb = ck::wave_tile_cols(tile_dim, num_consumer_waves) - 1;
    }
    const ck::GemmTuning t{tile_dim, segment_dim_k, sa, sb, bar_step_rows_a, bar_step_rows_b,
                           tile_group_m, num_stages, num_producer_waves, num_consumer_waves, num_cus, 0};
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, t, default_options(), stream, out16, Scratch{Scratch::ALLOCATE, nullptr, 0});
}
int ckopt_gemm_shmem_tc_async_opt_port_1(int dtype, const void* A, const void* Bt, const float* C, float* D,
                                         float alpha, float beta, int M, int N, int K, int tile_dim,
                                         int segment_dim_k, int bar_step_rows_a, int bar_step_rows_b,
                                         int tile_group_m, int num_stages, int num_producer_waves,
                                         int num_consumer_waves, int num_cus, void* stream) {
    return launch_port_1(dtype, A, Bt, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_step_rows_a, bar_step_rows_b, tile_group_m,
                         num_stages, num_producer_waves, num_consumer_waves, num_cus, stream, 0);
}
int ckopt_gemm_shmem_tc_async_opt_port_1_lp(int dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim,
                                            int segment_dim_k, int bar_step_rows_a, int bar_step_rows_b,
                                            int tile_group_m, int num_stages, int num_producer_waves,
                                            int num_consumer_waves, int num_cus, void* stream) {
    return launch_port_1(dtype, A, Bt, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, bar_step_rows_a, bar_step_rows_b, tile_group_m,
                         num_stages, num_producer_waves, num_consumer_waves, num_cus, stream, 1);
}

// port_0: one signal pair per stage; its legal set also holds a single producer wave (port_0.cu:538)
static int launch_port_0(int dtype, const void* A, const void* Bt, const void* C, void* D, float alpha, float beta, int M, int N, int K,
                         int tile_dim, int segment_dim_k, int tile_group_m, int num_stages, int num_producer_waves, int num_consumer_waves,
                         int num_cus, void* stream, int out16) {
    const ck::GemmTuning t{tile_dim, segment_dim_k, 0, 0, tile_dim, tile_dim, tile_group_m, num_stages, num_producer_waves, num_consumer_waves,
                           num_cus, 1};
    return gemm_launch(dtype, A, Bt, C, D, alpha, beta, M, N, K, t, default_options(), stream, out16, Scratch{Scratch::ALLOCATE, nullptr, 0});
}
int ckopt_gemm_shmem_tc_async_opt_port_0(int dtype, const void* A, const void* Bt, const float* C, float* D,
                                         float alpha, float beta, int M, int N, int K, int tile_dim,
                                         int segment_dim_k, int tile_group_m, int num_stages,
                                         int num_producer_waves, int num_consumer_waves, int num_cus, void* stream) {
    return launch_port_0(dtype, A, Bt, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, tile_group_m, num_stages, num_producer_waves,
                         num_consumer_waves, num_cus, stream, 0);
}
int ckopt_gemm_shmem_tc_async_opt_port_0_lp(int dtype, const void* A, const void* Bt, const void* C, void* D,
                                            float alpha, float beta, int M, int N, int K, int tile_dim,
                                            int segment_dim_k, int tile_group_m, int num_stages,
                                            int num_producer_waves, int num_consumer_waves, int num_cus, void* stream) {
    return launch_port_0(dtype, A, Bt, C, D, alpha, beta, M, N, K, tile_dim, segment_dim_k, tile_group_m, num_stages, num_producer_waves,
                         num_consumer_waves, num_cus, stream, 1);
}

int ckopt_get_lds_req(int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b, int bar_step_rows_a,
                      int bar_step_rows_b, int num_stages, int num_consumer_waves) {
    if (!(tile_dim == 64 || tile_dim == 128 || tile_dim == 256) || !(num_consumer_waves == 4 || num_consumer_waves == 8) ||
        segment_dim_k <= 0 || segment_dim_k % 8 || num_stages < 1 || bar_steps_a < 0 || bar_steps_b < 0)
        return ck::CK_ERR_BAD_PARAM;
    const int r = ck::get_lds_req(tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b,
                                  num_stages, num_consumer_waves);
    return r < 0 ? ck::CK_ERR_BAD_PARAM : r;
}

int ckopt_get_num_acc(int tile_dim, int num_consumer_waves) {
    if (!(tile_dim == 64 || tile_dim == 128 || tile_dim == 256) || !(num_consumer_waves == 4 || num_consumer_waves == 8))
        return ck::CK_ERR_BAD_PARAM;
    return ck::get_num_acc(tile_dim, num_consumer_waves);
}

int ckopt_get_warp_tile_rows(int tile_dim, int num_consumer_waves) {
    if (!(tile_dim == 64 || tile_dim == 128 || tile_dim == 256) || !(num_consumer_waves == 4 || num_consumer_waves == 8))
        return ck::CK_ERR_BAD_PARAM;
    return ck::get_warp_tile_rows(tile_dim, num_consumer_waves);
}

int64_t ckopt_get_tile_offset_cd(int M, int N, int tile_dim, int tile_group_m, int64_t tile_count) {
    if (M <= 0 || N <= 0 || tile_dim <= 0 || tile_group_m <= 0 || tile_count < 0) return ck::CK_ERR_BAD_PARAM;
    return ck::get_tile_offset_cd(M, N, tile_dim, tile_group_m, tile_count);
}

int ckopt_check_gemm_tuning(int tile_dim, int segment_dim_k, int bar_steps_a, int bar_steps_b,
                            int bar_step_rows_a, int bar_step_rows_b, int tile_group_m, int num_stages,
                            int num_producer_waves, int num_consumer_waves, int num_cus) {
    const ck::GemmTuning t{tile_dim, segment_dim_k, bar_steps_a, bar_steps_b, bar_step_rows_a, bar_step_rows_b,
                           tile_group_m, num_stages, num_producer_waves, num_consumer_waves, num_cus, 0};
    return ck::check_gemm_tuning(t);
}

int ckopt_suggest_gemm_tuning(int M, int N, int K, int num_cus, int* tuning_out) {
    using namespace ck;
    if (!tuning_out) return CK_ERR_NULL;
    if (M <= 0 || N <= 0 || K <= 0 || num_cus <= 0) return CK_ERR_BAD_PARAM;
    const Options opt = default_options();
    auto tiles = [&](int t) { return (int64_t)((M + t - 1) / t) * ((N + t - 1) / t); };
    // {tile, seg_k, bar_steps_a, bar_steps_b, rows_a, rows_b, group, stages, producers, consumers}
    static const int straight_line[10] = {256, 32, 0, 0, 256, 256, 4, 5, 0, 8};
    static const int fused_128[10] = {128, 128, 0, 0, 128, 128, 4, 2, 0, 8};
    static const int fused_64[10] = {64, 128, 0, 0, 64, 64, 4, 4, 0, 8};
    static const int pc_256[10] = {256, 64, 0, 0, 256, 256, 4, 2, 2, 8};
    const int* pick = fused_64;
    const int64_t t256 = tiles(256);
    const bool straight_ok = opt[OPT_STRAIGHT_LINE] && opt[OPT_SWIZZLE];
    if (!straight_ok) {
        // without the straight-line kernel: the reference's design on 256 tiles when they fill half the device
        if (t256 * 2 >= num_cus) pick = pc_256;
        else if (tiles(128) * 2 >= num_cus) pick = fused_128;
    } else {
        // the shortest of three estimates: the straight-line kernel as the launcher would run it on aligned operands (its K,
        // tile width and slice count: launch_k, stream_plan), and the general kernel on 128 and on 64 tiles - one
        // workgroup per CU, measured per 128 of K: 1.4 us for a 128 x 128 tile, 0.65 us for a 64 x 64 tile, about 4 us
        // per round besides
        const GemmTuning st{256, 32, 0, 0, 256, 256, 4, 5, 0, 8, num_cus, 0};
        const double straight_us = stream_plan(M, N, launch_k(K, true, st, opt), num_cus, opt).us;
        auto general_us = [&](int t, double seg_us) { return std::ceil((double)tiles(t) / num_cus) * ((double)K / 128.0 * seg_us + 4.0); };
        const double us_128 = general_us(128, 1.4), us_64 = general_us(64, 0.65);
        if (straight_us <= us_128 && straight_us <= us_64) pick = straight_line;
        else if (us_128 <= us_64) pick = fused_128;
    }
    for (int i = 0; i < 10; ++i) tuning_out[i] = pick[i];
    return CK_OK;
}

int ckopt_matmul_shmem(int dtype, const void* A, const void* B, void* C, int M, int N, int K, int tile_dim,
                       int block_rows, int b_transposed, void* stream) {
    using namespace ck;
    if (!(dtype == CK_DT_F32 || dtype == CK_DT_F16 || dtype == CK_DT_I32)) return CK_ERR_BAD_PARAM;
    const int rc = check_simt_tuning(tile_dim, block_rows);
    if (rc != CK_OK) return rc;
    if (M <= 0 || N <= 0 || K <= 0) return CK_ERR_BAD_PARAM;
    if (M % tile_dim || N % tile_dim || K % SIMT_KT) return CK_ERR_BAD_PARAM;
    if (!A || !B || !C) return CK_ERR_NULL;
    if (((uintptr_t)A & 15) || ((uintptr_t)B & 15) || ((uintptr_t)C & 3)) return CK_ERR_ALIGNMENT;
    if (N / tile_dim > 65535) return CK_ERR_TOO_LARGE;
    SimtArgs a{A, B, C, M, N, K};
    const hipError_t e = launch_matmul_shmem(dtype, tile_dim, tile_dim / block_rows, b_transposed != 0,
                                             dim3(M / tile_dim, N / tile_dim), static_cast<hipStream_t>(stream), a);
    if (e == hipErrorInvalidValue) return CK_ERR_NO_INSTANCE;
    return e == hipSuccess ? CK_OK : CK_ERR_HIP;
}

int ckopt_matmul_shmem_lds_req(int dtype, int tile_dim) {
    if (!(dtype == ck::CK_DT_F32 || dtype == ck::CK_DT_F16 || dtype == ck::CK_DT_I32)) return ck::CK_ERR_BAD_PARAM;
    if (!(tile_dim == 32 || tile_dim == 64 || tile_dim == 128)) return ck::CK_ERR_BAD_PARAM;
    return ck::simt_lds_req(tile_dim, 4);
}

int ckopt_check_matmul_shmem_tuning(int tile_dim, int block_rows) { return ck::check_simt_tuning(tile_dim, block_rows); }

int ckopt_device_status(void* stream) {
    unsigned int* p = nullptr;
    const int rc = status_ptr_for_current_device(&p);
    if (rc != ck::CK_OK) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned int v = 0;
    if (hipStreamSynchronize(s) != hipSuccess) return ck::CK_ERR_HIP;
    if (hipMemcpyAsync(&v, p, sizeof(v), hipMemcpyDeviceToHost, s) != hipSuccess) return ck::CK_ERR_HIP;
    if (hipStreamSynchronize(s) != hipSuccess) return ck::CK_ERR_HIP;
    if (v != 0) {
        const unsigned int zero = 0;
        if (hipMemcpyAsync(p, &zero, sizeof(zero), hipMemcpyHostToDevice, s) != hipSuccess) return ck::CK_ERR_HIP;
        if (hipStreamSynchronize(s) != hipSuccess) return ck::CK_ERR_HIP;
    }
    return (int)(v & 0x7fffffffu);
}

int ckopt_last_launch_clocks(void* stream, uint64_t* shader_cycles, uint64_t* ref_ticks) {
    unsigned int* p = nullptr;
    const int rc = status_ptr_for_current_device(&p);
    if (rc != ck::CK_OK) return rc;
    if (!shader_cycles || !ref_ticks) return ck::CK_ERR_NULL;
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned int v[8] = {};
    if (hipStreamSynchronize(s) != hipSuccess) return ck::CK_ERR_HIP;
    if (hipMemcpyAsync(v, p, sizeof(v), hipMemcpyDeviceToHost, s) != hipSuccess) return ck::CK_ERR_HIP;
    if (hipStreamSynchronize(s) != hipSuccess) return ck::CK_ERR_HIP;
    *shader_cycles = (uint64_t)v[2] | ((uint64_t)v[3] << 32);
    *ref_ticks = (uint64_t)v[4] | ((uint64_t)v[5] << 32);
    return ck::CK_OK;
}

int ckopt_trim_scratch_pool(size_t keep_bytes) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEV) return ck::CK_ERR_HIP;
    hipMemPool_t pool = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_status_mutex);
        pool = g_scratch_pool[dev];
    }
    if (!pool) return ck::CK_OK;
    return hipMemPoolTrimTo(pool, keep_bytes) == hipSuccess ? ck::CK_OK : ck::CK_ERR_HIP;
}

int ckopt_set_option(int key, int value) {
    if (key < 0 || key >= NUM_OPTIONS) return ck::CK_ERR_BAD_PARAM;
    if (OPTION_RULES[key].hi == 1) value = value != 0;   // switches take any non-zero value as on
    if (value < OPTION_RULES[key].lo || value > OPTION_RULES[key].hi) return ck::CK_ERR_BAD_PARAM;
    return g_option[key].exchange(value);
}

const char* ckopt_error_string(int code) {
    switch (code) {
        case ck::CK_OK: return "ok";
        case ck::CK_ERR_BAD_PARAM: return "parameter outside the legal set";
        case ck::CK_ERR_LDS_BUDGET: return "LDS ring exceeds 160 KiB";
        case ck::CK_ERR_NO_INSTANCE: return "no kernel instance compiled for this tuple";
        case ck::CK_ERR_HIP: return "HIP runtime error";
        case ck::CK_ERR_ALIGNMENT: return "pointer or row pitch misaligned";
        case ck::CK_ERR_NULL: return "required pointer is NULL";
        case ck::CK_ERR_TOO_LARGE: return "size exceeds what the entry point supports";
        default: return "unknown error";
    }
}

}  // extern "C"

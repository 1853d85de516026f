// Launchers of the straight-line kernel (one instance per element type, schedule, K-tail form and tile width).
#include <atomic>
#include "gemm_stream_kernel.hip.h"

namespace ck {

static_assert(STREAM_K_MULTIPLE == 64, "the host's slice rule assumes loop bodies of 64");

template <typename DT, bool ODD_ONLY, bool KTAIL, int WTC>
static hipError_t stream_launch_one(dim3 grid, hipStream_t stream, const GemmArgs& a) {
    auto kern = gemm_stream_kernel<DT, ODD_ONLY, KTAIL, WTC>;
    constexpr int lds_bytes = stream_lds_bytes(2 * WTC * 16);   // (this file holds the 256- and 128-wide instances; gemm_stream_inst_w6.hip the 192-wide ones)
    static std::atomic<bool> opted[64] = {};   // (threads may launch at once; setting the attribute twice is harmless)
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || !opted[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES_PER_CU);
        if (e != hipSuccess) return e;
        if (dev >= 0 && dev < 64) opted[dev].store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, grid, dim3(512), lds_bytes, stream, a);
    return hipGetLastError();
}

// K in whole loop bodies: the plain instance; otherwise (K a multiple of 8) the one whose last body masks the end of K
template <typename DT, bool ODD_ONLY, int WTC>
static hipError_t stream_launch_k(dim3 grid, hipStream_t stream, const GemmArgs& a) {
    return a.K % STREAM_K_MULTIPLE == 0 ? stream_launch_one<DT, ODD_ONLY, false, WTC>(grid, stream, a) : stream_launch_one<DT, ODD_ONLY, true, WTC>(grid, stream, a);
}
hipError_t launch_gemm_stream_w6(bool bf16, bool odd_only, dim3 grid, hipStream_t stream, const GemmArgs& a);   // gemm_stream_inst_w6.hip
template <typename DT, bool ODD_ONLY>
static hipError_t stream_launch(dim3 grid, hipStream_t stream, const GemmArgs& a, int tile_n) {
    if (tile_n == STREAM_TILE_N_THREE_QUARTERS) return launch_gemm_stream_w6(std::is_same<DT, bf16_tag>::value, ODD_ONLY, grid, stream, a);
    return tile_n == STREAM_TILE_N_HALF ? stream_launch_k<DT, ODD_ONLY, 4>(grid, stream, a) : stream_launch_k<DT, ODD_ONLY, 8>(grid, stream, a);
}

// barrier_every_kstep selects the schedule with a barrier in both k-steps of a loop body; tile_n the tile width: 256,
// 192 or 128 columns (a.tiles_n counts tiles of that width)
hipError_t launch_gemm_stream_f16(dim3 grid, hipStream_t stream, const GemmArgs& a, bool barrier_every_kstep, int tile_n) {
    return barrier_every_kstep ? stream_launch<f16_tag, false>(grid, stream, a, tile_n) : stream_launch<f16_tag, true>(grid, stream, a, tile_n);
}
hipError_t launch_gemm_stream_bf16(dim3 grid, hipStream_t stream, const GemmArgs& a, bool barrier_every_kstep, int tile_n) {
    return barrier_every_kstep ? stream_launch<bf16_tag, false>(grid, stream, a, tile_n) : stream_launch<bf16_tag, true>(grid, stream, a, tile_n);
}

// what the kernel assumes about a launch (the caller falls back to the general fused kernel otherwise)
bool gemm_stream_applies(const GemmArgs& a, int tile_dim, int segment_dim_k, int num_stages, int producer_waves, int consumer_waves) {
    return producer_waves == 0 && consumer_waves == 8 && tile_dim == STREAM_TILE && segment_dim_k == STREAM_SEGK &&
           num_stages == STREAM_STAGES && a.K % CHUNK_ELEMS == 0 && a.swizzle;
}

}  // namespace ck

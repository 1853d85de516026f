// Launchers of the straight-line kernel's 256 x 192 tile form (wave tiles of 64 x 96), in a translation unit of their own
// so that they compile next to the other widths.
#include <atomic>
#include "gemm_stream_kernel.hip.h"

namespace ck {

template <typename DT, bool ODD_ONLY, bool KTAIL>
static hipError_t stream_w6_launch_one(dim3 grid, hipStream_t stream, const GemmArgs& a) {
    auto kern = gemm_stream_kernel<DT, ODD_ONLY, KTAIL, 6>;
    constexpr int lds_bytes = stream_lds_bytes(STREAM_TILE_N_THREE_QUARTERS);
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
template <typename DT, bool ODD_ONLY>
static hipError_t stream_w6_launch_k(dim3 grid, hipStream_t stream, const GemmArgs& a) {
    return a.K % STREAM_K_MULTIPLE == 0 ? stream_w6_launch_one<DT, ODD_ONLY, false>(grid, stream, a) : stream_w6_launch_one<DT, ODD_ONLY, true>(grid, stream, a);
}

hipError_t launch_gemm_stream_w6(bool bf16, bool odd_only, dim3 grid, hipStream_t stream, const GemmArgs& a) {
    if (bf16) return odd_only ? stream_w6_launch_k<bf16_tag, true>(grid, stream, a) : stream_w6_launch_k<bf16_tag, false>(grid, stream, a);
    return odd_only ? stream_w6_launch_k<f16_tag, true>(grid, stream, a) : stream_w6_launch_k<f16_tag, false>(grid, stream, a);
}

}  // namespace ck

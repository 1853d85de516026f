// Launchers of the synchronous single-stage kernel (the no-pipeline, no-specialisation A/B partner).
#include <atomic>
#include "gemm_sync_kernel.hip.h"

namespace ck {

template <typename DT, int TILE, int SEGK, int CW>
static hipError_t sync_launch_one(dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a) {
    auto kern = gemm_sync_kernel<DT, TILE, SEGK, CW>;
    static std::atomic<bool> opted[64] = {};   // (threads may launch at once; setting the attribute twice is harmless)
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= 64 || !opted[dev].load(std::memory_order_acquire)) {
        e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES_PER_CU);
        if (e != hipSuccess) return e;
        if (dev >= 0 && dev < 64) opted[dev].store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(kern, grid, dim3(CW * WAVE), lds, stream, a);
    return hipGetLastError();
}

template <typename DT, int TILE, int CW>
static hipError_t sync_launch_segk(int segk, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a) {
    switch (segk) {
        case 32: return sync_launch_one<DT, TILE, 32, CW>(grid, lds, stream, a);
        case 64: return sync_launch_one<DT, TILE, 64, CW>(grid, lds, stream, a);
        case 128: return sync_launch_one<DT, TILE, 128, CW>(grid, lds, stream, a);
        default: return hipErrorInvalidValue;
    }
}

template <typename DT>
static hipError_t sync_launch(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a) {
    if (tile == 64 && cw == 4) return sync_launch_segk<DT, 64, 4>(segk, grid, lds, stream, a);
    if (tile == 64 && cw == 8) return sync_launch_segk<DT, 64, 8>(segk, grid, lds, stream, a);
    if (tile == 128 && cw == 4) return sync_launch_segk<DT, 128, 4>(segk, grid, lds, stream, a);
    if (tile == 128 && cw == 8) return sync_launch_segk<DT, 128, 8>(segk, grid, lds, stream, a);
    if (tile == 256 && cw == 8) return sync_launch_segk<DT, 256, 8>(segk, grid, lds, stream, a);
    return hipErrorInvalidValue;
}

hipError_t launch_gemm_sync_f16(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a) {
    return sync_launch<f16_tag>(tile, segk, cw, grid, lds, stream, a);
}
hipError_t launch_gemm_sync_bf16(int tile, int segk, int cw, dim3 grid, size_t lds, hipStream_t stream, const GemmArgs& a) {
    return sync_launch<bf16_tag>(tile, segk, cw, grid, lds, stream, a);
}

}  // namespace ck

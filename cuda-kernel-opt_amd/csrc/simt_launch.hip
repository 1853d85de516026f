// Instance table and dispatch of the matmul_shmem (SIMT) kernel.
#include "simt_kernel.hip.h"

namespace ck {

template <typename DT, int TILE, int RM, int RN>
static hipError_t simt_launch_one(bool bt, dim3 grid, hipStream_t stream, const SimtArgs& a) {
    constexpr int NT = TILE * TILE / (RM * RN);
    const size_t lds = simt_lds_req(TILE, 4);
    if (bt) hipLaunchKernelGGL((matmul_shmem_kernel<DT, TILE, RM, RN, true>), grid, dim3(NT), lds, stream, a);
    else hipLaunchKernelGGL((matmul_shmem_kernel<DT, TILE, RM, RN, false>), grid, dim3(NT), lds, stream, a);
    return hipGetLastError();
}

template <typename DT>
static hipError_t simt_dispatch(int tile, int accs, bool bt, dim3 grid, hipStream_t s, const SimtArgs& a) {
#define CK_SIMT_CASE(T, ACCS, RM, RN) if (tile == T && accs == ACCS) return simt_launch_one<DT, T, RM, RN>(bt, grid, s, a);
    CK_SIMT_CASE(32, 1, 1, 1) CK_SIMT_CASE(32, 2, 2, 1) CK_SIMT_CASE(32, 4, 2, 2) CK_SIMT_CASE(32, 8, 4, 2) CK_SIMT_CASE(32, 16, 4, 4)
    CK_SIMT_CASE(64, 4, 2, 2) CK_SIMT_CASE(64, 8, 4, 2) CK_SIMT_CASE(64, 16, 4, 4) CK_SIMT_CASE(64, 32, 8, 4) CK_SIMT_CASE(64, 64, 8, 8)
    CK_SIMT_CASE(128, 16, 4, 4) CK_SIMT_CASE(128, 32, 8, 4) CK_SIMT_CASE(128, 64, 8, 8)
#undef CK_SIMT_CASE
    return hipErrorInvalidValue;
}

hipError_t launch_matmul_shmem(int dtype, int tile, int accs, bool bt, dim3 grid, hipStream_t s, const SimtArgs& a) {
    switch (dtype) {
        case CK_DT_F32: return simt_dispatch<float>(tile, accs, bt, grid, s, a);
        case CK_DT_I32: return simt_dispatch<int>(tile, accs, bt, grid, s, a);
        case CK_DT_F16: return simt_dispatch<_Float16>(tile, accs, bt, grid, s, a);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace ck

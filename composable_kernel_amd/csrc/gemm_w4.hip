// Launchers of the four-wave 256 x 256 tile kernel (gemm_w4.hpp): the second body behind tile instance 0.
#include "gemm_w4.hpp"
#include "tile_launch.hpp"

#include <mutex>

namespace ckx {
namespace {

template <int DT, bool FUSED = false, int EPI = EPI_PASSTHROUGH>
hipError_t launch_w4(const GemmArgs& a, int tiles, hipStream_t s)
{
    using T    = GemmW4<DT, FUSED, EPI>;
    auto* kern = &gemm_w4_kernel<DT, FUSED, EPI>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    // one workgroup per CU (128 KB of LDS), a multiple of 8 so that workgroup b stays on XCD b % 8 over its tiles
    int grid = num_cus();
    grid -= grid % 8;
    grid = tiles < grid ? tiles : grid;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::NT), T::LDS, s, a);
    return hipGetLastError();
}

// int8: one kernel per plain epilogue (the requant form is a compile-time constant of the kernel)
hipError_t launch_w4_i8(const GemmArgs& a, int tiles, hipStream_t s)
{
    return a.epi == EPI_REQUANT_RND  ? launch_w4<DT_I8, false, EPI_REQUANT_RND>(a, tiles, s)
           : a.epi == EPI_REQUANT_CK ? launch_w4<DT_I8, false, EPI_REQUANT_CK>(a, tiles, s)
                                     : launch_w4<DT_I8, false, EPI_PASSTHROUGH>(a, tiles, s);
}

} // namespace

tile_launch_fn w4_tile(int dt, bool fused)
{
    if(fused)
        return dt == DT_F16 ? &launch_w4<DT_F16, true> : nullptr;
    return dt == DT_I8 ? &launch_w4_i8 : dt == DT_BF16 ? &launch_w4<DT_BF16> : &launch_w4<DT_F16>;
}

} // namespace ckx

// Launchers of the four-wave 256 x 256 tile kernel (gemm_w4.hpp): the second body behind tile instance 0.
#include "gemm_w4.hpp"
#include "tile_launch.hpp"

#include <mutex>

namespace ckx {
namespace {

template <int DT, bool FUSED = false>
hipError_t launch_w4(const GemmArgs& a, int tiles, hipStream_t s)
{
    using T    = GemmW4<DT, FUSED>;
    auto* kern = &gemm_w4_kernel<DT, FUSED>;
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

} // namespace

tile_launch_fn w4_tile(int dt, bool fused)
{
    if(fused)
        return dt == DT_F16 ? &launch_w4<DT_F16, true> : nullptr;
    return dt == DT_I8 ? &launch_w4<DT_I8> : dt == DT_BF16 ? &launch_w4<DT_BF16> : &launch_w4<DT_F16>;
}

} // namespace ckx

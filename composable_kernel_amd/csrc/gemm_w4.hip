// Launchers of the four-wave 256 x 256 tile kernel (gemm_w4.hpp): the second body behind tile instance 0.
#include "gemm_w4.hpp"
#include "tile_launch.hpp"

#include <mutex>

namespace ckx {
namespace {

template <int DT>
hipError_t launch_w4(const GemmArgs& a, int tiles, hipStream_t s)
{
    auto* kern = &gemm_w4_kernel<DT>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       GemmW4<DT>::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    // one workgroup per CU (128 KB of LDS), a multiple of 8 so that workgroup b stays on XCD b % 8 over its tiles
    int grid = num_cus();
    grid -= grid % 8;
    grid = tiles < grid ? tiles : grid;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(GemmW4<DT>::NT), GemmW4<DT>::LDS, s, a);
    return hipGetLastError();
}

} // namespace

tile_launch_fn w4_tile(int dt)
{
    return dt == DT_I8 ? &launch_w4<DT_I8> : dt == DT_BF16 ? &launch_w4<DT_BF16> : &launch_w4<DT_F16>;
}

} // namespace ckx

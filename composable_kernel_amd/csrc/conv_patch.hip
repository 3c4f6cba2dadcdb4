// Launchers of the input-patch conv kernels (conv_patch.hpp, conv_patch_wide.hpp): a translation unit of its own so that it compiles beside the others.
#include "conv_patch.hpp"
#include "conv_patch_wide.hpp"
#include "tile_launch.hpp"

#include <mutex>

namespace ckx {
namespace {

template <int DT, bool FUSED>
hipError_t launch_one(const ConvPatchArgs& a, hipStream_t s)
{
    using T    = ConvPatch<DT, 7, FUSED>;
    auto* kern = &conv_patch_kernel<DT, 7, FUSED>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    // a workgroup owns whole images
    const int grid = a.N < num_cus() ? a.N : num_cus();
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::NT), T::LDS, s, a);
    return hipGetLastError();
}

template <int DT, bool FUSED>
hipError_t launch_wide(const ConvPatchArgs& a, hipStream_t s)
{
    using T    = ConvPatchWide<DT, FUSED>;
    auto* kern = &conv_patch_wide_kernel<DT, FUSED>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    const int grid = a.N < num_cus() ? a.N : num_cus();
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::NT), T::LDS, s, a);
    return hipGetLastError();
}

} // namespace

hipError_t launch_conv_patch_wide(int dt, bool fused, const ConvPatchArgs& a, hipStream_t s)
{
    return dt == DT_I8 ? launch_wide<DT_I8, false>(a, s) : (fused ? launch_wide<DT_F16, true>(a, s) : launch_wide<DT_F16, false>(a, s));
}

hipError_t launch_conv_patch(int dt, bool fused, const ConvPatchArgs& a, hipStream_t s)
{
    return dt == DT_I8 ? (fused ? launch_one<DT_I8, true>(a, s) : launch_one<DT_I8, false>(a, s))
                       : (fused ? launch_one<DT_F16, true>(a, s) : launch_one<DT_F16, false>(a, s));
}

} // namespace ckx

// Launchers of the weight-streaming GEMM for up to 128 rows (gemm_astream.hpp): instances of the skinny family.
#include "gemm_astream.hpp"
#include "tile_launch.hpp"

#include <mutex>

namespace ckx {
namespace {

template <int DT, int MT, int NT>
hipError_t launch_astream(const GemmArgs& a, int grid, hipStream_t s)
{
#ifndef CKX_ASTREAM_RB
#define CKX_ASTREAM_RB 4
#endif
    using T    = GemmAStream<DT, MT, NT, CKX_ASTREAM_RB>;
    auto* kern = &gemm_astream_kernel<DT, MT, NT, CKX_ASTREAM_RB>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::NTHR), T::LDS, s, a);
    return hipGetLastError();
}

} // namespace

tile_launch_fn astream_launcher(int dt, int nt)
{
    if(nt != 3)
        return nullptr;
    return dt == DT_I8 ? &launch_astream<DT_I8, 8, 3> : dt == DT_BF16 ? &launch_astream<DT_BF16, 8, 3> : &launch_astream<DT_F16, 8, 3>;
}

} // namespace ckx

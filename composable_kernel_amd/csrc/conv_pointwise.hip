// Instantiations and launch of the weight-stationary pointwise conv kernel. A translation unit of its own
// so that it compiles next to ckx_api.hip.
#include "conv_pointwise.hpp"
#include "tile_launch.hpp"

namespace ckx {
namespace {

template <int DT, int KS, bool FUSED>
hipError_t launch_pw(const ConvPointwiseArgs& a, hipStream_t s)
{
    constexpr int MT = 16 / KS; // 16 KB ring slots
    using T          = ConvPointwise<DT, KS, MT, FUSED>;
    auto* kern       = &conv_pointwise_kernel<DT, KS, MT, FUSED>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    // one workgroup per CU and 512-channel block; every workgroup takes a contiguous run of bands
    const int nblk  = a.Kout / T::NWG;
    const long bands = ((long)a.M + T::MB - 1) / T::MB;
    int gx          = num_cus() / nblk;
    gx              = gx < 1 ? 1 : gx;
    gx              = bands < gx ? (int)bands : gx;
    hipLaunchKernelGGL(kern, dim3(gx, nblk), dim3(T::NT), T::LDS, s, a);
    return hipGetLastError();
}

} // namespace

hipError_t launch_conv_pointwise(int dt, int pixel_bytes, bool fused, const ConvPointwiseArgs& a, hipStream_t s)
{
    // one requant scale per output channel: 16 more registers per lane, which the 512-byte-pixel kernel (128 weight
    // registers) does not have -- the caller sends those layers to the tile instances
    if(dt == DT_I8 && fused)
        return pixel_bytes == 256 ? launch_pw<DT_I8, 4, true>(a, s) : hipErrorInvalidValue;
    if(dt == DT_I8)
        return pixel_bytes == 256 ? launch_pw<DT_I8, 4, false>(a, s) : launch_pw<DT_I8, 8, false>(a, s);
    if(pixel_bytes == 256)
        return fused ? launch_pw<DT_F16, 4, true>(a, s) : launch_pw<DT_F16, 4, false>(a, s);
    return fused ? launch_pw<DT_F16, 8, true>(a, s) : launch_pw<DT_F16, 8, false>(a, s);
}

} // namespace ckx

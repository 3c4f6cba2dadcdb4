// The streaming 1x1 conv kernel for short pixels (conv_rows.hpp), a translation unit of its own.
#include "conv_rows.hpp"

#include "tile_launch.hpp"

namespace ckx {

template <int DT, int KS, int NG, bool FUSED>
static hipError_t launch_rows(const ConvRowsArgs& a, hipStream_t s)
{
    constexpr int U  = KS >= 8 ? 1 : 2;
    const int groups = ((a.M + 15) / 16 + U - 1) / U;
    // four workgroups of four waves per CU at most; fewer when the rows do not give every wave two groups
    int wgs = num_cus() * 4;
    if(wgs > (groups + 7) / 8)
        wgs = (groups + 7) / 8;
    if(wgs < 1)
        wgs = 1;
    const int kblocks = (a.Kout + 64 * NG - 1) / (64 * NG);
    hipLaunchKernelGGL((conv_rows_kernel<DT, KS, NG, FUSED>), dim3(wgs, kblocks), dim3(256), 0, s, a);
    return hipGetLastError();
}

template <int DT, bool FUSED>
static hipError_t launch_rows_dt(int pixel_bytes, const ConvRowsArgs& a, hipStream_t s)
{
    const int ng = a.Kout <= 64 ? 1 : a.Kout <= 128 ? 2 : 4;
    if(pixel_bytes == 64)
        return ng == 1 ? launch_rows<DT, 1, 1, FUSED>(a, s) : ng == 2 ? launch_rows<DT, 1, 2, FUSED>(a, s) : launch_rows<DT, 1, 4, FUSED>(a, s);
    if(pixel_bytes == 128)
        return ng == 1 ? launch_rows<DT, 2, 1, FUSED>(a, s) : ng == 2 ? launch_rows<DT, 2, 2, FUSED>(a, s) : launch_rows<DT, 2, 4, FUSED>(a, s);
    // 256-byte pixels: up to 128 output channels (their weights are 64 / 128 registers); 512-byte pixels: 64
    if(pixel_bytes == 256)
        return ng == 1 ? launch_rows<DT, 4, 1, FUSED>(a, s) : launch_rows<DT, 4, 2, FUSED>(a, s);
    return launch_rows<DT, 8, 1, FUSED>(a, s);
}

hipError_t launch_conv_rows(int dt, int pixel_bytes, bool fused, const ConvRowsArgs& a, hipStream_t s)
{
    if((pixel_bytes != 64 && pixel_bytes != 128 && pixel_bytes != 256 && pixel_bytes != 512) || a.Kout % 64 ||
       (a.Kout > 256 && a.Kout % 256) || (pixel_bytes == 256 && a.Kout > 128) || (pixel_bytes == 512 && a.Kout > 64))
        return hipErrorInvalidValue;
    if(dt == DT_I8)
        return fused ? hipErrorInvalidValue : launch_rows_dt<DT_I8, false>(pixel_bytes, a, s);
    return fused ? launch_rows_dt<DT_F16, true>(pixel_bytes, a, s) : launch_rows_dt<DT_F16, false>(pixel_bytes, a, s);
}

} // namespace ckx

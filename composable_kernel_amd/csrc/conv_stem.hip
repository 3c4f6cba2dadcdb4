// Launcher of the stem conv kernel (conv_stem.hpp): a translation unit of its own so that it compiles beside the others.
#include "conv_stem.hpp"
#include "tile_launch.hpp"

#include <mutex>

namespace ckx {
namespace {

template <int DT>
hipError_t launch_one(const ConvStemArgs& a, hipStream_t s)
{
    using T       = ConvStem<DT>;
    auto* kern    = &conv_stem_kernel<DT>;
    const int lds = T::lds_bytes(a.Wo);
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    // bands of TH output rows, walked by two (fp16) or three (int8) workgroups per CU (their registers hold the weights)
    const long units = (long)a.N * ((a.Ho + T::TH - 1) / T::TH);
    int per_cu       = 160 * 1024 / lds;
    per_cu           = per_cu > (DT == DT_I8 ? 3 : 2) ? (DT == DT_I8 ? 3 : 2) : per_cu;
    long grid        = (long)num_cus() * per_cu;
    grid             = units < grid ? units : grid;
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(T::NTHR), lds, s, a);
    return hipGetLastError();
}

} // namespace

hipError_t launch_conv_stem(int dt, const ConvStemArgs& a, hipStream_t s)
{
    return dt == DT_I8 ? launch_one<DT_I8>(a, s) : launch_one<DT_F16>(a, s);
}

} // namespace ckx

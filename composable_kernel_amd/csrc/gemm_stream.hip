// Instances and launcher of the weight-streaming GEMM (a translation unit of its own: compiled beside the others).
#include "gemm_stream.hpp"

#include <mutex>

namespace ckx {

namespace {

template <int DT, int MT, int NTW, int D>
hipError_t launch_one(const GemmArgs& a, hipStream_t s)
{
    using T    = GemmStream<DT, MT, NTW, D>;
    auto* kern = &gemm_stream_kernel<DT, MT, NTW, D>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    hipLaunchKernelGGL(kern, dim3((unsigned)(a.tiles_n * a.ksplit)), dim3(T::NT), T::LDS, s, a);
    return hipGetLastError();
}

template <int MT, int NTW, int D>
hipError_t launch_dt(int dt, const GemmArgs& a, hipStream_t s)
{
    return dt == DT_I8 ? launch_one<DT_I8, MT, NTW, D>(a, s)
           : dt == DT_BF16 ? launch_one<DT_BF16, MT, NTW, D>(a, s)
                           : launch_one<DT_F16, MT, NTW, D>(a, s);
}

} // namespace

const StreamInstance kStreamInstances[] = {
    {"MI355X_Mfma16_Stream<rows 64, cols 64, B in registers 4 K tiles ahead, waves 4>", 64, 64},
    {"MI355X_Mfma16_Stream<rows 64, cols 128, B in registers 4 K tiles ahead, waves 4>", 64, 128},
    {"MI355X_Mfma16_Stream<rows 128, cols 64, B in registers 4 K tiles ahead, waves 4>", 128, 64},
    {"MI355X_Mfma16_Stream<rows 128, cols 128, B in registers 4 K tiles ahead, waves 4>", 128, 128},
};
const int kNumStreamInstances = sizeof(kStreamInstances) / sizeof(kStreamInstances[0]);

hipError_t launch_stream(int dt, int which, const GemmArgs& a, hipStream_t s)
{
    switch(which)
    {
    case 0: return launch_dt<4, 1, 4>(dt, a, s);
    case 1: return launch_dt<4, 2, 4>(dt, a, s);
    case 2: return launch_dt<8, 1, 4>(dt, a, s);
    case 3: return launch_dt<8, 2, 4>(dt, a, s);
    default: return hipErrorInvalidValue;
    }
}

} // namespace ckx

// Launcher of the element-granular GEMM / conv instance (a translation unit of its own so that its six kernels
// compile beside the others).
#include "gemm_generic.hpp"

namespace ckx {

template <int DT, int IM2COL>
static hipError_t launch_one(const GemmArgs& a, const GenericLayout& lay, hipStream_t s)
{
    const unsigned batches = a.batch > 1 ? (unsigned)a.batch : 1u;
    hipLaunchKernelGGL((gemm_generic_kernel<DT, IM2COL>), dim3((unsigned)a.tiles_m * (unsigned)a.tiles_n, batches), dim3(256), 0,
                       s, a, lay);
    return hipGetLastError();
}

hipError_t launch_generic(int dt, int im2col, const GemmArgs& a, const GenericLayout& lay, hipStream_t s)
{
    if(a.batch > 65535)
        return hipErrorInvalidValue;
    switch(dt * 3 + im2col)
    {
    case DT_I8 * 3 + 0: return launch_one<DT_I8, 0>(a, lay, s);
    case DT_I8 * 3 + 1: return launch_one<DT_I8, 1>(a, lay, s);
    case DT_I8 * 3 + 2: return launch_one<DT_I8, 2>(a, lay, s);
    case DT_F16 * 3 + 0: return launch_one<DT_F16, 0>(a, lay, s);
    case DT_F16 * 3 + 1: return launch_one<DT_F16, 1>(a, lay, s);
    case DT_F16 * 3 + 2: return launch_one<DT_F16, 2>(a, lay, s);
    case DT_BF16 * 3 + 0: return launch_one<DT_BF16, 0>(a, lay, s);
    default: return hipErrorInvalidValue;
    }
}

} // namespace ckx

// Launch of the persistent tile kernel and the list of tile shapes, shared by the translation
// units that instantiate it (K-contiguous operands and im2col in ckx_api.hip, K-major operands in
// gemm_layouts.hip).
#pragma once

#include <hip/hip_runtime.h>

#include <mutex>

#include "gemm_tile.hpp"

namespace ckx {

typedef hipError_t (*tile_launch_fn)(const GemmArgs&, int grid, hipStream_t);

// X(BM, BN, waves along M, waves along N, LDS stages, measured MFMA throughput relative to 256x256).
// The position in this list is the instance index of the C ABI.
#define CKX_FOR_EACH_TILE(X)     \
    X(256, 256, 2, 4, 2, 1.00f)  \
    X(256, 128, 4, 2, 3, 0.84f)  \
    X(128, 128, 2, 2, 2, 0.70f)  \
    X(128, 64, 4, 1, 2, 0.68f)   \
    X(64, 64, 4, 1, 2, 0.55f)    \
    X(32, 64, 2, 1, 2, 0.42f)    \
    X(16, 64, 1, 1, 2, 0.27f)    \
    X(256, 64, 8, 1, 2, 0.70f)   \
    X(64, 64, 4, 1, 4, 0.55f)

inline int num_cus()
{
    static int n = [] {
        int dev = 0, cus = 0;
        if(hipGetDevice(&dev) != hipSuccess ||
           hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        return cus;
    }();
    return n;
}

// Persistent launch: at most (workgroups that fit a CU) x (CUs) workgroups, a multiple of 8 so
// that workgroup b always lands on XCD b % 8 together with the tiles b, b + grid, ...
template <int DT, int BM, int BN, int WM, int WN, int BKB, int NST, int IM2COL, bool TA = false, bool TB = false,
          bool FUSED = false>
hipError_t launch_tile(const GemmArgs& a, int tiles, hipStream_t s)
{
    using T              = GemmTile<DT, BM, BN, WM, WN, BKB, NST, IM2COL, TA, TB, FUSED>;
    auto* kern           = &gemm_tile_kernel<DT, BM, BN, WM, WN, BKB, NST, IM2COL, TA, TB, FUSED>;
    static std::once_flag once;
    static hipError_t attr_err = hipSuccess;
    std::call_once(once, [&] {
        attr_err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, T::LDS);
    });
    if(attr_err != hipSuccess)
        return attr_err;
    int per_cu = 160 * 1024 / T::LDS;
    per_cu     = per_cu > 2048 / T::NT ? 2048 / T::NT : per_cu;
    per_cu     = per_cu < 1 ? 1 : per_cu;
    int grid   = num_cus() * per_cu;
    grid -= grid % 8;
    grid = tiles < grid ? tiles : grid;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(T::NT), T::LDS, s, a);
    return hipGetLastError();
}

// K-major operand layouts (gemm_layouts.hip): launcher of tile instance `tile` for element type dt
// (DT_*), A K-major (a_kmajor: column-major "km") and / or B K-major (b_kmajor: row-major "kn");
// null when that tile shape has no such variant (fewer than 64 rows)
tile_launch_fn layout_tile(int dt, int tile, bool a_kmajor, bool b_kmajor);

// four-wave body of the 256 x 256 tile instance (gemm_w4.hip): dense K-contiguous GEMM or strided batch, one K run; launcher for
// element type dt (DT_*) with the plain epilogues (PassThrough and the two uniform requant modes) or, fused (fp16 only,
// else null), with the D-operand epilogues
tile_launch_fn w4_tile(int dt, bool fused);

// weight-streaming GEMM for up to 128 rows (gemm_astream.hip): launcher for element type dt (DT_*) with 16 * nt output
// columns per workgroup (nt = 3), grid = number of such column blocks
tile_launch_fn astream_launcher(int dt, int nt);

// conv forward with three spatial dimensions (conv3d.hip): launcher of tile instance `tile` for DT_I8 / DT_F16
tile_launch_fn conv3d_tile(int dt, int tile);

} // namespace ckx

// Tile-kernel instantiations for the GEMM layouts with a K-major operand: A column-major ("km") and / or
// B row-major ("kn"), which the reference ships as separate instance lists
// (library/src/tensor_operation_instance/gpu/gemm/device_gemm_xdl_*_{km_kn,km_nk,mk_kn}_mn_instance.cpp).
// A translation unit of its own so that it compiles next to ckx_api.hip.
#include "tile_launch.hpp"

namespace ckx {
namespace {

struct LayoutTile
{
    tile_launch_fn fn[3][3]; // [dtype][0: km_nk, 1: mk_kn, 2: km_kn]
};

// A fragment of a K-major operand costs two LDS reads instead of one, so the waves of a workgroup are
// arranged to give the K-major side the FEWER fragments per wave: the arrangement of the K-contiguous
// instance (WM x WN waves) when only B is K-major, the mirrored one (WN x WM) when only A is and the
// mirrored wave tile still is a multiple of 16 x 64.
template <int BM, int BN, int WM, int WN, int NST>
constexpr LayoutTile make_layout_tile()
{
    if constexpr(BM >= 64 && BN >= 64)
    {
        constexpr bool more_a_frags = (BM / WM) / 16 > (BN / WN) / 16;
        constexpr bool mirror       = more_a_frags && (BM / WN) % 16 == 0 && (BN / WM) % 64 == 0;
        constexpr int AM = mirror ? WN : WM, AN = mirror ? WM : WN; // waves when only A is K-major
        return LayoutTile{{{&launch_tile<DT_I8, BM, BN, AM, AN, 128, NST, false, true, false>,
                            &launch_tile<DT_I8, BM, BN, WM, WN, 128, NST, false, false, true>,
                            &launch_tile<DT_I8, BM, BN, WM, WN, 128, NST, false, true, true>},
                           {&launch_tile<DT_F16, BM, BN, AM, AN, 128, NST, false, true, false>,
                            &launch_tile<DT_F16, BM, BN, WM, WN, 128, NST, false, false, true>,
                            &launch_tile<DT_F16, BM, BN, WM, WN, 128, NST, false, true, true>},
                           {&launch_tile<DT_BF16, BM, BN, AM, AN, 128, NST, false, true, false>,
                            &launch_tile<DT_BF16, BM, BN, WM, WN, 128, NST, false, false, true>,
                            &launch_tile<DT_BF16, BM, BN, WM, WN, 128, NST, false, true, true>}}};
    }
    else
        return LayoutTile{};
}

#define CKX_LAYOUT_TILE(BM, BN, WM, WN, NST, EFF) make_layout_tile<BM, BN, WM, WN, NST>(),
const LayoutTile kLayoutTiles[] = {CKX_FOR_EACH_TILE(CKX_LAYOUT_TILE)};
constexpr int kNumLayoutTiles = sizeof(kLayoutTiles) / sizeof(kLayoutTiles[0]);

} // namespace

tile_launch_fn layout_tile(int dt, int tile, bool a_kmajor, bool b_kmajor)
{
    if(dt < 0 || dt > 2 || tile < 0 || tile >= kNumLayoutTiles || (!a_kmajor && !b_kmajor))
        return nullptr;
    return kLayoutTiles[tile].fn[dt][a_kmajor && b_kmajor ? 2 : b_kmajor ? 1 : 0];
}

} // namespace ckx

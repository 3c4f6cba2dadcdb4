// Tile-kernel instantiations for the conv forward with three spatial dimensions (NDHWC / KZYXC / NDHWK),
// the NumDimSpatial == 3 case of DeviceConvNDFwdXdl_Input_N_Hi_Wi_C_Weight_K_Y_X_C_Output_N_Ho_Wo_K
// (device_convnd_fwd_xdl_nhwc_kyxc_nhwk.hpp:76-1046). A translation unit of its own so that it compiles
// next to ckx_api.hip.
#include "tile_launch.hpp"

namespace ckx {
namespace {

struct Conv3dTile
{
    tile_launch_fn i8, f16;
};
#define CKX_CONV3D_TILE(BM, BN, WM, WN, NST, EFF) \
    {&launch_tile<DT_I8, BM, BN, WM, WN, 128, NST, 2>, &launch_tile<DT_F16, BM, BN, WM, WN, 128, NST, 2>},
const Conv3dTile kConv3dTiles[] = {CKX_FOR_EACH_TILE(CKX_CONV3D_TILE)};
constexpr int kNumConv3dTiles = sizeof(kConv3dTiles) / sizeof(kConv3dTiles[0]);

} // namespace

tile_launch_fn conv3d_tile(int dt, int tile)
{
    if(tile < 0 || tile >= kNumConv3dTiles || (dt != DT_I8 && dt != DT_F16))
        return nullptr;
    return dt == DT_I8 ? kConv3dTiles[tile].i8 : kConv3dTiles[tile].f16;
}

} // namespace ckx

// Instantiations of the LDS-tile backward pass A (fp16).
#include "matchattn_bwd_tile.h"
#include "matchattn_launch.h"

namespace ma {

#ifndef MA_BWD_TILE_VPL
#define MA_BWD_TILE_VPL 2
#endif

template <int CH, int R>
static int launch_bwd_tile(const BwdArgs &A, const TileSort &S, hipStream_t s) {
    constexpr int VPL = CH >= 8 * MA_BWD_TILE_VPL ? MA_BWD_TILE_VPL : 1;      // vectors per lane
    typedef TileCfg<CH, R, kTileW, kTileH, VPL> Cfg;
    if (A.h % Cfg::HPG != 0) return -1;
    launch_tile_chunks(S, A.h, Cfg::QPP, s);
    const unsigned grid = tile_grid(2u * (unsigned)kTileGridMult);   // persistent: two workgroups fit a CU's LDS
    hipLaunchKernelGGL((bwd_h16_tile_kernel<CH, R, kTileW, kTileH, VPL>), dim3(grid), dim3(kTileNT), 0, s, A, S);
    return (int)hipGetLastError();
}

#define MA_BT_CASE(ch, r) \
    if (CH == ch && R == r) return launch_bwd_tile<ch, r>(A, S, s);

int launch_bwd_tile_f16(const BwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s) {
    MA_BT_CASE(16, 1) MA_BT_CASE(16, 2)
    MA_BT_CASE(32, 1) MA_BT_CASE(32, 2)
    MA_BT_CASE(64, 1) MA_BT_CASE(64, 2)
    (void)A; (void)S; (void)s;
    return -1;
}

}  // namespace ma

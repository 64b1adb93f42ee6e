// Instantiations of the LDS-tile forward kernel (fp16).
#include "matchattn_fwd_tile.h"
#include "matchattn_launch.h"

namespace ma {

const int kTileDims[2] = {kTileW, kTileH};
const int kTileCapHost = kTileCap;
void launch_tile_chunks(const TileSort &S, int h, int queries_per_pass, hipStream_t s) {
    hipLaunchKernelGGL(tile_chunks_kernel<0>, dim3(1), dim3(1024), 0, s, S, h, S.chunk_start, queries_per_pass > 0 ? queries_per_pass : 64);
}

#ifndef MA_TILE_VPL
#define MA_TILE_VPL 2
#endif
template <int CH, int R>
static int launch_tile(const FwdArgs &A, const TileSort &S, hipStream_t s) {
    constexpr int VPL = CH >= 8 * MA_TILE_VPL ? MA_TILE_VPL : 1;      // vectors per lane
    typedef TileCfg<CH, R, kTileW, kTileH, VPL> Cfg;
    if (A.h % Cfg::HPG != 0) return -1;
    FwdArgs B = A;
    launch_tile_chunks(S, A.h, Cfg::QPP, s);
    // persistent grid: a multiple of the 8 XCDs; two workgroups fit a CU's LDS
    const unsigned grid = tile_grid(2u * (unsigned)kTileGridMult);
    timer_mark(false, s);
    hipLaunchKernelGGL((fwd_h16_tile_kernel<CH, R, kTileW, kTileH, VPL>), dim3(grid), dim3(kTileNT), 0, s, B, S);
    timer_mark(true, s);
    return (int)hipGetLastError();
}

#define MA_TILE_CASE(ch, r)                                           \
    if (CH == ch && R == r) {                                         \
        *name = "fwd_tile_f16_ch" #ch "_r" #r;                        \
        return launch_tile<ch, r>(A, S, s);                           \
    }

int launch_fwd_tile_f16(const FwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s, const char **name) {
    MA_TILE_CASE(16, 1) MA_TILE_CASE(16, 2)
    MA_TILE_CASE(32, 1) MA_TILE_CASE(32, 2)
    MA_TILE_CASE(64, 1) MA_TILE_CASE(64, 2)
    (void)A; (void)S; (void)s; (void)name;
    return -1;
}

}  // namespace ma

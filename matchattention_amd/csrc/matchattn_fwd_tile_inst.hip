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
    // (heads of 64 channels, 6x6 window: as two half-heads of 32 each on the kernel with the matrix-unit phases -- 1.06x
    // to 1.14x faster than the instance for 64 channels; with the 4x4 window 0.84x to 0.89x, so not there)
    constexpr bool kPaired = CH == 64 && R == 2 && MA_TILE_VPL == 2;
    typedef TileCfg<kPaired ? 32 : CH, R, kTileW, kTileH, VPL> Cfg;
    if (!kPaired && A.h % Cfg::HPG != 0) return -1;
    FwdArgs B = A;
    launch_tile_chunks(S, A.h, Cfg::QPP, s);
    // persistent grid: a multiple of the 8 XCDs; two workgroups fit a CU's LDS
    const unsigned grid = tile_grid(2u * (unsigned)kTileGridMult);
    timer_mark(false, s);
    if constexpr (kPaired) hipLaunchKernelGGL((fwd_h16_tile_kernel<32, R, kTileW, kTileH, 2, half_t, true>), dim3(grid), dim3(kTileNT), 0, s, B, S);
    else
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

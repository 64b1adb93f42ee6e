// Instantiations of the LDS-tile backward pass A for fp32 and bf16 storage.
// Compile with -DMA_DTYPE=0 (fp32) or 2 (bf16).
#include "matchattn_bwd_tile_t.h"
#include "matchattn_launch.h"

#ifndef MA_DTYPE
#error "define MA_DTYPE"
#endif

namespace ma {

#if MA_DTYPE == 0
typedef float T;
#define MA_SUFFIX f32
#else
typedef bf16_t T;
#define MA_SUFFIX bf16
#endif
#define MA_CAT2(a, b) a##b
#define MA_CAT(a, b) MA_CAT2(a, b)

template <int CH, int R>
static int launch_bwd_tile(const BwdArgs &A, const TileSort &S, hipStream_t s) {
    constexpr int NT = CH * (int)sizeof(T) > 128 ? 2 * kTileNT : kTileNT;   // 256-byte heads: one workgroup of 512 per CU
    typedef TileCfgT<T, CH, R, kTileW, kTileH, 1, NT> Cfg;
    if (A.h % Cfg::HPG != 0) return -1;
    launch_tile_chunks(S, A.h, Cfg::QPP, s);
    const unsigned grid = tile_grid((unsigned)Cfg::WG_PER_CU * (unsigned)kTileGridMult);   // persistent: what fits a CU's LDS
    hipLaunchKernelGGL((bwd_tile_kernel<T, CH, R, kTileW, kTileH, NT>), dim3(grid), dim3(NT), 0, s, A, S);
    return (int)hipGetLastError();
}

#define MA_BT_CASE(ch, r) \
    if (CH == ch && R == r) return launch_bwd_tile<ch, r>(A, S, s);

int MA_CAT(launch_bwd_tile_, MA_SUFFIX)(const BwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s) {
    MA_BT_CASE(16, 1) MA_BT_CASE(16, 2)
    MA_BT_CASE(32, 1) MA_BT_CASE(32, 2)
    MA_BT_CASE(64, 1) MA_BT_CASE(64, 2)          // (64 fp32 channels: 256-byte pixels, one workgroup of 512 threads per CU)
    (void)A; (void)S; (void)s;
    return -1;
}

}  // namespace ma

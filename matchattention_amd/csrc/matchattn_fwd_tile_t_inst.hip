// Instantiations of the LDS-tile forward kernel for fp32 and bf16 storage.
// Compile with -DMA_DTYPE=0 (fp32) or 2 (bf16).
#include "matchattn_fwd_tile_t.h"
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
#define MA_STR2(a) #a
#define MA_STR(a) MA_STR2(a)

template <int CH, int R>
static int launch_tile(const FwdArgs &A, const TileSort &S, hipStream_t s) {
    constexpr int VPL = CH * (int)sizeof(T) >= 32 ? 2 : 1;            // vectors per lane
    constexpr int NT = CH * (int)sizeof(T) > 128 ? 2 * kTileNT : kTileNT;   // 256-byte heads: one workgroup of 512 per CU
    typedef TileCfgT<T, CH, R, kTileW, kTileH, VPL, NT> Cfg;
    if (A.h % Cfg::HPG != 0) return -1;
#if MA_DTYPE == 2
    // (64 bf16 channels per head, 6x6 window: as two half-heads of 32 each on the 16-bit kernel, 64 queries per head
    // and pass -- 1.22x to 1.37x faster than this file's kernel; with the 4x4 window 0.95x to 1.02x, so not there)
    launch_tile_chunks(S, A.h, CH == 64 && R == 2 ? 64 : Cfg::QPP, s);
#else
    launch_tile_chunks(S, A.h, Cfg::QPP, s);
#endif
    const unsigned grid = tile_grid((unsigned)Cfg::WG_PER_CU * (unsigned)kTileGridMult);   // persistent: what fits a CU's LDS
    timer_mark(false, s);
#if MA_DTYPE == 2
    // 32 bf16 channels per head: the 16-bit kernel with its sums and its aggregation on the matrix unit
    if constexpr (CH == 32) hipLaunchKernelGGL((fwd_h16_tile_kernel<CH, R, kTileW, kTileH, 2, bf16_t>), dim3(grid), dim3(kTileNT), 0, s, A, S);
    else if constexpr (CH == 64 && R == 2) hipLaunchKernelGGL((fwd_h16_tile_kernel<32, R, kTileW, kTileH, 2, bf16_t, true>), dim3(grid), dim3(kTileNT), 0, s, A, S);
    else
#endif
    hipLaunchKernelGGL((fwd_tile_kernel<T, CH, R, kTileW, kTileH, VPL, NT>), dim3(grid), dim3(NT), 0, s, A, S);
    timer_mark(true, s);
    return (int)hipGetLastError();
}

#define MA_TILE_CASE(ch, r)                                                  \
    if (CH == ch && R == r) {                                                \
        *name = "fwd_tile_" MA_STR(MA_SUFFIX) "_ch" #ch "_r" #r;             \
        return launch_tile<ch, r>(A, S, s);                                  \
    }

int MA_CAT(launch_fwd_tile_, MA_SUFFIX)(const FwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s, const char **name) {
    MA_TILE_CASE(16, 1) MA_TILE_CASE(16, 2)
    MA_TILE_CASE(32, 1) MA_TILE_CASE(32, 2)
    MA_TILE_CASE(64, 1) MA_TILE_CASE(64, 2)      // (64 fp32 channels: 256-byte pixels, one workgroup of 512 threads per CU)
    (void)A; (void)S; (void)s; (void)name;
    return -1;
}

}  // namespace ma

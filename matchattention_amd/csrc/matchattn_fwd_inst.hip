// Instantiations of the forward kernels for one storage dtype.
// Compile with -DMA_DTYPE=0 (fp32), 1 (fp16) or 2 (bf16).
#include "matchattn_fwd_h16.h"
#include "matchattn_launch.h"

#ifndef MA_DTYPE
#error "define MA_DTYPE"
#endif

namespace ma {

#if MA_DTYPE == 0
typedef float T;
#define MA_SUFFIX f32
#elif MA_DTYPE == 1
typedef half_t T;
#define MA_SUFFIX f16
#else
typedef bf16_t T;
#define MA_SUFFIX bf16
#endif
#define MA_CAT2(a, b) a##b
#define MA_CAT(a, b) MA_CAT2(a, b)
#define MA_STR2(a) #a
#define MA_STR(a) MA_STR2(a)

template <int CH, int R, int VPL>
static int launch_tiled(const FwdArgs &A, hipStream_t s) {
    typedef TiledCfg<T, CH, R, VPL> Cfg;
    const unsigned nblocks = (unsigned)((A.nhq + Cfg::HQ_PER_BLOCK - 1) / Cfg::HQ_PER_BLOCK);
#if MA_DTYPE == 1
    // grid of the head-group decomposition (see fwd_h16_kernel)
    FwdArgs B = A;
    const int npix = A.nhq / A.h;
    // heads per group: enough for a 128-byte line per pixel, a power of two dividing h, and a
    // number of groups that divides the 8 XCDs
    int hl = 0;
    while ((1 << hl) * CH * 2 < 128 && A.h % (2 << hl) == 0 && (Cfg::HQ_PER_BLOCK >> (hl + 1)) >= 1) ++hl;
    while (A.h % (1 << hl) == 0 && 8 % (A.h >> hl) != 0 && A.h % (2 << hl) == 0 && (Cfg::HQ_PER_BLOCK >> (hl + 1)) >= 1) ++hl;
    if (8 % (A.h >> hl) != 0) B.xcd_swizzle = 0;       // group count does not divide the XCDs
    B.hpg_log2 = hl;
    const int nhg = A.h >> hl, ppb = Cfg::HQ_PER_BLOCK >> hl;
    const unsigned pblocks = (unsigned)((npix + ppb - 1) / ppb);
    unsigned grid;
    if (B.xcd_swizzle) {
        const unsigned bands = 8u / (unsigned)nhg;
        grid = 8u * ((pblocks + bands - 1) / bands);
    } else {
        grid = pblocks * (unsigned)nhg;
    }
    (void)nblocks;
    hipLaunchKernelGGL((fwd_h16_kernel<CH, R, VPL>), dim3(grid), dim3(Cfg::BLOCK), 0, s, B);
#else
    hipLaunchKernelGGL((fwd_tiled_kernel<T, CH, R, VPL>), dim3(nblocks), dim3(Cfg::BLOCK), 0, s, A);
#endif
    return (int)hipGetLastError();
}

#define MA_CASE(ch, r, vpl)                                                            \
    if (CH == ch && R == r && VPL == vpl) {                                            \
        *name = "fwd_tiled_" MA_STR(MA_SUFFIX) "_ch" #ch "_r" #r "_vpl" #vpl;          \
        return launch_tiled<ch, r, vpl>(A, s);                                         \
    }

int MA_CAT(launch_fwd_tiled_, MA_SUFFIX)(const FwdArgs &A, int CH, int R, int VPL, hipStream_t s, const char **name) {
#if MA_DTYPE == 0
    // fp32: 4 channels per 16-byte vector
    MA_CASE(8, 1, 1) MA_CASE(8, 2, 1) MA_CASE(8, 1, 2) MA_CASE(8, 2, 2)
    MA_CASE(16, 1, 1) MA_CASE(16, 2, 1) MA_CASE(16, 1, 2) MA_CASE(16, 2, 2)
    MA_CASE(32, 1, 1) MA_CASE(32, 2, 1) MA_CASE(32, 1, 2) MA_CASE(32, 2, 2)
    MA_CASE(40, 1, 1) MA_CASE(40, 2, 1)
    MA_CASE(64, 1, 1) MA_CASE(64, 2, 1) MA_CASE(64, 1, 2) MA_CASE(64, 2, 2)
    // (the coarse levels of the reference's `small` and `base` variants in its default precision: 20, 24 and 32 vectors
    // per head, two per lane on 16 lanes)
    MA_CASE(80, 1, 2) MA_CASE(80, 2, 2)
    MA_CASE(96, 1, 2) MA_CASE(96, 2, 2)
    MA_CASE(128, 1, 2) MA_CASE(128, 2, 2)
    MA_CASE(192, 1, 2) MA_CASE(192, 2, 2)              // (24 lanes of 32 carry a head-query)
#else
    // 16-bit types: 8 channels per 16-byte vector
    MA_CASE(8, 1, 1) MA_CASE(8, 2, 1)
    MA_CASE(16, 1, 1) MA_CASE(16, 2, 1) MA_CASE(16, 1, 2) MA_CASE(16, 2, 2)
    MA_CASE(32, 1, 1) MA_CASE(32, 2, 1) MA_CASE(32, 1, 2) MA_CASE(32, 2, 2)
    MA_CASE(40, 1, 1) MA_CASE(40, 2, 1)
    MA_CASE(64, 1, 1) MA_CASE(64, 2, 1) MA_CASE(64, 1, 2) MA_CASE(64, 2, 2)
    MA_CASE(80, 1, 1) MA_CASE(80, 2, 1)
    MA_CASE(96, 1, 1) MA_CASE(96, 2, 1)
    MA_CASE(128, 1, 1) MA_CASE(128, 2, 1) MA_CASE(128, 1, 2) MA_CASE(128, 2, 2)
    MA_CASE(192, 1, 2) MA_CASE(192, 2, 2)
#endif
    (void)A; (void)s; (void)name;
    return -1;
}

int MA_CAT(launch_fwd_generic_, MA_SUFFIX)(const FwdArgs &A, int R, hipStream_t s, const char **name) {
    unsigned nblocks = (unsigned)((A.nhq + 255) / 256);
    if (A.defer && nblocks > 1024) nblocks = 1024;    // flag mode: a fixed grid strides over the flags
    switch (R) {
    case 1:
        *name = "fwd_generic_" MA_STR(MA_SUFFIX) "_r1";
        hipLaunchKernelGGL((fwd_generic_kernel<T, 1>), dim3(nblocks), dim3(256), 0, s, A);
        break;
    case 2:
        *name = "fwd_generic_" MA_STR(MA_SUFFIX) "_r2";
        hipLaunchKernelGGL((fwd_generic_kernel<T, 2>), dim3(nblocks), dim3(256), 0, s, A);
        break;
    case 3:
        *name = "fwd_generic_" MA_STR(MA_SUFFIX) "_r3";
        hipLaunchKernelGGL((fwd_generic_kernel<T, 3>), dim3(nblocks), dim3(256), 0, s, A);
        break;
    default:
        return -1;
    }
    return (int)hipGetLastError();
}

}  // namespace ma

// Instantiations of the backward kernels for one storage dtype.
// Compile with -DMA_DTYPE=0 (fp32), 1 (fp16) or 2 (bf16).
#include "matchattn_bwd_gather.h"
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

template <int CH, int R>
static int launch_tiled(const BwdArgs &A, hipStream_t s) {
    typedef TiledCfg<T, CH, R, 1> Cfg;
    const unsigned nblocks = (unsigned)((A.nhq + Cfg::HQ_PER_BLOCK - 1) / Cfg::HQ_PER_BLOCK);
    if (A.dl_ws)
        hipLaunchKernelGGL((bwd_tiled_kernel<T, CH, R, true>), dim3(nblocks), dim3(Cfg::BLOCK), 0, s, A);
    else
        hipLaunchKernelGGL((bwd_tiled_kernel<T, CH, R, false>), dim3(nblocks), dim3(Cfg::BLOCK), 0, s, A);
    return (int)hipGetLastError();
}

#define MA_CASE(ch)                                                         \
    if (CH == ch && R == 1) {                                               \
        *name = "bwd_tiled_" MA_STR(MA_SUFFIX) "_ch" #ch "_r1";             \
        return launch_tiled<ch, 1>(A, s);                                   \
    }                                                                       \
    if (CH == ch && R == 2) {                                               \
        *name = "bwd_tiled_" MA_STR(MA_SUFFIX) "_ch" #ch "_r2";             \
        return launch_tiled<ch, 2>(A, s);                                   \
    }

int MA_CAT(launch_bwd_tiled_, MA_SUFFIX)(const BwdArgs &A, int CH, int R, hipStream_t s, const char **name) {
    MA_CASE(8) MA_CASE(16) MA_CASE(32) MA_CASE(40) MA_CASE(64)
    // (the coarse levels of the reference's larger variants; beyond 16 vectors per head a head-query takes 32 lanes)
    MA_CASE(80) MA_CASE(96) MA_CASE(128) MA_CASE(192)
    (void)A; (void)s; (void)name;
    return -1;
}

template <int CH, int R>
static int launch_key(const BwdArgs &A, hipStream_t s) {
    constexpr int VPL = KeyVpl<T, CH, R>::value;
    typedef TiledCfg<T, CH, R, VPL> Cfg;
    const unsigned nblocks = (unsigned)((A.nhq + Cfg::HQ_PER_BLOCK - 1) / Cfg::HQ_PER_BLOCK);
    // (the compact form of a candidate: the pixel index in 25 bits, the pair array within a buffer descriptor's 4 GiB)
    const bool compact = A.nhq / A.h < (1 << 25) && (unsigned long long)A.nhq * Cfg::M * PairOf<T>::kBytes < 0xFFFFF000ull;
    if (compact) hipLaunchKernelGGL((bwd_key_kernel<T, CH, R, VPL, true>), dim3(nblocks), dim3(Cfg::BLOCK), 0, s, A);
    else hipLaunchKernelGGL((bwd_key_kernel<T, CH, R, VPL, false>), dim3(nblocks), dim3(Cfg::BLOCK), 0, s, A);
    return (int)hipGetLastError();
}

#define MA_KCASE(ch)                                                        \
    if (CH == ch && R == 1) return launch_key<ch, 1>(A, s);                 \
    if (CH == ch && R == 2) return launch_key<ch, 2>(A, s);

// pass B of the gather-mode backward (same instantiation set as the tiled pass A)
int MA_CAT(launch_bwd_key_, MA_SUFFIX)(const BwdArgs &A, int CH, int R, hipStream_t s) {
    MA_KCASE(8) MA_KCASE(16) MA_KCASE(32) MA_KCASE(40) MA_KCASE(64)
    MA_KCASE(80) MA_KCASE(96) MA_KCASE(128) MA_KCASE(192)
    (void)A; (void)s;
    return -1;
}

int MA_CAT(launch_bwd_generic_, MA_SUFFIX)(const BwdArgs &A, int R, hipStream_t s, const char **name) {
    const unsigned nblocks = (unsigned)((A.nhq + 255) / 256);
    switch (R) {
    case 1:
        *name = "bwd_generic_" MA_STR(MA_SUFFIX) "_r1";
        hipLaunchKernelGGL((bwd_generic_kernel<T, 1>), dim3(nblocks), dim3(256), 0, s, A);
        break;
    case 2:
        *name = "bwd_generic_" MA_STR(MA_SUFFIX) "_r2";
        hipLaunchKernelGGL((bwd_generic_kernel<T, 2>), dim3(nblocks), dim3(256), 0, s, A);
        break;
    case 3:
        *name = "bwd_generic_" MA_STR(MA_SUFFIX) "_r3";
        hipLaunchKernelGGL((bwd_generic_kernel<T, 3>), dim3(nblocks), dim3(256), 0, s, A);
        break;
    default:
        return -1;
    }
    return (int)hipGetLastError();
}

}  // namespace ma

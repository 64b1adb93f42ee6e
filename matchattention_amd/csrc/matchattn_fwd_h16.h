// Forward kernel specialised for fp16 storage (the dtype of every benchmarked shape).
//
// Same algorithm and lane ownership as fwd_tiled_kernel (matchattn_fwd.h); what differs is
// the register diet and the instruction count:
//   * the window state (scaled logits, later the attention weights) is kept as packed
//     halves -- these values are fp16 by definition (models/mat_pytorch_impl.py:74,
//     models/attention_blocks.py:86 run in the tensor dtype), so nothing is lost and the
//     window costs (2R+2)^2/2 registers instead of (2R+2)^2;
//   * the two roundings of a logit are one v_cvt_f16_f32 and one v_fma_mix{lo,hi}_f16;
//   * the softmax needs only the window maximum (tracked as a running minimum of the raw L1
//     sums: rounding and the negative scale are monotone) and the maximum of the inner
//     (2R)^2 block, which every sub-window contains, to decide whether one exponential per
//     tap can serve all four sub-windows;
//   * the aggregation feeds packed fp16 weights and values straight into v_fma_mix_f32.
#pragma once
#include "matchattn_fwd.h"

namespace ma {

template <int R>
__device__ __forceinline__ void unpack_window(const half2_t (&p)[2 * R + 2][R + 1], float (&f)[2 * R + 2][2 * R + 2]) {
#pragma unroll
    for (int j = 0; j < 2 * R + 2; ++j)
#pragma unroll
        for (int i = 0; i < R + 1; ++i) { f[j][2 * i] = (float)p[j][i].x; f[j][2 * i + 1] = (float)p[j][i].y; }
}

// Waves per SIMD the register allocation aims for (512 VGPRs per SIMD lane: 4 waves = 128
// registers, 3 = 168).  The 6x6 window does not fit 128 registers without spilling.
#ifndef MA_H16_WAVES_R2
#define MA_H16_WAVES_R2 3
#endif
// (two vectors per lane with the 6x6 window, the forward_variant = 2 option: 168 registers spilled 194-333, so two waves)
constexpr int h16_waves(int R, int VPL) { return R == 1 ? (VPL <= 2 ? 4 : 3) : (VPL >= 2 ? 2 : MA_H16_WAVES_R2); }

// Bytes of one group of heads per pixel (at least a full 128-byte line), heads per group, 16-byte pieces.
template <int CH> struct LdsGroup {
    static constexpr int GB = CH * 2 >= 128 ? CH * 2 : 128;    // bytes of one head group per pixel
    static constexpr int HPG = GB / (CH * 2);                  // heads per group
    static constexpr int CPP = GB / 16;                        // 16-byte chunks per pixel
};

template <int CH, int R, int VPL>
__global__ __launch_bounds__(256, h16_waves(R, VPL)) void fwd_h16_kernel(FwdArgs A) {
    typedef half_t T;
    typedef TiledCfg<T, CH, R, VPL> Cfg;
    typedef StageCfg<R, VPL> St;
    constexpr int EPV = 8, LPH = Cfg::LPH, WN = Cfg::WN, M = Cfg::M, HW = WN / 2;
    constexpr int G = St::G, SPR = St::SPR;

    // Work decomposition.  A block covers `ppb` consecutive pixels of one group of 2^hpg_log2
    // heads.  Workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2: XCD x
    // takes head group x % nhg of row band x / nhg, so that the K/V bytes one L2 has to hold
    // are one head group (at least a full 128-byte line per pixel) of a few image rows.
    const int sub = threadIdx.x % LPH;
    const int grp = threadIdx.x / LPH;                    // head-query slot within the block
    const int hpg = 1 << A.hpg_log2, nhg = A.h >> A.hpg_log2;
    const int ppb = Cfg::HQ_PER_BLOCK >> A.hpg_log2;      // pixels per block
    const int npix = A.nhq / A.h;
    int hgrp, pblk;
    if (A.xcd_swizzle) {
        const int xcd = blockIdx.x & 7, k = blockIdx.x >> 3;
        const int per_band = gridDim.x >> 3;              // pixel blocks per (band, head group)
        hgrp = xcd % nhg;
        pblk = (xcd / nhg) * per_band + k;
    } else {
        hgrp = blockIdx.x % nhg;
        pblk = blockIdx.x / nhg;
    }
    int slot = pblk * ppb + (grp >> A.hpg_log2);
    const int head = hgrp * hpg + (grp & (hpg - 1));
    const bool tail = slot >= npix;          // whole lane groups fall off the end together
    if (tail) slot = npix - 1;               // keep them in flight (DPP partners), store nothing
    const int pix = slot;
    const bool carries = sub < Cfg::NVL;
    const bool live = carries && !tail;
    const int bN = (npix == A.N) ? 0 : (pix / A.N) * A.N;   // first pixel of this batch item
    const uint32_t row_bytes = (uint32_t)A.C * 2u;
    const uint32_t total_bytes = (uint32_t)(A.nhq / A.h) * row_bytes;
    const uint32_t chan_bytes = (uint32_t)(head * CH + sub * VPL * EPV) * 2u;

    float x, y;
    sampling_position<T>(A, pix, head, x, y);
    float x0, y0, w[4];
    corner_weights<T>(x, y, x0, y0, w);
    const int ix = centre_index(x0), iy = centre_index(y0);
    const bool skip_last = A.row_skip && __builtin_amdgcn_ballot_w64(y != y0) == 0;
    const bool inside = ix - R >= 0 && ix + R + 1 <= A.W - 1 && iy - R >= 0 && iy + R + 1 <= A.H - 1;
    const bool linear = __builtin_amdgcn_ballot_w64(!inside) == 0;
    const uint32_t tap0_off =
        carries ? (uint32_t)(bN + clampi(iy - R, 0, A.H - 1) * A.W + clampi(ix - R, 0, A.W - 1)) * row_bytes + chan_bytes
                : kDeadOffset;

    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(A.out, out_span_bytes(A, 2));
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A.attn, attn_span_bytes(A, (uint32_t)(A.h * M), 2));
    const __amdgpu_buffer_rsrc_t rgate = make_rsrc(A.gate, A.gate ? total_bytes : 0u);

    u32x4 qv[VPL];
    const uint32_t q_off = carries ? (uint32_t)pix * row_bytes + chan_bytes : kDeadOffset;
#pragma unroll
    for (int u = 0; u < VPL; ++u) qv[u] = buf_load16(rq, q_off + u * 16);
    const float nscale = -A.scale;
    // LDS: the exact-softmax path parks the window here (M floats per lane)
    constexpr int kSmemBytes = M * 256 * 4;
    __shared__ __attribute__((aligned(16))) char smem[kSmemBytes];
    float (*park)[256] = reinterpret_cast<float (*)[256]>(smem);

    // `drop_last`: the last window row is neither fetched nor computed (only its SPR stages are
    // guarded, by wavefront-uniform branches, so the rest stays straight-line code).
    // MODE 0: per-tap clamped offsets; 1: uniform tap distances (every window inside the image)
    auto body = [&](auto mode_tag, const bool drop_last) __attribute__((always_inline)) {
        constexpr int MODE = decltype(mode_tag)::value;
        constexpr bool LINEAR = MODE != 0;
        constexpr int NSR = WN * SPR;
        constexpr int LAST0 = (WN - 1) * SPR;       // first stage of the last window row
        uint32_t col_off[WN], row_off[WN];
        if constexpr (!LINEAR) {
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                col_off[i] = carries ? (uint32_t)(bN + clampi(ix + i - R, 0, A.W - 1)) * row_bytes + chan_bytes : kDeadOffset;
                row_off[i] = carries ? (uint32_t)(clampi(iy + i - R, 0, A.H - 1) * A.W) * row_bytes : 0u;
            }
        }
        u32x4 buf[2][G][VPL];
        auto fetch = [&](const __amdgpu_buffer_rsrc_t &r, auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
#pragma unroll
            for (int t = 0; t < G; ++t)
#pragma unroll
                for (int u = 0; u < VPL; ++u)
                    if constexpr (MODE == 1)
                        buf[s & 1][t][u] = buf_load16(r, tap0_off + u * 16, (uint32_t)(j * A.W + i0 + t) * row_bytes);
                    else
                        buf[s & 1][t][u] = buf_load16(r, row_off[j] + col_off[i0 + t] + u * 16);
        };
        // ---- logits ------------------------------------------------------------------------
        half2_t lgp[WN][HW];
        const half_t ninf = (half_t)(-__builtin_inff());
#pragma unroll
        for (int i = 0; i < HW; ++i) lgp[WN - 1][i] = half2_t{ninf, ninf};   // stays if the row is left out
        float smin_all = __builtin_inff(), smin_in = __builtin_inff();        // minima of the raw L1 sums
        fetch(rk, std::integral_constant<int, 0>{});
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) {
                if (s + 1 < LAST0 || !drop_last) fetch(rk, std::integral_constant<int, s + 1>{});
            }
            if (s >= LAST0 && drop_last) return;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                const int i = i0 + t;
                float sum = 0.f;
#pragma unroll
                for (int u = 0; u < VPL; ++u) sum = l1_accum<T>(qv[u], buf[s & 1][t][u], sum);
                sum = group_sum<LPH>(sum);
                smin_all = fminf(smin_all, sum);
                if (j >= 1 && j <= 2 * R && i >= 1 && i <= 2 * R) smin_in = fminf(smin_in, sum);
                const half_t l16 = (half_t)sum;                       // channel sum stored in fp16
                const half_t s16 = (half_t)((float)l16 * nscale);     // scaled logit stored in fp16
                if (i & 1) lgp[j][i >> 1].y = s16; else lgp[j][i >> 1].x = s16;
            }
            __builtin_amdgcn_sched_barrier(0);
        });

        // ---- window softmax ----------------------------------------------------------------
        fetch(rv, std::integral_constant<int, 0>{});   // first V stage travels while the softmax runs
        const float gmax = (float)(half_t)((float)(half_t)smin_all * nscale);   // rounding is monotone
        const float imax = (float)(half_t)((float)(half_t)smin_in * nscale);
        const bool far = !(gmax - imax < kSharedExpLimit);
        half2_t ap[WN][HW];                             // attention weights, fp16 as stored
        const bool any_far = __builtin_amdgcn_ballot_w64(far) != 0;
        if (!any_far) {
            float e[WN][WN];
            const float gl = gmax * kLog2e;
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    e[j][2 * i] = __builtin_amdgcn_exp2f((float)lgp[j][i].x * kLog2e - gl);
                    e[j][2 * i + 1] = __builtin_amdgcn_exp2f((float)lgp[j][i].y * kLog2e - gl);
                }
            float ssum[4], c[4], c9[3][3];
            subwindow_sum<R>(e, ssum);
#pragma unroll
            for (int b = 0; b < 4; ++b) c[b] = w[b] * __builtin_amdgcn_rcpf(ssum[b]);
            coef9<R>(c, c9);
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    ap[j][i].x = (half_t)(e[j][2 * i] * c9[cls<R>(j)][cls<R>(2 * i)]);
                    ap[j][i].y = (half_t)(e[j][2 * i + 1] * c9[cls<R>(j)][cls<R>(2 * i + 1)]);
                }
        } else {
            // rare: some sub-window lies far below the window maximum; run the exact
            // per-sub-window softmax on a copy of the window parked in LDS
            float *col = &park[0][threadIdx.x];
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    col[(j * WN + 2 * i) * 256] = (float)lgp[j][i].x;
                    col[(j * WN + 2 * i + 1) * 256] = (float)lgp[j][i].y;
                }
            float sw[4] = {w[0], w[1], w[2], w[3]}, smx[4], sinv[4], sc[4];
            softmax_exact_lds<R>(col, 256, sw, smx, sinv, sc, true);
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i)
                    ap[j][i] = half2_t{(half_t)col[(j * WN + 2 * i) * 256], (half_t)col[(j * WN + 2 * i + 1) * 256]};
        }
        __builtin_amdgcn_sched_barrier(0);

        // ---- aggregation -------------------------------------------------------------------
        float acc[VPL][EPV];
#pragma unroll
        for (int u = 0; u < VPL; ++u)
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[u][e] = 0.f;
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) {
                if (s + 1 < LAST0 || !drop_last) fetch(rv, std::integral_constant<int, s + 1>{});
            }
            if (s >= LAST0 && drop_last) return;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                const int i = i0 + t;
                const float am = (float)((i & 1) ? ap[j][i >> 1].y : ap[j][i >> 1].x);
#pragma unroll
                for (int u = 0; u < VPL; ++u)
#pragma unroll
                    for (int e = 0; e < EPV; ++e) acc[u][e] += am * vec_elem<T>(buf[s & 1][t][u], e);
            }
            __builtin_amdgcn_sched_barrier(0);
        });

        // ---- stores (predicated by the buffer range check, not by a branch) -------------------
        const uint32_t o_off = live ? (uint32_t)pix * A.out_row_bytes + chan_bytes : kDeadOffset;
        u32x4 ov[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) ov[u] = vec_pack<T>(acc[u]);
        if (A.gate) {
            const uint32_t g_off = live ? (uint32_t)pix * row_bytes + chan_bytes : kDeadOffset;
#pragma unroll
            for (int u = 0; u < VPL; ++u) ov[u] = vec_mul<T>(ov[u], buf_load16(rgate, g_off + u * 16));
        }
#pragma unroll
        for (int u = 0; u < VPL; ++u) buf_store16(ro, o_off + u * 16, ov[u]);
        const uint32_t a_off = (sub == 0 && !tail) ? (uint32_t)pix * A.attn_row_bytes + (uint32_t)head * (uint32_t)(M * 2) : kDeadOffset;
#pragma unroll
        for (int m = 0; m < M / 2; m += 2)   // dword m of the row holds taps 2m, 2m+1
            buf_store8(ra, a_off + m * 4, u32x2{h2_as_u32(ap[m / HW][m % HW]), h2_as_u32(ap[(m + 1) / HW][(m + 1) % HW])});
    };
    if (linear)
        body(std::integral_constant<int, 1>{}, skip_last);
    else
        body(std::integral_constant<int, 0>{}, false);
}

}  // namespace ma

// Backward kernels of the MatchAttention operator for gfx950.
//
// The reference has no backward kernel: gradients exist only as autograd through
// models/mat_pytorch_impl.py:3-178.  These kernels evaluate the closed-form gradient of
// that definition.  With, per head-query, g_m = dA_m + <dO, v_m>:
//   dw_b  = sum_{m in S_b} p_b[m] g_m
//   dl_m  = scale * sum_{b: m in S_b} w_b p_b[m] (g_m - dw_b)        (w.r.t. -L1)
//   dq_c  = -sum_m dl_m sgn(q_c - k_mc),   dk[tap m]_c += dl_m sgn(q_c - k_mc)
//   dv[tap m]_c += a_m dO_c
//   dx = (1-fy)(dw_ne - dw_nw) + fy (dw_se - dw_sw),  dy = (1-fx)(dw_sw - dw_nw) + fx (dw_se - dw_ne)
// The forward is recomputed from q and k.  dK and dV are accumulated with fp32 atomics
// (into a staging buffer for the 16-bit dtypes) because several queries hit the same key.
#pragma once
#include "matchattn_fwd.h"

namespace ma {

struct BwdArgs {
    const void *mo, *q, *k, *v, *d_out, *d_attn;  // d_attn may be null
    void *dq, *dmo;
    float *dk_acc, *dv_acc;                       // scatter mode: fp32 [B*N*C], zero on entry
    // gather mode (deterministic, no atomics): pass A leaves, per head-query and tap, the logit
    // gradient and the attention weight; pass B sums them per key through the inverse index
    void *dl_ws;                                  // one array of B*N*h*M (dl, a) pairs (layout: PairLayout; PairOf<T>: pass B fetches both
                                                  //   with one load), or null in scatter mode
    void *dk, *dv;                                // outputs of pass B (dtype T)
    const int *perm, *centre, *bin_start, *row_start, *per_head;   // inverse index (matchattn_sort.h), exact bins
    const uint8_t *only_flagged;                  // pass A: optional [nhq] flags, compute only the head-queries whose flag is set
    int nrows;                                    // B*H
    int nhq;
    int N, H, W, C, h;
    float scale;
    int xcd_swizzle;
};

// Where the pair of (pixel, head, tap m) sits in the pair array.  Two layouts, chosen by the inverse index's own flag
// (BwdArgs::per_head[0], set on the device before pass A runs; writers and reader take the same word):
//   one offset shared by the heads: [pixel][tap / 2][head][tap % 2].  Every head reaches a key through the same tap of
//   the same query, so the lane groups of a key fetch 8 h contiguous bytes instead of h pieces M pairs apart -- the
//   pair fetches, not the q and dO rows, are what pass B waits for -- and the two taps of a block stay together:
//   neighbouring keys reach a candidate through neighbouring taps (2 x 384 x 384, 8 heads: 1.98 -> 1.90 ms);
//   an offset per head: [pixel][head][tap], a head-query's taps contiguous (the heads' candidates are unrelated; the
//   block layout measured 10 % slower there).
// Both are "pixel base + head term + block * stride + tap % 2"; a lane fixes the head term and the stride once.
#ifndef MA_PAIR_BLOCK
#define MA_PAIR_BLOCK 4
#endif
constexpr uint32_t kPairBlock = MA_PAIR_BLOCK;     // taps per block: (2r+2)^2 is a multiple of 4
struct PairLayout {
    uint32_t pix_stride, head_term, stride;
    __device__ __forceinline__ PairLayout(uint32_t head, uint32_t M, uint32_t h, bool per_head)
        : pix_stride(M * h), head_term(per_head ? head * M : head * kPairBlock), stride(per_head ? kPairBlock : kPairBlock * h) {}
    // index (in pairs) of tap m of this lane's head at pixel pix
    __device__ __forceinline__ uint32_t at(uint32_t pix, uint32_t m) const {
        return pix * pix_stride + head_term + __umul24(m / kPairBlock, stride) + (m % kPairBlock);
    }
};

// The (logit gradient, attention value) pair pass A leaves per head-query and tap for pass B.  fp32 tensors keep two
// floats; fp16 tensors keep two halves in one word: the attention value is a 16-bit number by definition, and the
// logit gradient, rounded to half precision (11 bits, like every gradient the call returns; saturated at the largest
// half instead of overflowing), halves what pass A writes and pass B reads through L2 per tap.
template <typename T> struct PairOf {
    static constexpr int kBytes = 4;
    typedef uint32_t Word;
    static __device__ __forceinline__ Word pack(float dl, float a) {
        const float s = __builtin_amdgcn_fmed3f(dl, -65504.0f, 65504.0f);
        return h2_as_u32(half2_t{(half_t)s, (half_t)a});
    }
    static __device__ __forceinline__ void unpack(Word w, float &dl, float &a) {
        const half2_t h = as_h2(w);
        dl = (float)h.x;
        a = (float)h.y;
    }
};
// bfloat16 tensors keep two bfloat16 values: the logit gradient then has the exponent range of the tensor type (the
// definition's own backward keeps it in bfloat16), so that gradients of 1e-6 and below -- a mean-reduced loss without
// loss scaling -- neither lose bits nor vanish as they would as halves.
template <> struct PairOf<bf16_t> {
    static constexpr int kBytes = 4;
    typedef uint32_t Word;
    static __device__ __forceinline__ Word pack(float dl, float a) {
        const uint32_t lo = (uint32_t)__builtin_bit_cast(uint16_t, (bf16_t)dl);
        const uint32_t hi = (uint32_t)__builtin_bit_cast(uint16_t, (bf16_t)a);
        return lo | (hi << 16);
    }
    static __device__ __forceinline__ void unpack(Word w, float &dl, float &a) {
        dl = as_f32(w << 16);
        a = as_f32(w & 0xffff0000u);
    }
};
template <> struct PairOf<float> {
    static constexpr int kBytes = 8;
    typedef u32x2 Word;
    static __device__ __forceinline__ Word pack(float dl, float a) { return u32x2{as_u32(dl), as_u32(a)}; }
    static __device__ __forceinline__ void unpack(Word w, float &dl, float &a) { dl = as_f32(w[0]); a = as_f32(w[1]); }
};

__device__ __forceinline__ void atomic_add_f32(float *p, float v) { unsafeAtomicAdd(p, v); }

// sgn(d) as a float in {-1, 0, 1}: exact for every finite d of the supported dtypes
// (2^60 lifts the smallest half/bfloat16 subnormal difference above 1 without overflowing).
__device__ __forceinline__ float sign_f(float d) { return __builtin_amdgcn_fmed3f(d * 0x1p60f, -1.0f, 1.0f); }

// dl[m] (gradient w.r.t. the unscaled negative-L1 logit) and dw[b], from the softmax state.
//   lg: e = exp(lg - gmax) if shared, else the scaled logits; g: in g_m, out dl_m
template <int R>
__device__ __forceinline__ void bilinear_softmax_bwd(bool shared, const float (&lg)[Win<R>::WN][Win<R>::WN],
                                                     const SoftmaxState<R> &st, float scale,
                                                     float (&g)[Win<R>::WN][Win<R>::WN], float (&dw)[4]) {
    constexpr int WN = Win<R>::WN;
    if (shared) {
        float eg[WN][WN];
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) eg[j][i] = lg[j][i] * g[j][i];
        subwindow_sum<R>(eg, dw);
        float cd[4], c9[3][3], cd9[3][3];
#pragma unroll
        for (int b = 0; b < 4; ++b) { dw[b] *= st.inv[b]; cd[b] = st.c[b] * dw[b]; }
        coef9<R>(st.c, c9);
        coef9<R>(cd, cd9);
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i)
                g[j][i] = scale * lg[j][i] * (g[j][i] * c9[cls<R>(j)][cls<R>(i)] - cd9[cls<R>(j)][cls<R>(i)]);
        return;
    }
    float dl[WN][WN];
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WN; ++i) dl[j][i] = 0.f;
#pragma unroll 1
    for (int b = 0; b < 4; ++b) {
        const int dx = b & 1, dy = b >> 1;
        const float mb = st.mx[b], inv = st.inv[b], cb = st.c[b];
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                const bool in = j >= dy && j <= 2 * R + dy && i >= dx && i <= 2 * R + dx;
                s += in ? __builtin_amdgcn_exp2f((lg[j][i] - mb) * kLog2e) * inv * g[j][i] : 0.f;
            }
        dw[b] = s;
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                const bool in = j >= dy && j <= 2 * R + dy && i >= dx && i <= 2 * R + dx;
                dl[j][i] += in ? cb * __builtin_amdgcn_exp2f((lg[j][i] - mb) * kLog2e) * (g[j][i] - s) : 0.f;
            }
    }
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WN; ++i) g[j][i] = scale * dl[j][i];
}

template <typename T>
__device__ __forceinline__ void offset_grad(float x, float y, const float (&dw)[4], float &dx, float &dy) {
    const float fx = x - floorf(x), fy = y - floorf(y);
    dx = (1.0f - fy) * (dw[1] - dw[0]) + fy * (dw[3] - dw[2]);
    dy = (1.0f - fx) * (dw[2] - dw[0]) + fx * (dw[3] - dw[1]);
}

// ---------------------------------------------------------------------------------------
// Tiled backward: same lane ownership as the forward with one 16-byte vector per lane.
// ---------------------------------------------------------------------------------------
#ifndef MA_BWD_WAVES_R2
#define MA_BWD_WAVES_R2 2
#endif
// GATHER: pass A of the gather mode (writes dl / a per head-query and tap, no atomics); otherwise the
// scatter mode (fp32 atomics on dK / dV).  A compile-time choice: the scatter path's addresses and
// branches would otherwise stay alive in the gather kernel.
template <typename T, int CH, int R, bool GATHER>
__global__ __launch_bounds__(256, R == 1 ? 3 : (GATHER ? MA_BWD_WAVES_R2 : 1)) void bwd_tiled_kernel(BwdArgs A) {
    typedef TiledCfg<T, CH, R, 1> Cfg;
    typedef Traits<T> Tr;
    constexpr int EPV = Cfg::EPV, LPH = Cfg::LPH, WN = Cfg::WN, M = Cfg::M;

    const unsigned blk = logical_block(blockIdx.x, gridDim.x, A.xcd_swizzle);
    const int sub = threadIdx.x % LPH;
    int hq = (int)(blk * Cfg::HQ_PER_BLOCK + threadIdx.x / LPH);
    const bool tail = hq >= A.nhq;
    if (tail) hq = A.nhq - 1;
    const bool carries = sub < Cfg::NVL;
    const bool live = carries && !tail;
    // finishing run after the LDS-tile pass A: only what that kernel flagged (whole lane groups leave together)
    if (A.only_flagged && A.only_flagged[hq] == 0) return;

    const int pix = hq / A.h, head = hq - pix * A.h;
    const int b = pix / A.N;
    const uint32_t row_bytes = (uint32_t)A.C * sizeof(T);
    const uint32_t total_bytes = (uint32_t)(A.nhq / A.h) * row_bytes;
    const uint32_t chan = (uint32_t)(head * CH + sub * EPV);
    const uint32_t chan_bytes = chan * sizeof(T);
    const uint32_t kDead = 0xFFFFFF00u;

    const T *mo = (const T *)A.mo + (size_t)hq * 2;
    const float x = Tr::to_f(mo[0]), y = Tr::to_f(mo[1]);
    float x0, y0, w[4];
    corner_weights<T>(x, y, x0, y0, w);
    const int ix = centre_index(x0), iy = centre_index(y0);

    uint32_t col_off[WN], row_off[WN];   // byte offsets of tap columns / rows in k and v
    uint32_t col_pix[GATHER ? 1 : WN], row_pix[GATHER ? 1 : WN];   // the same in pixels, for the fp32 accumulators
#pragma unroll
    for (int i = 0; i < WN; ++i) {
        const uint32_t cp = (uint32_t)(b * A.N + clampi(ix + i - R, 0, A.W - 1));
        const uint32_t rp = (uint32_t)(clampi(iy + i - R, 0, A.H - 1) * A.W);
        if constexpr (!GATHER) { col_pix[i] = cp; row_pix[i] = rp; }
        col_off[i] = carries ? cp * row_bytes + chan_bytes : kDead;
        row_off[i] = carries ? rp * row_bytes : 0u;   // kDead + row offset must not wrap
    }
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t rg = make_rsrc(A.d_out, total_bytes);
    const uint32_t q_off = carries ? (uint32_t)pix * row_bytes + chan_bytes : kDead;
    const u32x4 qv = buf_load16(rq, q_off);
    const u32x4 gv = buf_load16(rg, q_off);

    // ---- forward recompute: logits and softmax state ------------------------------------------
    float lg[WN][WN];
#pragma unroll
    for (int j = 0; j < WN; ++j) {
        u32x4 kv[WN];
#pragma unroll
        for (int i = 0; i < WN; ++i) kv[i] = buf_load16(rk, row_off[j] + col_off[i]);
#pragma unroll
        for (int i = 0; i < WN; ++i) {
            float s = group_sum<LPH>(l1_accum<T>(qv, kv[i], 0.f));
            lg[j][i] = Tr::round(-Tr::round(s) * A.scale);
        }
    }
    SoftmaxState<R> st;
    const bool shared = softmax_prepare<R>(lg, st);
    if (shared) softmax_shared_exp<R>(lg, w, st); else softmax_exact<R>(lg, w, st, false);
    float c9[3][3];
    coef9<R>(st.c, c9);

    float go[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) go[e] = vec_elem<T>(gv, e);

    // ---- g_m = dA_m + <dO, v_m>, and dV scatter -------------------------------------------------
    float g[WN][WN];
    const T *da = A.d_attn ? (const T *)A.d_attn + (size_t)hq * M : nullptr;
#pragma unroll
    for (int j = 0; j < WN; ++j) {
        u32x4 vv[WN];
#pragma unroll
        for (int i = 0; i < WN; ++i) vv[i] = buf_load16(rv, row_off[j] + col_off[i]);
#pragma unroll
        for (int i = 0; i < WN; ++i) {
            float s = 0.f;
#pragma unroll
            for (int e = 0; e < EPV; ++e) s += go[e] * vec_elem<T>(vv[i], e);
            s = group_sum<LPH>(s);
            if (da) s += Tr::to_f(da[j * WN + i]);
            g[j][i] = s;
            const float am = Tr::round(attn_value<R>(shared, lg, st, c9, j, i));   // the stored attention value
            if constexpr (GATHER) {
                (void)am;                                   // written with dl below, as one pair
            } else if (live && am != 0.f) {
                float *dst = A.dv_acc + (size_t)(row_pix[j] + col_pix[i]) * A.C + chan;
#pragma unroll
                for (int e = 0; e < EPV; ++e) atomic_add_f32(dst + e, am * go[e]);
            }
        }
    }

    // ---- through the softmax: dw_b and dl_m (dl overwrites g) ------------------------------------
    float dw[4];
    bilinear_softmax_bwd<R>(shared, lg, st, A.scale, g, dw);
    if (sub == 0 && !tail) {
        float dx, dy;
        offset_grad<T>(x, y, dw, dx, dy);
        T *dm = (T *)A.dmo + (size_t)hq * 2;
        dm[0] = Tr::from_f(dx);
        dm[1] = Tr::from_f(dy);
        if constexpr (GATHER) {
            typename PairOf<T>::Word *dst = (typename PairOf<T>::Word *)A.dl_ws;
            const PairLayout pairs((uint32_t)head, (uint32_t)M, (uint32_t)A.h, A.per_head[0] != 0);
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < WN; ++i)
                    dst[(size_t)pairs.at((uint32_t)pix, (uint32_t)(j * WN + i))] =
                        PairOf<T>::pack(g[j][i], Tr::round(attn_value<R>(shared, lg, st, c9, j, i)));
        }
    }

    // ---- dQ (registers) and dK scatter ---------------------------------------------------------
    float qf[EPV], dq[EPV];
#pragma unroll
    for (int e = 0; e < EPV; ++e) { qf[e] = vec_elem<T>(qv, e); dq[e] = 0.f; }
#pragma unroll
    for (int j = 0; j < WN; ++j) {
        u32x4 kv[WN];
#pragma unroll
        for (int i = 0; i < WN; ++i) kv[i] = buf_load16(rk, row_off[j] + col_off[i]);
#pragma unroll
        for (int i = 0; i < WN; ++i) {
            const float dl = g[j][i];
            if constexpr (GATHER) {
#pragma unroll
                for (int e = 0; e < EPV; ++e) dq[e] -= dl * sign_f(qf[e] - vec_elem<T>(kv[i], e));
            } else {
                float *dst = A.dk_acc + (size_t)(row_pix[j] + col_pix[i]) * A.C + chan;
                const bool push = live && dl != 0.f;
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    const float t = dl * sign_f(qf[e] - vec_elem<T>(kv[i], e));
                    dq[e] -= t;
                    if (push) atomic_add_f32(dst + e, t);
                }
            }
        }
    }
    if (live) *(u32x4 *)((char *)A.dq + (size_t)pix * row_bytes + chan_bytes) = vec_pack<T>(dq);
}

// ---------------------------------------------------------------------------------------
// Generic backward: one lane per head-query, any head size.
// ---------------------------------------------------------------------------------------
template <typename T, int R>
__global__ __launch_bounds__(256) void bwd_generic_kernel(BwdArgs A) {
    typedef Traits<T> Tr;
    constexpr int WN = 2 * R + 2, M = WN * WN;
    const long long hq = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (hq >= A.nhq) return;
    const int CH = A.C / A.h;
    const long long pix = hq / A.h;
    const int head = (int)(hq - pix * A.h);
    const long long b = pix / A.N;
    const T *mo = (const T *)A.mo + hq * 2;
    const float x = Tr::to_f(mo[0]), y = Tr::to_f(mo[1]);
    float x0, y0, w[4];
    corner_weights<T>(x, y, x0, y0, w);
    const int ix = centre_index(x0), iy = centre_index(y0);
    const long long hoff = head * CH;
    const T *qp = (const T *)A.q + pix * A.C + hoff;
    const T *gp = (const T *)A.d_out + pix * A.C + hoff;
    const long long boff = b * A.N * A.C + hoff;
    const T *kb = (const T *)A.k + boff;
    const T *vb = (const T *)A.v + boff;

    long long tap[WN][WN];
    float lg[WN][WN];
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WN; ++i) {
            tap[j][i] = ((long long)clampi(iy + j - R, 0, A.H - 1) * A.W + clampi(ix + i - R, 0, A.W - 1)) * A.C;
            const T *kp = kb + tap[j][i];
            float s = 0.f;
            for (int c = 0; c < CH; ++c) s += __builtin_fabsf(Tr::round(Tr::to_f(qp[c]) - Tr::to_f(kp[c])));
            lg[j][i] = Tr::round(-Tr::round(s) * A.scale);
        }
    SoftmaxState<R> st;
    const bool shared = softmax_prepare<R>(lg, st);
    if (shared) softmax_shared_exp<R>(lg, w, st); else softmax_exact<R>(lg, w, st, false);
    float c9[3][3];
    coef9<R>(st.c, c9);
    float g[WN][WN];
    const T *da = A.d_attn ? (const T *)A.d_attn + hq * M : nullptr;
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WN; ++i) {
            const T *vp = vb + tap[j][i];
            float *dst = A.dv_acc + boff + tap[j][i];
            const float am = Tr::round(attn_value<R>(shared, lg, st, c9, j, i));
            float s = da ? Tr::to_f(da[j * WN + i]) : 0.f;
            for (int c = 0; c < CH; ++c) {
                const float go = Tr::to_f(gp[c]);
                s += go * Tr::to_f(vp[c]);
                if (am != 0.f) atomic_add_f32(dst + c, am * go);
            }
            g[j][i] = s;
        }
    float dw[4];
    bilinear_softmax_bwd<R>(shared, lg, st, A.scale, g, dw);
    float dx, dy;
    offset_grad<T>(x, y, dw, dx, dy);
    T *dm = (T *)A.dmo + hq * 2;
    dm[0] = Tr::from_f(dx);
    dm[1] = Tr::from_f(dy);
    T *dqp = (T *)A.dq + pix * A.C + hoff;
    for (int c = 0; c < CH; ++c) {
        const float qc = Tr::to_f(qp[c]);
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                const float t = g[j][i] * sign_f(qc - Tr::to_f(kb[tap[j][i] + c]));
                s -= t;
                if (t != 0.f) atomic_add_f32(A.dk_acc + boff + tap[j][i] + c, t);
            }
        dqp[c] = Tr::from_f(s);
    }
}

}  // namespace ma

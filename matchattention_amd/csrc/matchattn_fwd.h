// Forward kernels of the MatchAttention operator for gfx950.
//
// Definition followed (reference, PyTorch path): models/mat_pytorch_impl.py:3-178
// sequenced by models/attention_blocks.py:82-91.  One fused pass replaces the seven
// launches of models/src/match_former_fused_forward.cu:531-623.
#pragma once
#include <type_traits>

#include "matchattn_softmax.h"

namespace ma {

struct FwdArgs {
    const void *mo, *q, *k, *v;
    void *out, *attn;
    int nhq;      // B*N*h head-queries
    int N, H, W, C, h;
    int h_log2;   // log2(h) when h is a power of two, else -1
    int hpg_log2; // fp16 kernel: log2 of the heads per block group (a power of two dividing h)
    float scale;
    int row_skip; // allow skipping the last window row when every lane has integer y
    int xcd_swizzle;
    const uint8_t *defer; // generic kernel: optional [nhq] flags, compute only the head-queries whose flag is set; or null
    // Output placement.  `out` holds one row of C values per pixel every out_row_bytes, `attn` one row of h*M
    // values per pixel every attn_row_bytes (contiguous tensors: C*sizeof(T) and h*M*sizeof(T)); both may be
    // column ranges of one wider matrix.  With `gate` ([pixels][C], contiguous) the value stored is
    // round(gate * round(out)), the product the attention module forms after the operator
    // (models/attention_blocks.py:96).
    uint32_t out_row_bytes, attn_row_bytes;
    const void *gate;
    // Sampling positions.  rel_heads == 0: `mo` holds them, [pixels][h][2], already clamped by the caller.  Otherwise
    // `mo` holds positions relative to each query pixel, [pixels][rel_heads][2] with rel_heads == h, or 1 for one
    // position every head shares, and the kernel itself adds the pixel's coordinates and clamps the sum to
    // [lo, hi] (sampling_position below; the kernels that read a position once per head-query do this, the LDS-tile
    // path is given positions a pass of its own has prepared).
    int rel_heads;
    float lo_x, hi_x, lo_y, hi_y;
};

// bytes the output views span (the last row ends with its data, not with its stride)
__host__ __device__ inline uint32_t out_span_bytes(const FwdArgs &A, uint32_t elem) {
    return (uint32_t)(A.nhq / A.h - 1) * A.out_row_bytes + (uint32_t)A.C * elem;
}
__host__ __device__ inline uint32_t attn_span_bytes(const FwdArgs &A, uint32_t row_elems, uint32_t elem) {
    return (uint32_t)(A.nhq / A.h - 1) * A.attn_row_bytes + row_elems * elem;
}

// Buckets produced by the tile sort (see SortArgs): a bucket is (batch item, tile row, tile column).
struct TileSort {
    const int *count;      // [h][nbins]  start of the bucket within its tile row
    const int *rowtot;     // [h][nrows]  start of the tile row
    const int *per_head;   // [0] != 0: every head has its own buckets, else head 0's serve all
    const int *perm;       // [h][L] pixel indices in bucket order
    uint8_t *defer;        // [nhq] written for every head-query: 1 = left for the generic kernel
    int *chunk_start;      // [nbins + 1] chunks of the buckets before each one, and their total
    int2 *chunk_item;      // [chunk_cap] work list: (bucket, index of the chunk within it)
    int chunk_cap;
    int bins_per_row, nbins, nrows, rows_per_img, L;     // in tiles
    int sub;               // `count` holds `sub` entries per tile (sub-buckets by the window's row in the tile), tile-major
    int *queue;            // [8] zero on entry: next unclaimed item of each XCD's share of the work list
    int *xcd_bounds;       // [9] chunks [xcd_bounds[x], xcd_bounds[x + 1]) of the work list are XCD x's share (equal cost)
};

// Map the hardware workgroup id to a logical one so that each of the 8 XCDs
// (workgroup ids are dealt to them round-robin) walks one contiguous eighth of the
// image: its L2 then holds one band of K/V rows instead of all of them.
__device__ __forceinline__ unsigned logical_block(unsigned bid, unsigned nblocks, int enable) {
    if (!enable || nblocks < 16) return bid;
    const unsigned per = nblocks >> 3;        // blocks per XCD, remainder handled below
    const unsigned body = per << 3;
    if (bid >= body) return bid;              // tail blocks keep their id
    return (bid & 7u) * per + (bid >> 3);
}

// fractional parts and corner weights, with the arithmetic rounded as the input dtype does
// (models/mat_pytorch_impl.py:11-25 runs in the tensor's dtype).
template <typename T>
__device__ __forceinline__ void corner_weights(float x, float y, float &x0, float &y0, float (&w)[4]) {
    typedef Traits<T> Tr;
    x0 = floorf(x);
    y0 = floorf(y);
    const float fx = x - x0, fy = y - y0;          // exact in every supported dtype
    const float gx = Tr::round(1.0f - fx), gy = Tr::round(1.0f - fy);
    w[0] = Tr::round(gx * gy);
    w[1] = Tr::round(fx * gy);
    w[2] = Tr::round(gx * fy);
    w[3] = Tr::round(fx * fy);
}

// The sampling position of (pixel, head).  With relative positions this is what the attention layer and module
// compute in four elementwise launches before the operator (models/attention_blocks.py:149-151 or 162-163: the
// pixel's own coordinates are added in the tensor dtype -- coordinates beyond the dtype's exact integers round as
// torch.arange in that dtype does; :45-59, :79: clamp to [r, size-1-r-1e-3] with the bounds rounded to the tensor
// dtype; torch.clamp keeps NaN).
template <typename T>
__device__ __forceinline__ void sampling_position(const FwdArgs &A, long long pix, int head, float &x, float &y) {
    typedef Traits<T> Tr;
    const long long at = A.rel_heads == 1 ? pix : pix * A.h + head;
    const T *p = (const T *)A.mo + at * 2;
    x = Tr::to_f(p[0]);
    y = Tr::to_f(p[1]);
    if (A.rel_heads != 0) {
        const int n = (int)(pix % A.N), py = n / A.W, px = n - py * A.W;
        x = Tr::round(x + Tr::round((float)px));
        y = Tr::round(y + Tr::round((float)py));
        x = x != x ? x : fminf(fmaxf(x, Tr::round(A.lo_x)), Tr::round(A.hi_x));
        y = y != y ? y : fminf(fmaxf(y, Tr::round(A.lo_y)), Tr::round(A.hi_y));
    }
}

// ---------------------------------------------------------------------------------------
// Tiled kernel.  A head-query (pixel, head) is owned by LPH adjacent lanes; each lane keeps
// VPL 16-byte vectors of the head's channels, so q/out accesses of a wavefront are one
// contiguous run and every K/V tap is fetched as whole 16-byte pieces.  Partial L1 sums are
// combined with DPP inside the lane group; all lanes of a group then hold the full window
// of logits and run the window softmax redundantly (it is small next to the tap loops).
// ---------------------------------------------------------------------------------------
template <typename T, int CH, int R, int VPL>
struct TiledCfg {
    static constexpr int EPV = Traits<T>::kEPV;
    static constexpr int NV = CH / EPV;                 // 16-byte vectors per head
    static constexpr int NVL = NV / VPL;                // lanes that carry data
    static constexpr int LPH = NVL <= 1 ? 1 : NVL <= 2 ? 2 : NVL <= 4 ? 4 : NVL <= 8 ? 8 : NVL <= 16 ? 16 : NVL <= 32 ? 32 : 64;
    static_assert(CH % EPV == 0 && NV % VPL == 0 && NVL <= 64, "unsupported head size for the tiled kernel");
    static constexpr int WN = 2 * R + 2;
    static constexpr int M = WN * WN;
    static constexpr int BLOCK = 256;
    static constexpr int HQ_PER_BLOCK = BLOCK / LPH;
};

#ifndef MA_FWD_WAVES
#define MA_FWD_WAVES 4
#endif
// The 6x6 window's kernel holds 36 logits, the stage buffers and the softmax state: 226 registers in fp32.  At four
// waves per SIMD (128 registers) it spilled 219 of them; at two it runs 1.2x to 2.7x faster (bf16: 1.3x to 2.7x).
#ifndef MA_FWD_WAVES_R2
#define MA_FWD_WAVES_R2 2
#endif

// Taps are fetched in stages of G taps, double-buffered: stage s+1 is in flight while stage s
// is consumed.  Scheduling barriers between stages stop the compiler from hoisting every
// load of a phase to its top, which would pin over a hundred registers.
template <int R, int VPL> struct StageCfg {
    static constexpr int WN = 2 * R + 2;
    static constexpr int G = (R == 1) ? (VPL == 1 ? 4 : 2) : (VPL == 1 ? 6 : VPL == 2 ? 3 : 2);
    static constexpr int SPR = WN / G;          // stages per window row
    static constexpr int NS = WN * SPR;         // stages in the window
    static_assert(WN % G == 0, "stage size must divide the window row");
};

template <typename T, int CH, int R, int VPL>
__global__ __launch_bounds__(256, R == 1 ? MA_FWD_WAVES : MA_FWD_WAVES_R2) void fwd_tiled_kernel(FwdArgs A) {
    typedef TiledCfg<T, CH, R, VPL> Cfg;
    typedef StageCfg<R, VPL> St;
    typedef Traits<T> Tr;
    constexpr int EPV = Cfg::EPV, LPH = Cfg::LPH, WN = Cfg::WN, M = Cfg::M;
    constexpr int G = St::G, SPR = St::SPR;

    const unsigned blk = logical_block(blockIdx.x, gridDim.x, A.xcd_swizzle);
    const int sub = threadIdx.x % LPH;
    int hq = (int)(blk * Cfg::HQ_PER_BLOCK + threadIdx.x / LPH);
    const bool tail = hq >= A.nhq;           // whole lane groups fall off the end together
    if (tail) hq = A.nhq - 1;                // keep them in flight (DPP partners), store nothing
    const bool carries = sub < Cfg::NVL;     // lanes beyond the head's vectors only pad the group
    const bool live = carries && !tail;

    const int pix = hq / A.h, head = hq - pix * A.h;
    const int b = pix / A.N;
    const uint32_t row_bytes = (uint32_t)A.C * sizeof(T);
    const uint32_t total_bytes = (uint32_t)(A.nhq / A.h) * row_bytes;
    const uint32_t chan_bytes = (uint32_t)(head * CH + sub * VPL * EPV) * sizeof(T);
    const uint32_t kDead = 0xFFFFFF00u;      // beyond any buffer: the load returns zeros

    // sampling centre
    float x, y;
    sampling_position<T>(A, pix, head, x, y);
    float x0, y0, w[4];
    corner_weights<T>(x, y, x0, y0, w);
    const int ix = centre_index(x0), iy = centre_index(y0);
    const bool skip_last = A.row_skip && __builtin_amdgcn_ballot_w64(y != y0) == 0;

    // Window fully inside the image for every lane (always so behind the module's clamp in
    // fp32; in fp16 the clamp's upper bound can round up by one): tap (j, i) then sits at a
    // fixed, wavefront-uniform distance from tap (0, 0) and needs no per-lane address math.
    const bool inside = ix - R >= 0 && ix + R + 1 <= A.W - 1 && iy - R >= 0 && iy + R + 1 <= A.H - 1;
    const bool linear = __builtin_amdgcn_ballot_w64(!inside) == 0;
    const uint32_t tap0_off =
        carries ? (uint32_t)(b * A.N + clampi(iy - R, 0, A.H - 1) * A.W + clampi(ix - R, 0, A.W - 1)) * row_bytes + chan_bytes
                : kDead;

    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(A.out, out_span_bytes(A, sizeof(T)));
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A.attn, attn_span_bytes(A, (uint32_t)(A.h * M), sizeof(T)));
    const __amdgpu_buffer_rsrc_t rgate = make_rsrc(A.gate, A.gate ? total_bytes : 0u);

    u32x4 qv[VPL];
    const uint32_t q_off = carries ? (uint32_t)pix * row_bytes + chan_bytes : kDead;
#pragma unroll
    for (int u = 0; u < VPL; ++u) qv[u] = buf_load16(rq, q_off + u * 16);

    // The last window row is left out (NROWS = WN-1) when its weights are exactly zero for
    // every lane of the wavefront (integer y: stereo).  The two bodies are separate
    // instantiations so that each is straight-line code.
    auto body = [&](auto nrows_tag, auto linear_tag) __attribute__((always_inline)) {
        constexpr int NROWS = decltype(nrows_tag)::value;
        constexpr bool LINEAR = decltype(linear_tag)::value;
        // clamped addressing: one offset per window column and per window row
        uint32_t col_off[WN], row_off[WN];
        if constexpr (!LINEAR) {
#pragma unroll
            for (int i = 0; i < WN; ++i) {
                col_off[i] = carries ? (uint32_t)(b * A.N + clampi(ix + i - R, 0, A.W - 1)) * row_bytes + chan_bytes : kDead;
                // padding lanes keep a zero row offset so that kDead + row offset cannot wrap into the buffer
                row_off[i] = carries ? (uint32_t)(clampi(iy + i - R, 0, A.H - 1) * A.W) * row_bytes : 0u;
            }
        }
        constexpr int NSR = NROWS * SPR;            // stages actually run
        u32x4 buf[2][G][VPL];
        auto fetch = [&](const __amdgpu_buffer_rsrc_t &r, auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
#pragma unroll
            for (int t = 0; t < G; ++t)
#pragma unroll
                for (int u = 0; u < VPL; ++u)
                    if constexpr (LINEAR)
                        buf[s & 1][t][u] = buf_load16(r, tap0_off + u * 16, (uint32_t)(j * A.W + i0 + t) * row_bytes);
                    else
                        buf[s & 1][t][u] = buf_load16(r, row_off[j] + col_off[i0 + t] + u * 16);
        };

        // ---- logits: -scale * sum_c |q_c - k_c| for every tap -----------------------------
        float lg[WN][WN];
#pragma unroll
        for (int i = 0; i < WN; ++i) lg[WN - 1][i] = -__builtin_inff();   // stays if the row is left out
        fetch(rk, std::integral_constant<int, 0>{});
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) fetch(rk, std::integral_constant<int, s + 1>{});
#pragma unroll
            for (int t = 0; t < G; ++t) {
                float sum = 0.f;
#pragma unroll
                for (int u = 0; u < VPL; ++u) sum = l1_accum<T>(qv[u], buf[s & 1][t][u], sum);
                sum = group_sum<LPH>(sum);
                // rounding points of the half-precision definition: the channel sum and the
                // scaled logit are each stored in the tensor dtype
                lg[j][i0 + t] = Tr::round(-Tr::round(sum) * A.scale);
            }
            __builtin_amdgcn_sched_barrier(0);
        });

        // ---- window softmax (in place: lg becomes the attention weights) -------------------
        fetch(rv, std::integral_constant<int, 0>{});   // first V stage travels while the softmax runs
        SoftmaxState<R> st;
        bilinear_softmax_fwd<R>(lg, w, st);
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) lg[j][i] = Tr::round(lg[j][i]);   // attn is stored, and reused, in T
        __builtin_amdgcn_sched_barrier(0);

        // ---- aggregation: out_c = sum_m a_m * v[tap m]_c --------------------------------------
        float acc[VPL][EPV];
#pragma unroll
        for (int u = 0; u < VPL; ++u)
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[u][e] = 0.f;
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) fetch(rv, std::integral_constant<int, s + 1>{});
            if constexpr (std::is_same<T, bf16_t>::value && G % 2 == 0 && R == 1) {
                // (the 4x4 window only: with the 6x6 window's register budget of four waves per SIMD this form spills)
                // bf16, two taps at a time: the weights (already bf16 values) packed as a pair, a channel's two values
                // gathered into one word by a byte permute, one bf16 dot product per channel and tap pair
#pragma unroll
                for (int t = 0; t < G; t += 2) {
                    const bf16x2_t wp = {(__bf16)lg[j][i0 + t], (__bf16)lg[j][i0 + t + 1]};
#pragma unroll
                    for (int u = 0; u < VPL; ++u)
#pragma unroll
                        for (int p = 0; p < 4; ++p) {
                            const uint32_t w0 = buf[s & 1][t][u][p], w1 = buf[s & 1][t + 1][u][p];
                            const uint32_t lo = __builtin_amdgcn_perm(w1, w0, 0x05040100u), hi = __builtin_amdgcn_perm(w1, w0, 0x07060302u);
                            acc[u][2 * p] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, lo), wp, acc[u][2 * p], false);
                            acc[u][2 * p + 1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, hi), wp, acc[u][2 * p + 1], false);
                        }
                }
            } else {
#pragma unroll
                for (int t = 0; t < G; ++t)
#pragma unroll
                    for (int u = 0; u < VPL; ++u)
#pragma unroll
                        for (int e = 0; e < EPV; ++e) acc[u][e] += lg[j][i0 + t] * vec_elem<T>(buf[s & 1][t][u], e);
            }
            __builtin_amdgcn_sched_barrier(0);
        });

        // Stores are predicated through the buffer range check rather than a branch: a branch
        // would let the compiler sink the whole accumulation into it, keeping every fetched
        // vector alive until then.
        const uint32_t o_off = live ? (uint32_t)pix * A.out_row_bytes + chan_bytes : kDeadOffset;
        u32x4 ov[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) ov[u] = vec_pack<T>(acc[u]);
        if (A.gate) {
#pragma unroll
            for (int u = 0; u < VPL; ++u) ov[u] = vec_mul<T>(ov[u], buf_load16(rgate, q_off + u * 16));
        }
#pragma unroll
        for (int u = 0; u < VPL; ++u) buf_store16(ro, o_off + u * 16, ov[u]);
        // attn row of this head-query: M values of T, written by the group's first lane
        const uint32_t a_off = (sub == 0 && !tail) ? (uint32_t)pix * A.attn_row_bytes + (uint32_t)head * (uint32_t)(M * sizeof(T))
                                                   : kDeadOffset;
        constexpr int PER8 = 8 / sizeof(T);       // elements per 8-byte store (M*sizeof(T) % 8 == 0)
        const float *af = &lg[0][0];
#pragma unroll
        for (int m = 0; m < M; m += PER8) {
            u32x2 pk;
            if constexpr (sizeof(T) == 4) {
                pk = u32x2{as_u32(af[m]), as_u32(af[m + 1])};
            } else {
                T t4[4] = {Tr::from_f(af[m]), Tr::from_f(af[m + 1]), Tr::from_f(af[m + 2]), Tr::from_f(af[m + 3])};
                pk = __builtin_bit_cast(u32x2, t4);
            }
            buf_store8(ra, a_off + m * sizeof(T), pk);
        }
    };
    if (!linear)
        body(std::integral_constant<int, WN>{}, std::false_type{});
    else if (skip_last)
        body(std::integral_constant<int, WN - 1>{}, std::true_type{});
    else
        body(std::integral_constant<int, WN>{}, std::true_type{});
}

// ---------------------------------------------------------------------------------------
// Generic kernel: one lane per head-query, any head size, window radius up to kMaxR,
// element-wise loads with 64-bit addressing.  Slow; it exists so that every shape the
// operator accepts has a path (e.g. tensors above 4 GiB, head sizes that are not a
// multiple of a 16-byte vector).
// ---------------------------------------------------------------------------------------
template <typename T, int R> __device__ __forceinline__ void fwd_generic_one(const FwdArgs &A, long long hq);

template <typename T, int R>
__global__ __launch_bounds__(256) void fwd_generic_kernel(FwdArgs A) {
    if (A.defer) {
        // flag mode: a fixed grid scans the flags another kernel left, 16 at a time, and computes the
        // (normally very few) head-queries that are set
        const int nvec = (A.nhq + 15) / 16;
        for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += gridDim.x * blockDim.x) {
            const int base = i * 16;
            if (base + 16 <= A.nhq && (reinterpret_cast<uintptr_t>(A.defer) & 15u) == 0) {
                const u32x4 f = *(const u32x4 *)(A.defer + base);
                if ((f[0] | f[1] | f[2] | f[3]) == 0) continue;
            }
            for (int e = 0; e < 16 && base + e < A.nhq; ++e)
                if (A.defer[base + e]) fwd_generic_one<T, R>(A, (long long)(base + e));
        }
        return;
    }
    const long long hq = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (hq >= A.nhq) return;
    fwd_generic_one<T, R>(A, hq);
}

template <typename T, int R>
__device__ __forceinline__ void fwd_generic_one(const FwdArgs &A, long long hq) {
    typedef Traits<T> Tr;
    constexpr int WN = 2 * R + 2, M = WN * WN;
    const int CH = A.C / A.h;
    const long long pix = hq / A.h;
    const int head = (int)(hq - pix * A.h);
    const long long b = pix / A.N;
    float x, y;
    sampling_position<T>(A, pix, head, x, y);
    float x0, y0, w[4];
    corner_weights<T>(x, y, x0, y0, w);
    const int ix = centre_index(x0), iy = centre_index(y0);
    const T *qp = (const T *)A.q + pix * A.C + head * CH;
    const T *kb = (const T *)A.k + b * A.N * A.C + head * CH;
    const T *vb = (const T *)A.v + b * A.N * A.C + head * CH;

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
    bilinear_softmax_fwd<R>(lg, w, st);
    float (&a)[WN][WN] = lg;
    T *ap = (T *)((char *)A.attn + (size_t)pix * A.attn_row_bytes) + head * M;
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int i = 0; i < WN; ++i) {
            a[j][i] = Tr::round(a[j][i]);
            ap[j * WN + i] = Tr::from_f(a[j][i]);
        }
    T *op = (T *)((char *)A.out + (size_t)pix * A.out_row_bytes) + head * CH;
    const T *gp = A.gate ? (const T *)A.gate + pix * A.C + head * CH : nullptr;
    for (int c = 0; c < CH; ++c) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) s += a[j][i] * Tr::to_f(vb[tap[j][i] + c]);
        op[c] = gp ? Tr::from_f(Tr::round(s) * Tr::to_f(gp[c])) : Tr::from_f(s);
    }
}

}  // namespace ma

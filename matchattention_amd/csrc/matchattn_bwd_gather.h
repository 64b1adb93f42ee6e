// Backward, pass B: dK and dV gathered per key (deterministic, no atomics).
//
// Pass A (bwd_tiled_kernel in gather mode) leaves for every head-query its per-tap logit
// gradient dl[hq][m] and attention weight a[hq][m].  An inverse index of the sampling centres
// (counting sort with one bin per target pixel, matchattn_sort.h) lists, for every pixel, the
// queries centred on it.  A key (kx, ky) is touched only by queries centred within the window
// reach: target rows ky-R-1 .. ky+R and, in each, the contiguous run of bins kx-R-1 .. kx+R.
// For a candidate with true (unclamped) centre (cx, cy) the taps that land on the key are the
// intervals { i : clamp(cx+i-R) == kx } x { j : clamp(cy+j-R) == ky } -- a single tap for
// interior keys, several when the replicate clamp folds taps onto a border key.
//   dk[key] = sum dl[hq][m] * sgn(q[hq] - k[key]),   dv[key] = sum a[hq][m] * dO[hq]
#pragma once
#include "matchattn_bwd.h"

namespace ma {

// taps t in [0, WN) with clamp(c + t - R, 0, n-1) == key
__device__ __forceinline__ void tap_interval(int c, int key, int n, int R, int WN, int &lo, int &hi) {
    if (key > 0 && key < n - 1) { lo = hi = key - c + R; }
    else if (key == 0) { lo = 0; hi = R - c; }
    else { lo = n - 1 - c + R; hi = WN - 1; }
    lo = max(lo, 0);
    hi = min(hi, WN - 1);      // empty when lo > hi
}

// Vectors per lane of pass B.  The (dl, a) fetch and the addressing of a candidate are shared by all vectors of a
// lane, so two vectors per lane save instructions per key -- but cost registers, i.e. waves in flight, and memory
// and arithmetic of a wave do not overlap much here (switching off the pair loads, the q/dO loads or the sums each
// shortens the kernel by about a third), so waves in flight matter more: one vector per lane runs at 96 registers,
// 5 waves per SIMD, two at 128 and 4.  Measured (fp16, 32 channels per head, 6x6 window): one vector is 1 % faster
// with a shared offset and 1.5 % faster with per-head offsets; with the 4x4 window 10 %.  Squeezing the registers
// further (6 or 8 waves) spills.
// (heads of more than 16 vectors -- 80, 96, 128 fp32 channels, 192 in the 16-bit types -- take two per lane)
template <typename T, int CH, int R> struct KeyVpl { static constexpr int value = CH * (int)sizeof(T) > 256 ? 2 : 1; };

// COMPACT (maps below 2^25 pixels whose pair array stays below 4 GiB: chosen by the host): away from the border a
// prepared candidate travels as one word, (query pixel << 6) | tap, or -1 for none -- one lane exchange instead of two
// and nothing to unpack -- and its pair is fetched through a buffer descriptor, whose range check stands in for the
// selects a missing candidate otherwise needs (an offset beyond the array reads zeros).
template <typename T, int CH, int R, int VPL, bool COMPACT>
__global__ __launch_bounds__(256) void bwd_key_kernel(BwdArgs A) {
    typedef TiledCfg<T, CH, R, VPL> Cfg;
    constexpr int EPV = Cfg::EPV, LPH = Cfg::LPH, WN = Cfg::WN, M = Cfg::M;

    const int sub = threadIdx.x % LPH;
    // each XCD (workgroup ids are dealt to them round-robin) takes one contiguous band of keys: neighbouring
    // keys share most of their candidate queries, which then meet in one L2.  Not with an index per head and 16-bit
    // tensors: the heads of a key then walk eight unrelated lists, and dealing the blocks round-robin measured 4 %
    // faster in fp16 (2 x 384 x 384, 8 heads, offsets N(0, 24 px) per head: 3.22 -> 3.09 ms for the whole backward),
    // the same in bf16 and 4 % slower in fp32 (4.23 -> 4.42 ms), which keeps its bands.
    const unsigned blk = logical_block(blockIdx.x, gridDim.x, A.xcd_swizzle && (A.per_head[0] == 0 || sizeof(T) == 4));
    int khq = (int)(blk * Cfg::HQ_PER_BLOCK + threadIdx.x / LPH);   // (key pixel, head)
    const bool tail = khq >= A.nhq;
    if (tail) khq = A.nhq - 1;
    const bool carries = sub < Cfg::NVL;
    const bool live = carries && !tail;
    const int kp = khq / A.h, head = khq - kp * A.h;
    const int b = kp / A.N, kn = kp - b * A.N;
    const int ky = kn / A.W, kx = kn - ky * A.W;
    const int npix = A.nhq / A.h;
    const uint32_t row_bytes = (uint32_t)A.C * sizeof(T);
    const uint32_t total_bytes = (uint32_t)npix * row_bytes;
    const uint32_t chan_bytes = (uint32_t)(head * CH + sub * VPL * EPV) * sizeof(T);    // vector u of the lane: + 16 u
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rg = make_rsrc(A.d_out, total_bytes);
    [[maybe_unused]] const __amdgpu_buffer_rsrc_t rp =
        make_rsrc(A.dl_ws, COMPACT ? (uint32_t)A.nhq * (uint32_t)(M * PairOf<T>::kBytes) : 0u);

    u32x4 kv[VPL];
    float dk[VPL][EPV], dv[VPL][EPV];
#pragma unroll
    for (int w = 0; w < VPL; ++w) {
        kv[w] = buf_load16(rk, (carries ? (uint32_t)kp * row_bytes + chan_bytes : kDeadOffset) + w * 16);
#pragma unroll
        for (int e = 0; e < EPV; ++e) { dk[w][e] = 0.f; dv[w][e] = 0.f; }
    }

    const bool pairs_per_head = A.per_head[0] != 0;    // (also the layout of the pair array: PairLayout)
    const int src = pairs_per_head ? head : 0;         // whose index lists this head's queries
    const PairLayout pairs((uint32_t)head, (uint32_t)M, (uint32_t)A.h, pairs_per_head);
    const int *perm = A.perm + (size_t)src * npix;
    const int *centre = A.centre + (size_t)src * npix;
    const int *bin_start = A.bin_start + (size_t)src * A.nrows * A.W;   // start of a bin within its row
    const int *row_start = A.row_start + (size_t)src * A.nrows;

    // Candidate entries: for each of the 2R+2 target rows around the key, one contiguous run of the index
    // (bins kx-R-1 .. kx+R of that row).  All run bounds are fetched at once, the runs are then walked as one
    // flat sequence, U entries per step, with the next step's index entries already in flight.
    const int bx_lo = max(kx - R - 1, 0), bx_hi = min(kx + R, A.W - 1);
    int rpos[WN], cum[WN + 1], shift[WN];
    cum[0] = 0;
#pragma unroll
    for (int r = 0; r < WN; ++r) {
        const int by = ky - R - 1 + r;
        const bool in = by >= 0 && by <= A.H - 1;
        const int row = b * A.H + clampi(by, 0, A.H - 1);
        const int base = row_start[row];
        const int row_end = row + 1 < A.nrows ? row_start[row + 1] : npix;
        const int first = bin_start[(size_t)row * A.W + bx_lo];
        const int last = bin_start[(size_t)row * A.W + min(bx_hi + 1, A.W - 1)];
        const int pos = clampi(base + first, 0, npix);    // (the index is scratch memory: never trust it for addressing)
        const int end = clampi(bx_hi + 1 < A.W ? base + last : row_end, pos, npix);
        rpos[r] = pos;
        shift[r] = pos - cum[r];
        cum[r + 1] = cum[r] + (in ? end - pos : 0);
    }
    const int total = cum[WN];
    // flat candidate number -> position in the index: the last run that starts at or before t holds t.  As a sum of
    // steps, in registers: a chain of selects between the shifts is turned by the compiler into a selected index
    // into a table it keeps in LDS, one LDS round trip per chunk of candidates (cfg2 backward 4 % slower).
    int dshift[WN];
#pragma unroll
    for (int r = 1; r < WN; ++r) dshift[r] = shift[r] - shift[r - 1];
    auto locate = [&](int t) __attribute__((always_inline)) {
        int d = shift[0];
#pragma unroll
        for (int r = 1; r < WN; ++r) d += t >= cum[r] ? dshift[r] : 0;
        return min(t + d, npix - 1);
    };
    // every key of the wavefront away from the map's border: a candidate then reaches its key through exactly one tap
    const bool one_tap = __builtin_amdgcn_ballot_w64(!(kx > 0 && kx < A.W - 1 && ky > 0 && ky < A.H - 1)) == 0;
    // The walk itself -- position in the index, query pixel, centre, taps -- is the same for every lane that works on
    // the same key with the same index: the LPH lanes of a head, and all h*LPH lanes of a key pixel when the heads
    // share one offset.  The GW lanes of such a group split it: each prepares one candidate of a chunk of GW and
    // the group then goes through the chunk together, fetching each prepared candidate from its lane.
    // (A group lies within one wavefront and starts at a multiple of GW: 256/LPH head-queries per block, h | 256/LPH.)
    const int whole = A.h * LPH;
    const int GW = (A.per_head[0] == 0 && (whole & (whole - 1)) == 0 && whole <= 64 && (Cfg::HQ_PER_BLOCK % A.h) == 0) ? whole : LPH;
    const int lane = (int)(threadIdx.x & 63), gl = lane & (GW - 1), gb = lane - gl;
    constexpr int U = 1;                               // candidates per batch (independent loads)
    const int step = min(U, GW);                       // a batch lies within one chunk
    struct Batch { float dl[U], am[U]; u32x4 qv[U][VPL], gv[U][VPL]; };
    // my candidate of the chunk that starts at t0: which taps of its window land on the key
    // (packed: hit | j_hi | j_lo | i_hi | i_lo)
    auto make_info = [&](int t0, int cc) __attribute__((always_inline)) {
        const int cx = (int)(int16_t)(cc & 0xffff), cy = cc >> 16;
        int i_lo, i_hi, j_lo, j_hi;
        tap_interval(cx, kx, A.W, R, WN, i_lo, i_hi);
        tap_interval(cy, ky, A.H, R, WN, j_lo, j_hi);
        const bool hit = t0 + gl < total && i_lo <= i_hi && j_lo <= j_hi;
        return hit ? (1 << 12) | (j_hi << 9) | (j_lo << 6) | (i_hi << 3) | i_lo : 0;
    };
    // the same for a key away from the border, as one word: (query pixel << 6) | tap, or -1
    [[maybe_unused]] auto make_word = [&](int t0, int cc, int qp) __attribute__((always_inline)) {
        const int cx = (int)(int16_t)(cc & 0xffff), cy = cc >> 16;
        const int i = kx - cx + R, j = ky - cy + R;
        const bool hit = t0 + gl < total && i >= 0 && i < WN && j >= 0 && j < WN;
        return hit ? (qp << 6) | (j * WN + i) : -1;
    };
    auto sum = [&](const Batch &bt) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if constexpr (std::is_same<T, half_t>::value) {
                // packed fp16 difference (exact sign); sgn(d) per element as in pass A: the half times 2^60 in one
                // mixed-precision instruction, the median of (x, -1, 1), a plain fp32 multiply-add; dO is read by its
                // multiply-add as a half-precision operand
#pragma unroll
                for (int w = 0; w < VPL; ++w)
#pragma unroll
                    for (int p2 = 0; p2 < 4; ++p2) {
                        const half2_t d = as_h2(bt.qv[u][w][p2]) - as_h2(kv[w][p2]);
                        const half2_t gp = as_h2(bt.gv[u][w][p2]);
                        const float s0 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)d.x, 0x1p60f, 0.0f), -1.0f, 1.0f);
                        const float s1 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)d.y, 0x1p60f, 0.0f), -1.0f, 1.0f);
                        dk[w][2 * p2] = __builtin_fmaf(s0, bt.dl[u], dk[w][2 * p2]);
                        dk[w][2 * p2 + 1] = __builtin_fmaf(s1, bt.dl[u], dk[w][2 * p2 + 1]);
                        dv[w][2 * p2] += bt.am[u] * (float)gp.x;
                        dv[w][2 * p2 + 1] += bt.am[u] * (float)gp.y;
                    }
            } else {
#pragma unroll
                for (int w = 0; w < VPL; ++w)
#pragma unroll
                    for (int e = 0; e < EPV; ++e) {
                        dk[w][e] += bt.dl[u] * sign_f(vec_elem<T>(bt.qv[u][w], e) - vec_elem<T>(kv[w], e));
                        dv[w][e] += bt.am[u] * vec_elem<T>(bt.gv[u][w], e);
                    }
            }
        }
    };
    // (two copies of the walk: with the data-dependent number of loads of the border case in the loop the compiler
    // cannot count the loads in flight and waits for all of them before every batch)
    auto walk = [&](auto one_tap_tag) __attribute__((always_inline)) {
        constexpr bool ONE = decltype(one_tap_tag)::value;
        constexpr bool PACKED = ONE && COMPACT;
        int t0 = 0, tf = 0;                            // start of the prepared chunk; next candidate to fetch
        int qp_m, cc_m, qp_n, cc_n;
        { const int p = locate(gl); qp_m = clampi(perm[p], 0, npix - 1); cc_m = centre[p]; }
        { const int p = locate(GW + gl); qp_n = perm[p]; cc_n = centre[p]; }
        int info_m;
        if constexpr (PACKED) info_m = make_word(0, cc_m, qp_m); else info_m = make_info(0, cc_m);
        auto fetch = [&](Batch &bt) __attribute__((always_inline)) {
            if (tf >= t0 + GW) {                       // the chunk is used up (the same for the whole group): next one,
                t0 += GW;                              // and the index entries of the one after it go in flight
                qp_m = clampi(qp_n, 0, npix - 1);
                if constexpr (PACKED) info_m = make_word(t0, cc_n, qp_m); else info_m = make_info(t0, cc_n);
                const int p = locate(t0 + GW + gl);
                qp_n = perm[p]; cc_n = centre[p];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int idx = tf + u - t0;
                const int from = (gb + min(idx, GW - 1)) * 4;
                if constexpr (PACKED) {
                    const int word = u < step ? __builtin_amdgcn_ds_bpermute(from, info_m) : -1;
                    const bool hit = word >= 0;
                    const uint32_t qp = (uint32_t)word >> 6;
                    const uint32_t poff = hit ? pairs.at(qp, (uint32_t)word & 63u) * (uint32_t)PairOf<T>::kBytes : kDeadOffset;
                    typename PairOf<T>::Word da;
                    if constexpr (PairOf<T>::kBytes == 4) da = (typename PairOf<T>::Word)__builtin_amdgcn_raw_buffer_load_b32(rp, (int)poff, 0, 0);
                    else da = __builtin_amdgcn_raw_buffer_load_b64(rp, (int)poff, 0, 0);
                    PairOf<T>::unpack(da, bt.dl[u], bt.am[u]);
                    const uint32_t off = (carries && hit) ? qp * row_bytes + chan_bytes : kDeadOffset;
#pragma unroll
                    for (int w = 0; w < VPL; ++w) {
                        bt.qv[u][w] = buf_load16(rq, off + w * 16);
                        bt.gv[u][w] = buf_load16(rg, off + w * 16);
                    }
                    continue;
                }
                const int qp = __builtin_amdgcn_ds_bpermute(from, qp_m);
                const int info = (u < step && tf + u < total) ? __builtin_amdgcn_ds_bpermute(from, info_m) : 0;
                const bool hit = (info >> 12) != 0;
                const int i_lo = info & 7, i_hi = (info >> 3) & 7, j_lo = (info >> 6) & 7, j_hi = (info >> 9) & 7;
                if constexpr (ONE) {
                    const typename PairOf<T>::Word da = ((const typename PairOf<T>::Word *)A.dl_ws)[(size_t)pairs.at((uint32_t)qp, (uint32_t)(hit ? j_lo * WN + i_lo : 0))];
                    float dl_t, a_t;
                    PairOf<T>::unpack(da, dl_t, a_t);
                    bt.dl[u] = hit ? dl_t : 0.f;
                    bt.am[u] = hit ? a_t : 0.f;
                } else {
                    bt.dl[u] = 0.f; bt.am[u] = 0.f;
                    if (hit) {                          // several taps of one query on this key simply add up
                        for (int j = j_lo; j <= j_hi; ++j)
                            for (int i = i_lo; i <= i_hi; ++i) {
                                const typename PairOf<T>::Word da = ((const typename PairOf<T>::Word *)A.dl_ws)[(size_t)pairs.at((uint32_t)qp, (uint32_t)(j * WN + i))];
                                float dl_t, a_t;
                                PairOf<T>::unpack(da, dl_t, a_t);
                                bt.dl[u] += dl_t;
                                bt.am[u] += a_t;
                            }
                    }
                }
                const uint32_t off = (carries && hit) ? (uint32_t)qp * row_bytes + chan_bytes : kDeadOffset;
#pragma unroll
                for (int w = 0; w < VPL; ++w) {        // (the dead offset leaves room for + 16 w)
                    bt.qv[u][w] = buf_load16(rq, off + w * 16);
                    bt.gv[u][w] = buf_load16(rg, off + w * 16);
                }
            }
            tf += step;
        };
        // two batches under fixed names: while one is summed the loads of the other are in flight
        // (lane groups of a wavefront have different numbers of candidates: plain divergent loop)
        Batch b0, b1;
        if (total > 0) fetch(b0);
        for (int ts = 0; ts < total; ts += 2 * step) {
            fetch(b1);
            sum(b0);
            fetch(b0);
            sum(b1);
        }
    };
    if (one_tap) walk(std::true_type{}); else walk(std::false_type{});
    if (live) {
#pragma unroll
        for (int w = 0; w < VPL; ++w) {
            *(u32x4 *)((char *)A.dk + (size_t)kp * row_bytes + chan_bytes + w * 16) = vec_pack<T>(dk[w]);
            *(u32x4 *)((char *)A.dv + (size_t)kp * row_bytes + chan_bytes + w * 16) = vec_pack<T>(dv[w]);
        }
    }
}

}  // namespace ma

// Backward, pass A on LDS tiles (fp16, gfx950).
//
// Same work decomposition as the forward tile kernel (matchattn_fwd_tile.h): queries bucketed by the
// 16x8 tile of K/V their window centre falls in, one work item = (head group, chunk of a bucket), the
// tile plus halo of K and V staged in LDS once per item.  A pass then takes all three sweeps over the
// window from LDS -- the logits (K), g_m = dA_m + <dO, v_m> (V) and dQ = -sum_m dl_m sgn(q - k_m) (K again)
// -- where the direct kernel (matchattn_bwd.h) gathers each of them through L2.  It writes, per head-query,
// dQ, d max_offset and the (dl, a) pairs pass B consumes.
//
// Unlike the forward, nothing is skipped for integer y: the south sub-windows have zero weight there but
// their softmax still enters d max_offset.  Queries the tile cannot serve (centre far outside the image,
// exact per-sub-window softmax needed) are flagged and done by bwd_tiled_kernel afterwards.
#pragma once
#include "matchattn_bwd.h"
#include "matchattn_fwd_tile.h"

namespace ma {

template <int CH, int R, int TW, int TH, int VPL>
__global__ __launch_bounds__(kTileNT, 2) void bwd_h16_tile_kernel(BwdArgs A, TileSort S) {
    typedef half_t T;
    typedef TileCfg<CH, R, TW, TH, VPL> Cfg;
    typedef StageCfg<R, VPL> St;
    constexpr int WN = Cfg::WN, M = Cfg::M, HW = WN / 2, BW = Cfg::BW, BH = Cfg::BH;
    constexpr int GB = Cfg::GB, HPG = Cfg::HPG, CPP = Cfg::CPP, PSTR = Cfg::PSTR, LPH = Cfg::LPH, QPP = Cfg::QPP;
    constexpr int G = St::G, SPR = St::SPR, NSR = WN * SPR;

    __shared__ __attribute__((aligned(16))) char smem[2 * Cfg::TILE_BYTES];   // K tile, then V tile

    const int nhg = A.h / HPG;
    const int npix = S.L;
    const uint32_t row_bytes = (uint32_t)A.C * 2u;
    const uint32_t total_bytes = (uint32_t)npix * row_bytes;
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t rg = make_rsrc(A.d_out, total_bytes);
    const __amdgpu_buffer_rsrc_t rdq = make_rsrc(A.dq, total_bytes);
    const __amdgpu_buffer_rsrc_t rm = make_rsrc(A.mo, (uint32_t)A.nhq * 4u);
    const __amdgpu_buffer_rsrc_t rdm = make_rsrc(A.dmo, (uint32_t)A.nhq * 4u);
    const __amdgpu_buffer_rsrc_t rda = make_rsrc(A.d_attn, A.d_attn ? (uint32_t)A.nhq * (uint32_t)(M * 2) : 0u);
    const __amdgpu_buffer_rsrc_t rws = make_rsrc(A.dl_ws, (uint32_t)A.nhq * (uint32_t)(M * 4));   // (dl, a) as two halves per tap
    const bool pairs_per_head = A.per_head[0] != 0;    // layout of the pair array (PairLayout): the inverse index's flag, not the tile buckets'
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(S.defer, (uint32_t)A.nhq);
    const int sub = threadIdx.x % LPH;
    const int grp = threadIdx.x / LPH;
    const int hslot = grp % HPG, gi = grp / HPG;
    const int par = VPL == 2 ? (gi & 1) : 0;          // vector order alternates (LDS bank groups, see the forward)
    const uint32_t lane_lds = (uint32_t)(hslot * CH * 2 + sub * 16);
    uint32_t vec_off[VPL];
#pragma unroll
    for (int u = 0; u < VPL; ++u) vec_off[u] = (uint32_t)((u ^ par) * LPH * 16);
    const float nscale = -A.scale;

    const int nchunks = min(max(S.chunk_start[S.nbins], 0), S.chunk_cap);
    const int xcd = blockIdx.x & 7;
    // XCD x takes the x-th share of the work list (consecutive chunks, shares of equal cost: tile_chunks_kernel), the
    // head groups of a chunk being neighbours in the item order; bounds read from scratch memory are clamped
    const int share_lo = clampi(S.xcd_bounds[xcd], 0, nchunks), share_hi = clampi(S.xcd_bounds[xcd + 1], share_lo, nchunks);
    const int xcd_start = share_lo * nhg, item_end = share_hi * nhg;
    const bool per_head = *S.per_head != 0;
    // (the order of an item's prologue follows the forward kernel: staging addresses, the two index loads, the
    // staging loads, then the first pass's rows while the staging loads are in flight; the work-list entry is
    // fetched one item ahead)
    // items are claimed from a counter per XCD, two ahead; the index reaches the workgroup through LDS between
    // the two barriers of an item (see the fp16 forward kernel)
    __shared__ int s_claim;
    int *const queue = S.queue + xcd;
    if (threadIdx.x == 0) s_claim = atomicAdd(queue, 2);
    __syncthreads();
    const int item0 = xcd_start + *(volatile int *)&s_claim;
    int item_next = item0 + 1;
    int2 entry = int2{0, 0};
    if (item0 < item_end) entry = S.chunk_item[item0 / nhg];
    for (int item = item0; item < item_end;) {
    int claim = 0;
    if (threadIdx.x == 0) claim = atomicAdd(queue, 1);
        const int hgrp = item - (item / nhg) * nhg;
        const int bin = clampi(entry.x, 0, S.nbins - 1), part = max(entry.y, 0);
        const int head = hgrp * HPG + hslot;
        const PairLayout pairs((uint32_t)head, (uint32_t)M, (uint32_t)A.h, pairs_per_head);
        int lo, hi;
        bucket_bounds(S, per_head ? head : 0, bin, lo, hi);
        const int row = bin / S.bins_per_row, tx = bin - row * S.bins_per_row;
        const int b = min(row / S.rows_per_img, npix / A.N - 1), ty = row - (row / S.rows_per_img) * S.rows_per_img;
        const int box_x = tx * TW - R, box_y = ty * TH - R;
        lo = min(lo + part * kTileCap, hi);
        hi = min(hi, lo + kTileCap);
        const uint32_t chan_bytes = (uint32_t)(head * CH + sub * 8) * 2u;
        auto load_pix_raw = [&](int slot) __attribute__((always_inline)) {
            return S.perm[(size_t)(per_head ? head : 0) * npix + min(slot, npix - 1)];
        };
        auto load_pix = [&](int slot) __attribute__((always_inline)) { return clampi(load_pix_raw(slot), 0, npix - 1); };

        uint32_t src[Cfg::CPT], dst[Cfg::CPT];
#pragma unroll
        for (int c = 0; c < Cfg::CPT; ++c) {
            const int f = (int)threadIdx.x + c * kTileNT;
            const int p = f / CPP, ch = f - p * CPP;
            const int py = p / BW, px = p - py * BW;
            const int gy = clampi(box_y + py, 0, A.H - 1), gx = clampi(box_x + px, 0, A.W - 1);
            const bool in = f < Cfg::NCHUNK;
            src[c] = in ? (uint32_t)(b * A.N + gy * A.W + gx) * row_bytes + (uint32_t)(hgrp * GB + ch * 16) : kDeadOffset;
            dst[c] = in ? (uint32_t)(p * PSTR + ch * 16) : 0xffffffffu;
        }
        int slot = lo + gi;
        __builtin_amdgcn_sched_barrier(0);
        int pix = load_pix_raw(slot), pix_n = load_pix_raw(slot + QPP);     // (used, and bounded, after the staging loads are issued)
        u32x4 kv[2][Cfg::CPT];
#pragma unroll
        for (int c = 0; c < Cfg::CPT; ++c) {
            kv[0][c] = buf_load16(rk, src[c]);
            kv[1][c] = buf_load16(rv, src[c]);
        }
        __builtin_amdgcn_sched_barrier(0);            // (the wait for the pixel indices comes after these loads)
        pix = clampi(pix, 0, npix - 1);
        pix_n = clampi(pix_n, 0, npix - 1);
        uint32_t xyu = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)(pix * A.h + head) * 4u), 0, 0);
        u32x4 qv[VPL], gv[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) {
            qv[u] = buf_load16(rq, (uint32_t)pix * row_bytes + chan_bytes + vec_off[u]);
            gv[u] = buf_load16(rg, (uint32_t)pix * row_bytes + chan_bytes + vec_off[u]);
        }
        const int item_n = min(item_next, item_end - 1);
        const int2 entry_n = S.chunk_item[item_n / nhg];

        __syncthreads();                              // every wave is done with the previous tiles
#pragma unroll
        for (int c = 0; c < Cfg::CPT; ++c)
            if (dst[c] != 0xffffffffu) {
                *(u32x4 *)(smem + dst[c]) = kv[0][c];
                *(u32x4 *)(smem + Cfg::TILE_BYTES + dst[c]) = kv[1][c];
            }
        if (threadIdx.x == 0) s_claim = claim;
        __syncthreads();                              // tiles are in place
        const int item_nn = xcd_start + *(volatile int *)&s_claim;
        __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): see the forward kernel
        bool valid = slot < hi;
        if (__builtin_amdgcn_ballot_w64(valid) != 0) do {
            const int pix_nn = load_pix(slot + 2 * QPP);
            const uint32_t xyu_n = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)(pix_n * A.h + head) * 4u), 0, 0);
            u32x4 qv_n[VPL], gv_n[VPL];
#pragma unroll
            for (int u = 0; u < VPL; ++u) {
                qv_n[u] = buf_load16(rq, (uint32_t)pix_n * row_bytes + chan_bytes + vec_off[u]);
                gv_n[u] = buf_load16(rg, (uint32_t)pix_n * row_bytes + chan_bytes + vec_off[u]);
            }

            const int hq = pix * A.h + head;
            const half2_t xy = as_h2(xyu);
            const float x = (float)xy.x, y = (float)xy.y;
            float x0, y0, w[4];
            corner_weights<T>(x, y, x0, y0, w);
            const int ix = centre_index(x0), iy = centre_index(y0);
            const int cx = ix - R - box_x, cy = iy - R - box_y;
            const bool fits = cx >= 0 && cx + WN <= BW && cy >= 0 && cy + WN <= BH;
            const uint32_t tap0 = (uint32_t)(((fits ? cy : 0) * BW + (fits ? cx : 0)) * PSTR) + lane_lds;

            u32x4 buf[2][G][VPL];
            auto fetch = [&](auto tile_tag, auto s_tag) __attribute__((always_inline)) {
                constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
                constexpr int base = decltype(tile_tag)::value * Cfg::TILE_BYTES;
                uint32_t at[VPL];
#pragma unroll
                for (int u = 0; u < VPL; ++u) {
                    at[u] = tap0 + vec_off[u];
                    asm volatile("" : "+v"(at[u]));   // opaque per stage: keeps the LDS reads in their stage
                }
#pragma unroll
                for (int t = 0; t < G; ++t)
#pragma unroll
                    for (int u = 0; u < VPL; ++u)
                        buf[s & 1][t][u] = *(const u32x4 *)(smem + at[u] + (uint32_t)(base + (j * BW + i0 + t) * PSTR));
            };
            typedef std::integral_constant<int, 0> KT;
            typedef std::integral_constant<int, 1> VT;

            // ---- sweep 1 (K): logits, rounded as the forward rounds them ---------------------------
            half2_t lgp[WN][HW];
            fetch(KT{}, std::integral_constant<int, 0>{});
            static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
                constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
                if constexpr (s + 1 < NSR) fetch(KT{}, std::integral_constant<int, s + 1>{});
#pragma unroll
                for (int t = 0; t < G; ++t) {
                    const int i = i0 + t;
                    float sum = l1_sum<T>(qv[0], buf[s & 1][t][0]);
#pragma unroll
                    for (int u = 1; u < VPL; ++u) sum += l1_sum<T>(qv[u], buf[s & 1][t][u]);   // per vector, then added: the
                                                  // same bits whichever order the lane holds its vectors in
                    sum = group_sum<LPH>(sum);
                    const half_t l16 = (half_t)sum;
                    const half_t s16 = (half_t)((float)l16 * nscale);
                    if (i & 1) lgp[j][i >> 1].y = s16; else lgp[j][i >> 1].x = s16;
                    uint32_t pinned = h2_as_u32(lgp[j][i >> 1]);
                    asm volatile("" : "+v"(pinned));
                    lgp[j][i >> 1] = as_h2(pinned);
                }
                __builtin_amdgcn_sched_barrier(0);
            });

            // ---- softmax state (shared-exponential form) --------------------------------------------
            half2_t mall = lgp[0][0], min2[HW];
#pragma unroll
            for (int i = 0; i < HW; ++i) min2[i] = lgp[1][i];
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    if (j || i) mall = __builtin_elementwise_max(mall, lgp[j][i]);
                    if (j >= 2 && j <= 2 * R) min2[i] = __builtin_elementwise_max(min2[i], lgp[j][i]);
                }
            const float gmax = fmaxf((float)mall.x, (float)mall.y);
            float imax = fmaxf((float)min2[0].y, (float)min2[HW - 1].x);
#pragma unroll
            for (int i = 1; i < HW - 1; ++i) imax = fmaxf(imax, fmaxf((float)min2[i].x, (float)min2[i].y));
            int far = !(gmax - imax < kSharedExpLimit);
            asm volatile("" : "+v"(far));
            float e[WN][WN];
            {
                const float gl = gmax * kLog2e;
#pragma unroll
                for (int j = 0; j < WN; ++j)
#pragma unroll
                    for (int i = 0; i < HW; ++i) {
                        e[j][2 * i] = __builtin_amdgcn_exp2f((float)lgp[j][i].x * kLog2e - gl);
                        e[j][2 * i + 1] = __builtin_amdgcn_exp2f((float)lgp[j][i].y * kLog2e - gl);
                    }
            }
            float ssum[4], inv[4], c[4], c9[3][3];
            subwindow_sum<R>(e, ssum);
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) { inv[bb] = __builtin_amdgcn_rcpf(ssum[bb]); c[bb] = w[bb] * inv[bb]; }
            coef9<R>(c, c9);
            __builtin_amdgcn_sched_barrier(0);

            // ---- sweep 2 (V): g_m = dA_m + <dO, v_m> ---------------------------------------------------
            u32x2 dav[M / 4];                          // dA row of this head-query (M halves), 8 bytes at a time
            const uint32_t da_off = A.d_attn ? (uint32_t)hq * (uint32_t)(M * 2) : kDeadOffset;
#pragma unroll
            for (int k2 = 0; k2 < M / 4; ++k2) {
                const auto r2 = __builtin_amdgcn_raw_buffer_load_b64(rda, (int)(da_off + k2 * 8), 0, 0);
                dav[k2] = __builtin_bit_cast(u32x2, r2);
            }
            {
                uint32_t dep = as_u32(c9[1][1]);       // the V sweep starts after the softmax state
                asm volatile("" : "+v"(dep));
                c9[1][1] = as_f32(dep);
            }
            float g[WN][WN];
            fetch(VT{}, std::integral_constant<int, 0>{});
            static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
                constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
                if constexpr (s + 1 < NSR) fetch(VT{}, std::integral_constant<int, s + 1>{});
#pragma unroll
                for (int t = 0; t < G; ++t) {
                    float sum = 0.f;
#pragma unroll
                    for (int u = 0; u < VPL; ++u) {           // per vector, then added (see the logits)
                        float su = 0.f;
#pragma unroll
                        for (int p2 = 0; p2 < 4; ++p2)
                            su = __builtin_amdgcn_fdot2(as_h2(gv[u][p2]), as_h2(buf[s & 1][t][u][p2]), su, false);
                        sum += su;
                    }
                    sum = group_sum<LPH>(sum);
                    asm volatile("" : "+v"(sum));     // finished here (see the logits above)
                    g[j][i0 + t] = sum;
                }
                __builtin_amdgcn_sched_barrier(0);
            });
#pragma unroll
            for (int m = 0; m < M; ++m) {              // dA (zero when the caller has none: the loads returned 0)
                const half2_t pr = as_h2(dav[m / 4][(m / 2) & 1]);
                g[m / WN][m % WN] += (float)((m & 1) ? pr.y : pr.x);
            }

            // ---- through the softmax: dw_b, dl_m (overwrites g), a_m ---------------------------------
            float dw[4];
            {
                float eg[WN][WN];
#pragma unroll
                for (int j = 0; j < WN; ++j)
#pragma unroll
                    for (int i = 0; i < WN; ++i) eg[j][i] = e[j][i] * g[j][i];
                subwindow_sum<R>(eg, dw);
            }
            float cd[4], cd9[3][3];
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) { dw[bb] *= inv[bb]; cd[bb] = c[bb] * dw[bb]; }
            coef9<R>(cd, cd9);
            const bool mine = valid && fits && !far;
            // (offsets of lanes that store nothing are chosen per store: a dead base plus a tap's offset could wrap into
            // the array)
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < WN; i += 2) {
                    float dl2[2], a2[2];
#pragma unroll
                    for (int d = 0; d < 2; ++d) {
                        const float cc = c9[cls<R>(j)][cls<R>(i + d)];
                        dl2[d] = A.scale * e[j][i + d] * (g[j][i + d] * cc - cd9[cls<R>(j)][cls<R>(i + d)]);
                        a2[d] = (float)(half_t)(e[j][i + d] * cc);                // the stored attention value
                        g[j][i + d] = dl2[d];
                    }
                    // (dl, a) pairs of two taps (neighbours in either layout of the pair array): one 8-byte store
                    static_assert(WN % 2 == 0 && M % 2 == 0, "two taps of a window row are neighbours in both layouts of the pair array");
                    const uint32_t off = (mine && sub == 0) ? pairs.at((uint32_t)pix, (uint32_t)(j * WN + i)) * 4u : kDeadOffset;
                    buf_store8(rws, off, u32x2{PairOf<T>::pack(dl2[0], a2[0]), PairOf<T>::pack(dl2[1], a2[1])});
                }
            {
                float dx, dy;
                offset_grad<T>(x, y, dw, dx, dy);
                const half2_t dm = half2_t{(half_t)dx, (half_t)dy};
                __builtin_amdgcn_raw_buffer_store_b32(h2_as_u32(dm), rdm, (mine && sub == 0) ? (int)((uint32_t)hq * 4u) : (int)kDeadOffset, 0, 0);
            }
            __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(mine ? 0 : 1), rd, (valid && sub == 0) ? hq : (int)kDeadOffset, 0, 0);
            __builtin_amdgcn_sched_barrier(0);

            // ---- sweep 3 (K again): dQ = -sum_m dl_m sgn(q - k_m) -------------------------------------
            float dq[VPL][8];
#pragma unroll
            for (int u = 0; u < VPL; ++u)
#pragma unroll
                for (int el = 0; el < 8; ++el) dq[u][el] = 0.f;
            {
                uint32_t dep = as_u32(g[WN - 1][WN - 1]);
                asm volatile("" : "+v"(dep));
                g[WN - 1][WN - 1] = as_f32(dep);
            }
            fetch(KT{}, std::integral_constant<int, 0>{});
            static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
                constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
                if constexpr (s + 1 < NSR) fetch(KT{}, std::integral_constant<int, s + 1>{});
#pragma unroll
                for (int t = 0; t < G; ++t) {
                    // The difference is a packed half subtraction (exact sign).  sgn(d) per element: the half widened and
                    // multiplied by 2^60 in one mixed-precision instruction (the smallest subnormal difference, 2^-24, lands
                    // above 1), then the median of (x, -1, 1) -- 0, 1.0 or -1.0 -- and a plain fp32 multiply-add.  (In packed
                    // half arithmetic -- two multiplications by 2^15, maximum, minimum -- the sign cost four instructions
                    // that issue at half the rate of these: identical bits, 1 % of the call slower.)
                    const float ndl = -g[j][i0 + t];
#pragma unroll
                    for (int u = 0; u < VPL; ++u)
#pragma unroll
                        for (int p2 = 0; p2 < 4; ++p2) {
                            const half2_t d = as_h2(qv[u][p2]) - as_h2(buf[s & 1][t][u][p2]);
                            const float s0 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)d.x, 0x1p60f, 0.0f), -1.0f, 1.0f);
                            const float s1 = __builtin_amdgcn_fmed3f(__builtin_fmaf((float)d.y, 0x1p60f, 0.0f), -1.0f, 1.0f);
                            dq[u][2 * p2] = __builtin_fmaf(s0, ndl, dq[u][2 * p2]);
                            dq[u][2 * p2 + 1] = __builtin_fmaf(s1, ndl, dq[u][2 * p2 + 1]);
                        }
                }
#pragma unroll
                for (int u = 0; u < VPL; ++u)
                    asm volatile("" : "+v"(dq[u][0]), "+v"(dq[u][1]), "+v"(dq[u][2]), "+v"(dq[u][3]), "+v"(dq[u][4]), "+v"(dq[u][5]), "+v"(dq[u][6]), "+v"(dq[u][7]));
                __builtin_amdgcn_sched_barrier(0);
            });
#pragma unroll
            for (int u = 0; u < VPL; ++u)
                buf_store16(rdq, mine ? (uint32_t)pix * row_bytes + chan_bytes + vec_off[u] : kDeadOffset, vec_pack<T>(dq[u]));

            slot += QPP;
            pix = pix_n; pix_n = pix_nn; xyu = xyu_n;
#pragma unroll
            for (int u = 0; u < VPL; ++u) { qv[u] = qv_n[u]; gv[u] = gv_n[u]; }
            valid = slot < hi;
        } while (__builtin_amdgcn_ballot_w64(valid) != 0);
        entry = entry_n;
        item = item_next;
        item_next = item_nn;
    }   // items
}

}  // namespace ma

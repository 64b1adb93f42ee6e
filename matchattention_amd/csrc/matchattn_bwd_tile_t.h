// Pass A of the gather-mode backward with every tap read from LDS, for fp32 and bf16 storage (gfx950).
//
// The item machinery is the forward's (matchattn_fwd_tile_t.h: buckets of queries per K/V tile, work list, K and V
// tile plus halo staged in LDS, passes over the bucket); the arithmetic of a pass is the direct kernel's
// (bwd_tiled_kernel in gather mode, matchattn_bwd.h): logits and softmax recomputed, g_m = dA_m + <dO, v_m>,
// through the softmax, d max_offset, dQ, and the (dl, a) pairs for pass B.  One 16-byte vector per lane.
// A window that does not fit the staged rectangle is flagged and finished by the direct kernel.
#pragma once
#include "matchattn_bwd.h"
#include "matchattn_fwd_tile_t.h"

namespace ma {

template <typename T, int CH, int R, int TW, int TH, int NT = kTileNT>
__global__ __launch_bounds__(NT, MA_TILE_WAVES) void bwd_tile_kernel(BwdArgs A, TileSort S) {
    typedef TileCfgT<T, CH, R, TW, TH, 1, NT> Cfg;
    typedef Traits<T> Tr;
    constexpr int ES = Cfg::ES, EPV = Cfg::EPV, WN = Cfg::WN, M = Cfg::M, BW = Cfg::BW, BH = Cfg::BH;
    constexpr int GB = Cfg::GB, HPG = Cfg::HPG, CPP = Cfg::CPP, PSTR = Cfg::PSTR, LPH = Cfg::LPH, QPP = Cfg::QPP;
    constexpr int NDA = M * ES / 8;                    // 8-byte pieces of a dA row

    __shared__ __attribute__((aligned(16))) char smem[2 * Cfg::TILE_BYTES];   // K tile, then V tile

    const int nhg = A.h / HPG;
    const int npix = S.L;
    const uint32_t row_bytes = (uint32_t)A.C * (uint32_t)ES;
    const uint32_t total_bytes = (uint32_t)npix * row_bytes;
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t rg = make_rsrc(A.d_out, total_bytes);
    const __amdgpu_buffer_rsrc_t rdq = make_rsrc(A.dq, total_bytes);
    const __amdgpu_buffer_rsrc_t rm = make_rsrc(A.mo, (uint32_t)A.nhq * (uint32_t)(2 * ES));
    const __amdgpu_buffer_rsrc_t rdm = make_rsrc(A.dmo, (uint32_t)A.nhq * (uint32_t)(2 * ES));
    const __amdgpu_buffer_rsrc_t rda = make_rsrc(A.d_attn, A.d_attn ? (uint32_t)A.nhq * (uint32_t)(M * ES) : 0u);
    const __amdgpu_buffer_rsrc_t rws = make_rsrc(A.dl_ws, (uint32_t)A.nhq * (uint32_t)(M * PairOf<T>::kBytes));
    const bool pairs_per_head = A.per_head[0] != 0;    // layout of the pair array (PairLayout): the inverse index's flag, not the tile buckets'
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(S.defer, (uint32_t)A.nhq);
    const int sub = threadIdx.x % LPH;
    const int grp = threadIdx.x / LPH;
    const int hslot = grp % HPG, gi = grp / HPG;
    const uint32_t lane_lds = (uint32_t)(hslot * Cfg::HB + sub * 16);

    const int nchunks = min(max(S.chunk_start[S.nbins], 0), S.chunk_cap);
    const int xcd = blockIdx.x & 7;
    // XCD x takes the x-th share of the work list (consecutive chunks, shares of equal cost: tile_chunks_kernel), the
    // head groups of a chunk being neighbours in the item order; bounds read from scratch memory are clamped
    const int share_lo = clampi(S.xcd_bounds[xcd], 0, nchunks), share_hi = clampi(S.xcd_bounds[xcd + 1], share_lo, nchunks);
    const int xcd_start = share_lo * nhg, item_end = share_hi * nhg;
    const bool per_head = *S.per_head != 0;
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
        const uint32_t chan_bytes = (uint32_t)(head * Cfg::HB + sub * 16);
        auto load_pix_raw = [&](int slot) __attribute__((always_inline)) {
            return S.perm[(size_t)(per_head ? head : 0) * npix + min(slot, npix - 1)];
        };
        auto load_pix = [&](int slot) __attribute__((always_inline)) { return clampi(load_pix_raw(slot), 0, npix - 1); };

        // staging, in the forward kernel's order: addresses, the two index loads, the staging loads, the first
        // pass's rows
        uint32_t src[Cfg::CPT], dst[Cfg::CPT];
#pragma unroll
        for (int c = 0; c < Cfg::CPT; ++c) {
            const int f = (int)threadIdx.x + c * NT;
            const int p = f / CPP, ch = f - p * CPP;
            const int py = p / BW, px = p - py * BW;
            const int gy = clampi(box_y + py, 0, A.H - 1), gx = clampi(box_x + px, 0, A.W - 1);
            const bool in = f < Cfg::NCHUNK;
            src[c] = in ? (uint32_t)(b * A.N + gy * A.W + gx) * row_bytes + (uint32_t)(hgrp * GB + ch * 16) : kDeadOffset;
            dst[c] = in ? (uint32_t)(p * PSTR + ch * 16) : 0xffffffffu;
        }
        int slot = lo + gi;
        __builtin_amdgcn_sched_barrier(0);
        int pix = load_pix_raw(slot), pix_n = load_pix_raw(slot + QPP);
        u32x4 kvs[2][Cfg::CPT];
#pragma unroll
        for (int c = 0; c < Cfg::CPT; ++c) {
            kvs[0][c] = buf_load16(rk, src[c]);
            kvs[1][c] = buf_load16(rv, src[c]);
        }
        __builtin_amdgcn_sched_barrier(0);
        pix = clampi(pix, 0, npix - 1);
        pix_n = clampi(pix_n, 0, npix - 1);
        RawPosition<T> pos = load_position<T>(rm, pix * A.h + head);
        u32x4 qv = buf_load16(rq, (uint32_t)pix * row_bytes + chan_bytes);
        u32x4 gv = buf_load16(rg, (uint32_t)pix * row_bytes + chan_bytes);
        const int item_n = min(item_next, item_end - 1);
        const int2 entry_n = S.chunk_item[item_n / nhg];

        __syncthreads();                              // every wave is done with the previous tiles
#pragma unroll
        for (int c = 0; c < Cfg::CPT; ++c)
            if (dst[c] != 0xffffffffu) {
                *(u32x4 *)(smem + dst[c]) = kvs[0][c];
                *(u32x4 *)(smem + Cfg::TILE_BYTES + dst[c]) = kvs[1][c];
            }
        if (threadIdx.x == 0) s_claim = claim;
        __syncthreads();                              // tiles are in place
        const int item_nn = xcd_start + *(volatile int *)&s_claim;
        __builtin_amdgcn_s_waitcnt(0x0F70);           // vmcnt(0): see the fp16 forward kernel
        bool valid = slot < hi;
        if (__builtin_amdgcn_ballot_w64(valid) != 0) do {
            const int pix_nn = load_pix(slot + 2 * QPP);
            const RawPosition<T> pos_n = load_position<T>(rm, pix_n * A.h + head);
            const u32x4 qv_n = buf_load16(rq, (uint32_t)pix_n * row_bytes + chan_bytes);
            const u32x4 gv_n = buf_load16(rg, (uint32_t)pix_n * row_bytes + chan_bytes);
            const int hq = pix * A.h + head;
            // dA row of this head-query, 8 bytes at a time (no dA: every load is out of range and returns zero)
            u32x2 dav[NDA];
            const uint32_t da_off = A.d_attn ? (uint32_t)hq * (uint32_t)(M * ES) : kDeadOffset;
#pragma unroll
            for (int k2 = 0; k2 < NDA; ++k2)
                dav[k2] = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rda, (int)(da_off + k2 * 8), 0, 0));

            float x, y, x0, y0, w[4];
            position_xy<T>(pos, x, y);
            corner_weights<T>(x, y, x0, y0, w);
            const int ix = centre_index(x0), iy = centre_index(y0);
            const int cx = ix - R - box_x, cy = iy - R - box_y;
            const bool fits = cx >= 0 && cx + WN <= BW && cy >= 0 && cy + WN <= BH;
            const uint32_t tap0 = (uint32_t)(((fits ? cy : 0) * BW + (fits ? cx : 0)) * PSTR) + lane_lds;
            // one window row of a tile at a time; the address is an opaque copy made where the row is wanted, so
            // that the reads stay there (nothing writes the tiles inside the loop)
            auto fetch_row = [&](int tile, int j, u32x4 (&rowv)[WN]) __attribute__((always_inline)) {
                uint32_t at = tap0 + (uint32_t)(tile * Cfg::TILE_BYTES + j * BW * PSTR);
                asm volatile("" : "+v"(at));
#pragma unroll
                for (int i = 0; i < WN; ++i) rowv[i] = *(const u32x4 *)(smem + at + (uint32_t)(i * PSTR));
            };

            // ---- forward recompute: logits and softmax state ------------------------------------------
            float lg[WN][WN];
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                u32x4 kv[WN];
                fetch_row(0, j, kv);
#pragma unroll
                for (int i = 0; i < WN; ++i) {
                    const float s = group_sum<LPH>(l1_accum<T>(qv, kv[i], 0.f));
                    lg[j][i] = Tr::round(-Tr::round(s) * A.scale);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            SoftmaxState<R> st;
            const bool shared = softmax_prepare<R>(lg, st);
            if (shared) softmax_shared_exp<R>(lg, w, st); else softmax_exact<R>(lg, w, st, false);
            float c9[3][3];
            coef9<R>(st.c, c9);

            float go[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) go[e] = vec_elem<T>(gv, e);

            // ---- g_m = dA_m + <dO, v_m> ---------------------------------------------------------------
            float g[WN][WN];
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                u32x4 vv[WN];
                fetch_row(1, j, vv);
#pragma unroll
                for (int i = 0; i < WN; ++i) {
                    float s = 0.f;
                    if constexpr (std::is_same<T, bf16_t>::value) {     // <dO, v> on the packed words: no unpacking
#pragma unroll
                        for (int p = 0; p < 4; ++p) {
                            const uint32_t gw = gv[p], vw = vv[i][p];      // (copies: a bit cast applied to a vector's element reads element 0)
                            s = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, gw), __builtin_bit_cast(bf16x2_t, vw), s, false);
                        }
                    } else {
#pragma unroll
                        for (int e = 0; e < EPV; ++e) s += go[e] * vec_elem<T>(vv[i], e);
                    }
                    s = group_sum<LPH>(s);
                    const int m = j * WN + i;
                    const u32x4 piece = {dav[m * ES / 8][0], dav[m * ES / 8][1], 0, 0};
                    g[j][i] = s + vec_elem<T>(piece, m % (8 / ES));
                }
                __builtin_amdgcn_sched_barrier(0);
            }

            // ---- through the softmax: dw_b and dl_m (dl overwrites g); d max_offset and the pairs -----------
            float dw[4];
            bilinear_softmax_bwd<R>(shared, lg, st, A.scale, g, dw);
            const bool mine = valid && fits;
            {
                float dx, dy;
                offset_grad<T>(x, y, dw, dx, dy);
                const bool wr = mine && sub == 0;
                if constexpr (ES == 4) {
                    buf_store8(rdm, wr ? (uint32_t)hq * 8u : kDeadOffset, u32x2{as_u32(dx), as_u32(dy)});
                } else {
                    T t2[2] = {Tr::from_f(dx), Tr::from_f(dy)};
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, t2), rdm, wr ? (int)((uint32_t)hq * 4u) : (int)kDeadOffset, 0, 0);
                }
                // (offsets of lanes that store nothing are chosen per store: a dead base plus a tap's offset could wrap
                // into the array)
#pragma unroll
                for (int j = 0; j < WN; ++j)
#pragma unroll
                    for (int i = 0; i < WN; ++i)
                    {
                        const auto pw = PairOf<T>::pack(g[j][i], Tr::round(attn_value<R>(shared, lg, st, c9, j, i)));
                        const uint32_t p_off = wr ? pairs.at((uint32_t)pix, (uint32_t)(j * WN + i)) *
                                                        (uint32_t)PairOf<T>::kBytes : kDeadOffset;
                        if constexpr (PairOf<T>::kBytes == 8) buf_store8(rws, p_off, pw);
                        else __builtin_amdgcn_raw_buffer_store_b32(pw, rws, (int)p_off, 0, 0);
                    }
            }

            // ---- dQ = -sum_m dl_m sgn(q - k_m) -----------------------------------------------------------
            float qf[EPV], dq[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) { qf[e] = vec_elem<T>(qv, e); dq[e] = 0.f; }
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                u32x4 kv[WN];
                fetch_row(0, j, kv);
#pragma unroll
                for (int i = 0; i < WN; ++i) {
                    const float dl = g[j][i];
#pragma unroll
                    for (int e = 0; e < EPV; ++e) dq[e] -= dl * sign_f(qf[e] - vec_elem<T>(kv[i], e));
                }
#pragma unroll
                for (int e = 0; e < EPV; ++e) asm volatile("" : "+v"(dq[e]));
                __builtin_amdgcn_sched_barrier(0);
            }
            buf_store16(rdq, mine ? (uint32_t)pix * row_bytes + chan_bytes : kDeadOffset, vec_pack<T>(dq));
            // what this tile cannot serve is flagged for the direct kernel (a flag per head-query, written for all)
            __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(mine ? 0 : 1), rd, (valid && sub == 0) ? hq : (int)kDeadOffset, 0, 0);

            slot += QPP;
            pix = pix_n; pix_n = pix_nn; pos = pos_n; qv = qv_n; gv = gv_n;
            valid = slot < hi;
        } while (__builtin_amdgcn_ballot_w64(valid) != 0);
        entry = entry_n;
        item = item_next;
        item_next = item_nn;
    }   // items
}

}  // namespace ma

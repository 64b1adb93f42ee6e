// Forward kernel that gathers every tap from LDS, for fp32 and bf16 storage (gfx950).
//
// The item machinery is the one of the fp16 kernel in matchattn_fwd_tile.h (buckets of queries per K/V tile,
// work list, a persistent grid, K and V tile plus halo staged in LDS, passes over the bucket); the arithmetic of
// a pass is the one of the direct kernel in matchattn_fwd.h (fp32 logits rounded as the storage type rounds
// them, the exact per-sub-window softmax), so only a window that does not fit the staged rectangle is left to
// the generic kernel.
#pragma once
#include "matchattn_fwd_tile.h"
#include "matchattn_softmax.h"

namespace ma {

// NT: threads per workgroup.  256 with two workgroups per CU (a head group of 128 bytes per pixel); heads of 256 bytes
// (64 fp32 channels) take 512 threads and a CU's whole LDS: still eight wavefronts per CU, in one workgroup.
template <typename T, int CH, int R, int TW_, int TH_, int VPL_, int NT_ = kTileNT>
struct TileCfgT {
    static constexpr int NT = NT_;
    static constexpr int ES = (int)sizeof(T), EPV = 16 / ES;
    static constexpr int VPL = VPL_, TW = TW_, TH = TH_;
    static constexpr int WN = 2 * R + 2, M = WN * WN;
    static constexpr int BW = TW + 2 * R + 1, BH = TH + 2 * R + 1;   // staged rectangle
    static constexpr int HB = CH * ES;                               // bytes of one head per pixel
    static constexpr int GB = HB >= 128 ? HB : 128;                  // bytes of one head group per pixel
    static constexpr int HPG = GB / HB, CPP = GB / 16;               // heads per group, 16-byte pieces per pixel
    static constexpr int PSTR = GB;
    static constexpr int TILE_BYTES = BW * BH * PSTR;
    static constexpr int LPH = HB / 16 / VPL;                        // lanes per head-query (VPL x 16 bytes each)
    static_assert(HB % (16 * VPL) == 0, "head size");
    static constexpr int QPP = NT / LPH / HPG;                       // queries per head and pass
    static constexpr int NCHUNK = BW * BH * CPP;
    static constexpr int CPT = (NCHUNK + NT - 1) / NT;
    static_assert(LPH == 1 || LPH == 2 || LPH == 4 || LPH == 8 || LPH == 16, "head size");
    static constexpr int WG_PER_CU = 2 * kTileNT / NT;               // eight wavefronts per CU
    static_assert(WG_PER_CU >= 1 && 2 * TILE_BYTES * WG_PER_CU + 1024 <= 160 * 1024, "K and V tiles of a CU's workgroups must fit its LDS");
    static_assert(kTileCap % QPP == 0, "a chunk is a whole number of passes");
};

// the sampling position of head-query hq, two elements of T: loaded as raw words, converted where it is used (a
// conversion next to the load would wait for it)
template <typename T> struct RawPosition { uint32_t w[sizeof(T) == 4 ? 2 : 1]; };
template <typename T>
__device__ __forceinline__ RawPosition<T> load_position(const __amdgpu_buffer_rsrc_t &rm, int hq) {
    RawPosition<T> p;
    if constexpr (sizeof(T) == 4) {
        p.w[0] = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)hq * 8u), 0, 0);
        p.w[1] = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)hq * 8u + 4u), 0, 0);
    } else {
        p.w[0] = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)hq * 4u), 0, 0);
    }
    return p;
}
template <typename T>
__device__ __forceinline__ void position_xy(const RawPosition<T> &p, float &x, float &y) {
    if constexpr (sizeof(T) == 4) {
        x = as_f32(p.w[0]);
        y = as_f32(p.w[1]);
    } else {
        const u32x4 v = {p.w[0], 0, 0, 0};
        x = vec_elem<T>(v, 0);
        y = vec_elem<T>(v, 1);
    }
}

template <typename T, int CH, int R, int TW, int TH, int VPL, int NT = kTileNT>
__global__ __launch_bounds__(NT, MA_TILE_WAVES) void fwd_tile_kernel(FwdArgs A, TileSort S) {
    typedef TileCfgT<T, CH, R, TW, TH, VPL, NT> Cfg;
    typedef StageCfg<R, VPL> St;
    typedef Traits<T> Tr;
    constexpr int ES = Cfg::ES, EPV = Cfg::EPV, WN = Cfg::WN, M = Cfg::M, BW = Cfg::BW, BH = Cfg::BH;
    constexpr int GB = Cfg::GB, HPG = Cfg::HPG, CPP = Cfg::CPP, PSTR = Cfg::PSTR, LPH = Cfg::LPH, QPP = Cfg::QPP;
    // taps per stage: even for bf16, whose aggregation takes the taps two at a time
    constexpr bool kBf16 = std::is_same<T, bf16_t>::value;
    constexpr int G = (kBf16 && St::G % 2) ? 2 : St::G, SPR = WN / G, NSR = WN * SPR, LAST0 = (WN - 1) * SPR;
    static_assert(WN % G == 0, "stage size must divide the window row");

    __shared__ __attribute__((aligned(16))) char smem[2 * Cfg::TILE_BYTES];   // K tile, then V tile

    const int nhg = A.h / HPG;
    const int npix = S.L;
    const uint32_t row_bytes = (uint32_t)A.C * (uint32_t)ES;
    const uint32_t total_bytes = (uint32_t)npix * row_bytes;
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(A.out, out_span_bytes(A, ES));
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A.attn, attn_span_bytes(A, (uint32_t)(A.h * M), ES));
    const __amdgpu_buffer_rsrc_t rgate = make_rsrc(A.gate, A.gate ? total_bytes : 0u);   // (no gate: every load is out of range)
    const __amdgpu_buffer_rsrc_t rm = make_rsrc(A.mo, (uint32_t)A.nhq * (uint32_t)(2 * ES));
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(S.defer, (uint32_t)A.nhq);
    const int sub = threadIdx.x % LPH;
    const int grp = threadIdx.x / LPH;
    const int hslot = grp % HPG, gi = grp / HPG;
    // lane `sub` owns the 16-byte vectors sub, sub + LPH, ... of its head; with two vectors per lane odd lane
    // groups take theirs in the opposite order (LDS bank groups, as in the fp16 kernel)
    const int par = VPL == 2 ? (gi & 1) : 0;
    const uint32_t lane_lds = (uint32_t)(hslot * Cfg::HB + sub * 16);
    uint32_t vec_off[VPL];
#pragma unroll
    for (int u = 0; u < VPL; ++u) vec_off[u] = (uint32_t)((u ^ par) * LPH * 16);

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
    int lo, hi;
    bucket_bounds(S, per_head ? head : 0, bin, lo, hi);
    const int row = bin / S.bins_per_row, tx = bin - row * S.bins_per_row;
    const int b = min(row / S.rows_per_img, npix / A.N - 1), ty = row - (row / S.rows_per_img) * S.rows_per_img;
    const int box_x = tx * TW - R, box_y = ty * TH - R;
    lo = min(lo + part * kTileCap, hi);
    hi = min(hi, lo + kTileCap);
    const uint32_t chan_bytes = (uint32_t)(head * Cfg::HB + sub * 16);     // vector u adds u * LPH * 16 bytes

    auto load_pix_raw = [&](int slot) __attribute__((always_inline)) {
        return S.perm[(size_t)(per_head ? head : 0) * npix + min(slot, npix - 1)];
    };
    auto load_pix = [&](int slot) __attribute__((always_inline)) { return clampi(load_pix_raw(slot), 0, npix - 1); };

    // ---- stage the K and V rectangles (replicate-clamped at the image border); the order of the loads is the
    // fp16 kernel's: addresses, the two index loads, the staging loads, then the first pass's rows
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
    u32x4 kv[2][Cfg::CPT];
#pragma unroll
    for (int c = 0; c < Cfg::CPT; ++c) {
        kv[0][c] = buf_load16(rk, src[c]);
        kv[1][c] = buf_load16(rv, src[c]);
    }
    __builtin_amdgcn_sched_barrier(0);
    pix = clampi(pix, 0, npix - 1);
    pix_n = clampi(pix_n, 0, npix - 1);
    RawPosition<T> pos = load_position<T>(rm, pix * A.h + head);
    u32x4 qv[VPL];
#pragma unroll
    for (int u = 0; u < VPL; ++u) qv[u] = buf_load16(rq, (uint32_t)pix * row_bytes + chan_bytes + vec_off[u]);
    const int item_n = min(item_next, item_end - 1);
    const int2 entry_n = S.chunk_item[item_n / nhg];

    __syncthreads();                                  // every wave is done with the previous tiles
#pragma unroll
    for (int c = 0; c < Cfg::CPT; ++c)
        if (dst[c] != 0xffffffffu) {
            *(u32x4 *)(smem + dst[c]) = kv[0][c];
            *(u32x4 *)(smem + Cfg::TILE_BYTES + dst[c]) = kv[1][c];
        }
    if (threadIdx.x == 0) s_claim = claim;
    __syncthreads();                                  // tiles are in place
    const int item_nn = xcd_start + *(volatile int *)&s_claim;

    __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): see the fp16 kernel
    bool valid = slot < hi;
    if (__builtin_amdgcn_ballot_w64(valid) != 0) do {
        const int pix_nn = load_pix(slot + 2 * QPP);
        const RawPosition<T> pos_n = load_position<T>(rm, pix_n * A.h + head);
        u32x4 qv_n[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) qv_n[u] = buf_load16(rq, (uint32_t)pix_n * row_bytes + chan_bytes + vec_off[u]);
        u32x4 gatev[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) gatev[u] = buf_load16(rgate, (uint32_t)pix * row_bytes + chan_bytes + vec_off[u]);

        const int hq = pix * A.h + head;
        float x, y, x0, y0, w[4];
        position_xy<T>(pos, x, y);
        corner_weights<T>(x, y, x0, y0, w);
        const int ix = centre_index(x0), iy = centre_index(y0);
        const int cx = ix - R - box_x, cy = iy - R - box_y;
        const bool fits = cx >= 0 && cx + WN <= BW && cy >= 0 && cy + WN <= BH;
        const bool drop_last = A.row_skip && __builtin_amdgcn_ballot_w64(y != y0) == 0;
        const uint32_t tap0 = (uint32_t)(((fits ? cy : 0) * BW + (fits ? cx : 0)) * PSTR) + lane_lds;

        u32x4 buf[2][G][VPL];
        auto fetch = [&](auto tile_tag, auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            constexpr int base = decltype(tile_tag)::value * Cfg::TILE_BYTES;
            uint32_t at[VPL];
#pragma unroll
            for (int u = 0; u < VPL; ++u) {
                at[u] = tap0 + vec_off[u];
                asm volatile("" : "+v"(at[u]));       // (each stage's reads stay where the stage starts)
            }
#pragma unroll
            for (int t = 0; t < G; ++t)
#pragma unroll
                for (int u = 0; u < VPL; ++u)
                    buf[s & 1][t][u] = *(const u32x4 *)(smem + at[u] + (uint32_t)(base + (j * BW + i0 + t) * PSTR));
        };
        typedef std::integral_constant<int, 0> KT;
        typedef std::integral_constant<int, 1> VT;

        // ---- logits ----------------------------------------------------------------------------
        float lg[WN][WN];
#pragma unroll
        for (int i = 0; i < WN; ++i) lg[WN - 1][i] = -__builtin_inff();   // stays if the row is left out
        fetch(KT{}, std::integral_constant<int, 0>{});
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) {
                if (s + 1 < LAST0 || !drop_last) fetch(KT{}, std::integral_constant<int, s + 1>{});
            }
            if (s >= LAST0 && drop_last) return;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                float sum = l1_sum<T>(qv[0], buf[s & 1][t][0]);
#pragma unroll
                for (int u = 1; u < VPL; ++u) sum += l1_sum<T>(qv[u], buf[s & 1][t][u]);   // per vector, then added: the
                                                  // same bits whichever order the lane holds its vectors in
                sum = group_sum<LPH>(sum);
                lg[j][i0 + t] = Tr::round(-Tr::round(sum) * A.scale);     // rounding points of the definition
                asm volatile("" : "+v"(lg[j][i0 + t]));                   // (the finished logit is pinned here)
            }
            __builtin_amdgcn_sched_barrier(0);
        });
        // a lane with integer y gives the last row zero weight; dropping it per lane keeps each result
        // independent of which queries share the wavefront
        if (A.row_skip && y == y0) {
#pragma unroll
            for (int i = 0; i < WN; ++i) lg[WN - 1][i] = -__builtin_inff();
        }

        // ---- window softmax (in place: lg becomes the attention weights) ---------------------------
        SoftmaxState<R> st;
        bilinear_softmax_fwd<R>(lg, w, st);
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int i = 0; i < WN; ++i) lg[j][i] = Tr::round(lg[j][i]);   // attn is stored, and reused, in T
        __builtin_amdgcn_sched_barrier(0);
        {
            uint32_t last = as_u32(lg[WN - 2][WN - 1]);
            asm volatile("" : "+v"(last));            // (the first V stage waits for the softmax)
            lg[WN - 2][WN - 1] = as_f32(last);
        }
        fetch(VT{}, std::integral_constant<int, 0>{});

        // ---- aggregation -----------------------------------------------------------------------
        float acc[VPL][EPV];
#pragma unroll
        for (int u = 0; u < VPL; ++u)
#pragma unroll
            for (int e = 0; e < EPV; ++e) acc[u][e] = 0.f;
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) {
                if (s + 1 < LAST0 || !drop_last) fetch(VT{}, std::integral_constant<int, s + 1>{});
            }
            if (s >= LAST0 && drop_last) return;
            if constexpr (kBf16) {
                // two taps at a time: the weights (already bf16 values) packed as a pair, the two taps' values of a
                // channel gathered into one word by a byte permute, one bf16 dot product per channel and tap pair
                // -- no element is unpacked
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
#pragma unroll
            for (int u = 0; u < VPL; ++u)
#pragma unroll
                for (int e = 0; e < EPV; ++e) asm volatile("" : "+v"(acc[u][e]));
            __builtin_amdgcn_sched_barrier(0);
        });

        // ---- stores; a window the tile cannot serve is flagged for the generic kernel -------------------
        const bool mine = valid && fits;
        __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(mine ? 0 : 1), rd, (valid && sub == 0) ? hq : (int)kDeadOffset, 0, 0);
        u32x4 ov[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) ov[u] = vec_pack<T>(acc[u]);
        if (A.gate) {
#pragma unroll
            for (int u = 0; u < VPL; ++u) ov[u] = vec_mul<T>(ov[u], gatev[u]);
        }
#pragma unroll
        for (int u = 0; u < VPL; ++u)
            buf_store16(ro, mine ? (uint32_t)pix * A.out_row_bytes + chan_bytes + vec_off[u] : kDeadOffset, ov[u]);
        const uint32_t a_off = (mine && sub == 0) ? (uint32_t)pix * A.attn_row_bytes + (uint32_t)head * (uint32_t)(M * ES) : kDeadOffset;
        constexpr int PER8 = 8 / ES;                  // elements per 8-byte store
        const float *af = &lg[0][0];
#pragma unroll
        for (int m = 0; m < M; m += PER8) {
            u32x2 pk;
            if constexpr (ES == 4) {
                pk = u32x2{as_u32(af[m]), as_u32(af[m + 1])};
            } else {
                T t4[4] = {Tr::from_f(af[m]), Tr::from_f(af[m + 1]), Tr::from_f(af[m + 2]), Tr::from_f(af[m + 3])};
                pk = __builtin_bit_cast(u32x2, t4);
            }
            buf_store8(ra, a_off + m * ES, pk);
        }

        slot += QPP;
        pix = pix_n; pix_n = pix_nn; pos = pos_n;
#pragma unroll
        for (int u = 0; u < VPL; ++u) qv[u] = qv_n[u];
        valid = slot < hi;
    } while (__builtin_amdgcn_ballot_w64(valid) != 0);
    entry = entry_n;
    item = item_next;
    item_next = item_nn;
    }   // items
}

}  // namespace ma

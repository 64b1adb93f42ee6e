// fp16 forward kernel that gathers every tap from LDS (gfx950).
//
// The queries are first bucketed by the K/V tile their sampling centre falls in (a counting
// sort on tiles of TW x TH key pixels, matchattn_sort.h).  A workgroup then owns one tile and
// one group of heads: it copies the tile plus the halo a window can reach -- (TW + 2R + 1) x
// (TH + 2R + 1) key pixels of that head group, K and V -- from global memory to LDS once, and
// works through the queries of its bucket, 256 / LPH at a time, reading all (2R+2)^2 taps of
// both phases from LDS.  Each K/V byte then crosses L2 -> CU about twice per call instead of
// once per tap, whatever the offset field looks like.
//
// The halo is staged with replicate-clamped coordinates, so a window that leaves the image
// reads the border pixels as the operator defines.  Queries the tile cannot serve are flagged
// and computed afterwards by the generic kernel: windows whose centre lies more than
// a halo outside the image (possible only without the input-domain clamp) and windows whose
// sub-windows need the exact per-sub-window softmax.
#pragma once
#include "matchattn_fwd_h16.h"

namespace ma {

// Tile of key pixels one workgroup serves.
#ifndef MA_TILE_W
#define MA_TILE_W 16
#endif
#ifndef MA_TILE_H
#define MA_TILE_H 8
#endif
constexpr int kTileW = MA_TILE_W, kTileH = MA_TILE_H;

// Threads per workgroup and the waves per SIMD the register allocation aims for: two workgroups
// fit a CU's LDS: 8 waves per CU, 2 per SIMD.
#ifndef MA_TILE_NT
#define MA_TILE_NT 256
#endif
#ifndef MA_TILE_WAVES
#define MA_TILE_WAVES 2
#endif
constexpr int kTileNT = MA_TILE_NT;

template <int CH, int R, int TW_, int TH_, int VPL_ = 1>
struct TileCfg {
    static constexpr int VPL = VPL_;                                 // 16-byte vectors of the head per lane
    static constexpr int TW = TW_, TH = TH_;
    static constexpr int WN = 2 * R + 2, M = WN * WN;
    static constexpr int BW = TW + 2 * R + 1, BH = TH + 2 * R + 1;   // staged rectangle
    static constexpr int GB = LdsGroup<CH>::GB, HPG = LdsGroup<CH>::HPG, CPP = LdsGroup<CH>::CPP;
    static constexpr int PSTR = GB;                                  // LDS bytes from one pixel to the next
    static constexpr int TILE_BYTES = BW * BH * PSTR;
    static constexpr int LPH = CH / 8 / VPL;                         // lanes per head-query (VPL x 16 bytes each)
    static_assert(CH % (8 * VPL) == 0, "head size");
    static constexpr int QPP = kTileNT / LPH / HPG;                     // queries per head and pass
    static constexpr int NCHUNK = BW * BH * CPP;                     // 16-byte pieces of one tile
    static constexpr int CPT = (NCHUNK + kTileNT - 1) / kTileNT;                // pieces per thread
    static_assert(LPH == 1 || LPH == 2 || LPH == 4 || LPH == 8 || LPH == 16, "head size");
    static_assert(2 * TILE_BYTES <= 160 * 1024, "K and V tiles must fit LDS");
};


// Queries per head one work item takes from a bucket: border tiles collect the clamped centres of a whole
// margin of the image and hold many times the average, so buckets are cut into chunks of this size.
#ifndef MA_TILE_CAP
#define MA_TILE_CAP 192
#endif
constexpr int kTileCap = MA_TILE_CAP;
#ifndef MA_TILE_GRID_MULT
#define MA_TILE_GRID_MULT 2
#endif
constexpr int kTileGridMult = MA_TILE_GRID_MULT;
// 1: the bf16 forward subtracts q - k on the matrix unit (fwd_h16_tile_kernel, K phase)
#ifndef MA_TILE_BF16_MFMA_SUB
#define MA_TILE_BF16_MFMA_SUB 1
#endif
// 1: the fp16 forward with 32 channels per head aggregates on the matrix unit (fwd_h16_tile_kernel, V phase)
#ifndef MA_TILE_MFMA_AGG
#define MA_TILE_MFMA_AGG 1
#endif

// [lo, hi) of bucket `bin` (tile row `row` over all images, tile column `tx`) in the bucket order of head `src`,
// clamped so that values read from scratch memory never become addresses unchecked
__device__ __forceinline__ void bucket_bounds_at(const TileSort &S, int src, int bin, int row, int tx, int &lo, int &hi) {
    // four independent loads (both candidates for the end are fetched, then one is chosen): one latency
    const int row_start = S.rowtot[src * S.nrows + row];
    const int next_row = S.rowtot[src * S.nrows + min(row + 1, S.nrows - 1)];
    const int start = S.count[(src * S.nbins + bin) * S.sub];
    const int next = S.count[(src * S.nbins + min(bin + 1, S.nbins - 1)) * S.sub];
    lo = row_start + start;
    hi = tx + 1 < S.bins_per_row ? row_start + next : (row + 1 < S.nrows ? next_row : S.L);
    lo = clampi(lo, 0, S.L);
    hi = clampi(hi, lo, S.L);
}
__device__ __forceinline__ void bucket_bounds(const TileSort &S, int src, int bin, int &lo, int &hi) {
    const int row = bin / S.bins_per_row;
    bucket_bounds_at(S, src, bin, row, bin - row * S.bins_per_row, lo, hi);
}

// Order in which the work list visits the tiles of an image: strips of kTileStrip tile columns, each walked row by
// row from the top.  The workgroups of an XCD take consecutive items, so the tiles in flight form a block about as
// tall as it is wide and the K/V rows a tile shares with the tile below it are still in that XCD's L2 when the
// tile below is staged (in row-major order a whole tile row -- more than the L2 holds, with the query, output
// and attention streams of its items -- passes in between, and the vertical halo is fetched from memory again).
// TileWalk stands at one position of that order and steps to the next without a division (the one workgroup that
// builds the work list is bound by its integer arithmetic: the position -> tile formula costs five divisions).
#ifndef MA_TILE_STRIP
#define MA_TILE_STRIP 8
#endif
constexpr int kTileStrip = MA_TILE_STRIP;
struct TileWalk {
    int img, strip, r, c, w;      // image, strip, tile row within the image, column within the strip, the strip's width
    int nfull, last_w, rows, bpr;
    __device__ __forceinline__ TileWalk(const TileSort &S, int k) {
        rows = S.rows_per_img; bpr = S.bins_per_row;
        const bool strips = kTileStrip > 0 && bpr > kTileStrip;
        nfull = strips ? bpr / kTileStrip : 0;                 // (without strips: one strip as wide as the image)
        last_w = bpr - nfull * kTileStrip;
        const int per_img = rows * bpr;
        img = k / per_img;
        const int kk = k - img * per_img;
        strip = strips ? min(kk / (rows * kTileStrip), nfull) : 0;
        w = strip < nfull ? kTileStrip : last_w;
        const int within = kk - strip * rows * kTileStrip;
        r = within / max(w, 1);
        c = within - r * w;
    }
    __device__ __forceinline__ int row() const { return img * rows + r; }
    __device__ __forceinline__ int col() const { return strip * kTileStrip + c; }
    __device__ __forceinline__ int bin() const { return row() * bpr + col(); }
    __device__ __forceinline__ void next() {
        if (++c < w) return;
        c = 0;
        if (++r < rows) return;
        r = 0;
        ++strip;
        if (strip > nfull || (strip == nfull && last_w == 0)) { strip = 0; ++img; }
        w = strip < nfull ? kTileStrip : last_w;
    }
};

// chunk_start[bin] = number of chunks in the buckets visited before `bin` (exclusive scan in visiting order),
// chunk_start[nbins] = all of them; chunk_item[c] = (bucket, index within the bucket) of chunk c.  A bucket has
// ceil(n / kTileCap) chunks, n being its largest population over the heads; empty buckets have none.
// xcd_bounds[x] = first chunk of XCD x's share of the list: the shares are consecutive runs of equal cost, a chunk
// being priced at kPassCost per pass (ceil(population / qpp) passes) plus kChunkFixedCost for staging its tiles.  (Shares of equal
// length differ in cost by the chunks of the border tiles, which collect the clamped centres of a whole margin
// of the image and are full, while interior chunks hold a tile's own queries.)  One workgroup of 1024 threads.
constexpr int kPassCost = 2, kChunkFixedCost = 1;     // (measured at cfg3/cfg4: 1+1 and 4+3 within 1 % of 2+1, 1+0 and 2+3 1.5 % off)
// (A template so that every translation unit may include this header; only launch_tile_chunks names it, so one
// translation unit alone holds the kernel.)
template <int Unused = 0>
__global__ __launch_bounds__(1024) void tile_chunks_kernel(TileSort S, int h, int *chunk_start, int qpp) {
    __shared__ int part[1024];
    __shared__ int cost_part[1024];
    const int per = (S.nbins + 1023) / 1024;
    const int b0 = min((int)threadIdx.x * per, S.nbins), b1 = min(b0 + per, S.nbins);
    const int nh = *S.per_head ? h : 1;
    const int full_cost = (kTileCap + qpp - 1) / qpp * kPassCost + kChunkFixedCost;
    auto price = [&](int n, int &chunks, int &cost) __attribute__((always_inline)) {
        const int full = n / kTileCap, rem = n - full * kTileCap;
        chunks += full + (rem ? 1 : 0);
        cost += full * full_cost + (rem ? (rem + qpp - 1) / qpp * kPassCost + kChunkFixedCost : 0);
    };
    // Up to kChunkKeep buckets of a thread stay in registers -- tile and population, the populations fetched by loads
    // that do not depend on one another: one memory round trip instead of one per bucket, and the second walk reads
    // nothing.  Larger maps park the populations in chunk_start between the walks.
    constexpr int kChunkKeep = 4;
    const bool keep = per <= kChunkKeep;
    int kept_bin[kChunkKeep], kept_n[kChunkKeep];
    int sum = 0, cost_sum = 0;
    if (b0 < b1) {
        TileWalk at(S, b0);
        if (keep) {
            int lo[kChunkKeep], hi[kChunkKeep];
            TileWalk tile[kChunkKeep] = {at, at, at, at};
#pragma unroll
            for (int i = 0; i < kChunkKeep; ++i) {
                tile[i] = at;
                kept_bin[i] = at.bin();
                if (b0 + i + 1 < b1) at.next();           // (past the thread's last bucket the tile repeats and is masked below:
                                                          //  no position beyond the buckets is ever formed)
            }
            if (nh > 1) {
                // heads with their own orders: the sort's scatter kernel has left every bucket's largest population
                // over the heads in chunk_start (one load per bucket here instead of four per bucket and head)
#pragma unroll
                for (int i = 0; i < kChunkKeep; ++i) kept_n[i] = clampi(chunk_start[kept_bin[i]], 0, S.L);   // (read from scratch memory: bounded)
            } else {
#pragma unroll
                for (int i = 0; i < kChunkKeep; ++i) bucket_bounds_at(S, 0, kept_bin[i], tile[i].row(), tile[i].col(), lo[i], hi[i]);
#pragma unroll
                for (int i = 0; i < kChunkKeep; ++i) kept_n[i] = hi[i] - lo[i];
            }
#pragma unroll
            for (int i = 0; i < kChunkKeep; ++i) {
                if (b0 + i >= b1) kept_n[i] = 0;
                price(kept_n[i], sum, cost_sum);
            }
        } else {
            for (int pos = b0; pos < b1; ++pos, at.next()) {
                int n;
                if (nh > 1) {
                    n = clampi(chunk_start[at.bin()], 0, S.L);    // (left there by the sort's scatter kernel)
                } else {
                    int lo, hi;
                    bucket_bounds_at(S, 0, at.bin(), at.row(), at.col(), lo, hi);
                    n = hi - lo;
                }
                chunk_start[at.bin()] = n;                // (population for now: the second walk prices the chunks from it)
                price(n, sum, cost_sum);
            }
        }
    }
    part[threadIdx.x] = sum;
    cost_part[threadIdx.x] = cost_sum;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {          // Hillis-Steele inclusive scan of the partial sums
        const int v = (int)threadIdx.x >= d ? part[threadIdx.x - d] : 0;
        const int cv = (int)threadIdx.x >= d ? cost_part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        cost_part[threadIdx.x] += cv;
        __syncthreads();
    }
    const long long total_cost = cost_part[1023];
    int run = part[threadIdx.x] - sum;
    long long cost_run = cost_part[threadIdx.x] - cost_sum;
    int next_share = total_cost > 0 ? (int)(cost_run * 8 / total_cost) + 1 : 8;     // first share bound not yet behind this thread
    // the work list itself: entry = (bucket, which chunk of it), so that a workgroup finds its item with one load
    auto emit = [&](int bin, int n) __attribute__((always_inline)) {
        const int c = (n + kTileCap - 1) / kTileCap;
        chunk_start[bin] = run;
        for (int k = 0; k < c; ++k) {
            if (run + k < S.chunk_cap) S.chunk_item[run + k] = int2{bin, k};
            const int pop = min(n - k * kTileCap, kTileCap);
            const long long after = cost_run + (pop + qpp - 1) / qpp * kPassCost + kChunkFixedCost;
            // share x starts behind the chunk in which the running cost reaches x eighths of the total
            for (; next_share <= 7 && next_share * total_cost <= after * 8; ++next_share)
                S.xcd_bounds[next_share] = min(run + k + 1, S.chunk_cap);
            cost_run = after;
        }
        run += c;
    };
    if (b0 < b1) {
        if (keep) {
#pragma unroll
            for (int i = 0; i < kChunkKeep; ++i)
                if (b0 + i < b1) emit(kept_bin[i], kept_n[i]);
        } else {
            TileWalk at(S, b0);
            for (int pos = b0; pos < b1; ++pos, at.next()) emit(at.bin(), chunk_start[at.bin()]);
        }
    }
    if (threadIdx.x == 1023) {
        chunk_start[S.nbins] = min(part[1023], S.chunk_cap);
        S.xcd_bounds[0] = 0;
        S.xcd_bounds[8] = min(part[1023], S.chunk_cap);
    }
}

// T = half_t, or bf16_t (only in the form that runs both the L1 sums and the aggregation on the matrix unit: 32
// channels per head).  bf16 has no packed arithmetic on this GPU: the differences are taken in fp32 from unpacked
// halves (q is unpacked once per pass) and rounded to bf16 -- where the definition rounds them -- by the packed
// conversion that feeds the matrix instruction; logits and weights are kept as packed bf16 pairs and unpacked by
// shifts where the softmax needs them.
// PAIRED: a head has 64 channels and is handled as two half-heads of 32 (CH = 32 here): the kernel's "heads" are then
// the half-heads -- its head groups, 128 bytes per pixel, are the real heads -- whose L1 sums are added before anything is
// rounded (the two half-heads of a query sit in neighbouring lanes: one cross-lane addition per tap), so that both hold
// the head's logits, run the same softmax and aggregate their own 32 channels with the same weights on the matrix
// unit.  Sampling position, bucket order, attention row and hand-over flag belong to the real head.
template <int CH, int R, int TW, int TH, int VPL, typename T = half_t, bool PAIRED = false>
__global__ __launch_bounds__(kTileNT, MA_TILE_WAVES) void fwd_h16_tile_kernel(FwdArgs A, TileSort S) {
    constexpr bool kBf = std::is_same<T, bf16_t>::value;
    static_assert(kBf || std::is_same<T, half_t>::value, "16-bit storage types");
    typedef TileCfg<CH, R, TW, TH, VPL> Cfg;
    typedef StageCfg<R, VPL> St;
    constexpr int WN = Cfg::WN, M = Cfg::M, HW = WN / 2, BW = Cfg::BW, BH = Cfg::BH;
    constexpr int GB = Cfg::GB, HPG = Cfg::HPG, CPP = Cfg::CPP, PSTR = Cfg::PSTR, LPH = Cfg::LPH, QPP = Cfg::QPP;
    constexpr int G = St::G, SPR = St::SPR, NSR = WN * SPR, LAST0 = (WN - 1) * SPR;

    // With two lanes per head-query and two heads per group (32 channels per head) the aggregation runs on the matrix
    // unit as well (see the V phase below); it needs 32 - BW pixels of readable zeros behind the V tile and, per
    // wavefront, one row of weights (24 halves) for each of its 32 head-queries.
    constexpr bool kMatrixAgg = MA_TILE_MFMA_AGG && LPH == 2 && VPL == 2 && HPG == 2 && CH == 32 && BW <= 24;
    // The V rectangle then has a pixel stride of 136 bytes: one transposing read touches 8 bytes in each of four 16-byte
    // pieces of 16 pixels, which a stride of 128 bytes (32 banks) puts on the same banks eight times over and a stride of
    // 34 banks spreads over all of them (two to three accesses per bank; 128 accesses of two banks on 64 banks).
    constexpr int VSTR = kMatrixAgg ? PSTR + 8 : PSTR;
    constexpr int V_OFF = Cfg::TILE_BYTES;
    constexpr int V_RECT_BYTES = BW * BH * VSTR;
    constexpr int V_BYTES = kMatrixAgg ? (BW * BH + 32 - BW) * VSTR : Cfg::TILE_BYTES;     // with the zeros behind the rectangle
    constexpr int V_ZERO16 = (V_OFF + V_RECT_BYTES + 15) / 16 * 16;                         // 16 aligned bytes of those zeros
    constexpr int WM_ROW_BYTES = 48, WM_WAVE_BYTES = 32 * WM_ROW_BYTES, WM_BYTES = kMatrixAgg ? (kTileNT / 64) * WM_WAVE_BYTES : 0;
    constexpr int WM_OFF = (V_OFF + V_BYTES + 15) / 16 * 16;
    static_assert(WM_OFF + WM_BYTES + 64 <= 80 * 1024, "two workgroups per CU");
    static_assert(!kMatrixAgg || V_ZERO16 + 16 <= V_OFF + V_BYTES, "zeros for the lanes beyond a row");
    __shared__ __attribute__((aligned(16))) char smem[WM_OFF + WM_BYTES];   // K tile, V tile (+ zeros), weight rows

    static_assert(!PAIRED || (CH == 32 && HPG == 2 && VPL == 2), "a head of 64 channels as two half-heads of 32");
    const int nhg = PAIRED ? A.h : A.h / HPG;
    const int npix = S.L;
    const uint32_t row_bytes = (uint32_t)A.C * 2u;
    const uint32_t total_bytes = (uint32_t)npix * row_bytes;
    const __amdgpu_buffer_rsrc_t rq = make_rsrc(A.q, total_bytes);
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(A.k, total_bytes);
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(A.v, total_bytes);
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(A.out, out_span_bytes(A, 2));
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A.attn, attn_span_bytes(A, (uint32_t)(A.h * M), 2));
    const __amdgpu_buffer_rsrc_t rgate = make_rsrc(A.gate, A.gate ? total_bytes : 0u);   // (no gate: every load is out of range)
    const __amdgpu_buffer_rsrc_t rm = make_rsrc(A.mo, (uint32_t)A.nhq * 4u);
    const __amdgpu_buffer_rsrc_t rd = make_rsrc(S.defer, (uint32_t)A.nhq);
    // With two lanes per head-query the pair is lanes l and l ^ 16 of a wavefront (not neighbours): the sum of a
    // tap's |q - k| over the pair's 32 channels is then what one matrix instruction delivers to both lanes
    // (see row_ones0 / row_ones1 below), and the vector ALU is left with the subtractions and the sign masks.
    constexpr bool kMatrixSum = LPH == 2 && VPL == 2;
    const int lane_w = threadIdx.x & 63;
    const int sub = kMatrixSum ? ((lane_w >> 4) & 1) : (int)(threadIdx.x % LPH);
    const int grp = kMatrixSum ? (int)(threadIdx.x >> 6) * 32 + (lane_w & 15) + ((lane_w >> 5) << 4) : (int)(threadIdx.x / LPH);
    const int hslot = grp % HPG, gi = grp / HPG;
    // A operand of v_mfma_f32_16x16x32_f16 (16 x 32, lane i + 16 (k / 8) holds A[i][k..k+7]) that is 1 where row i and
    // column block k / 8 belong to the same half of the wavefront's four 16-lane blocks and 0 elsewhere: with the
    // |q - k| halves as the B operand (lane j + 16 b holds column j, rows 8 b .. 8 b + 7) a result row holds the sum
    // over the 8 halves of lanes l and l ^ 16.  A lane receives rows 4 b .. 4 b + 3 of its column in its four result
    // registers; row_ones0 has its ones in the rows i % 4 == 0 only, row_ones1 in the rows i % 4 == 1, so that an
    // accumulator chained through one instruction with each keeps the two sums apart in registers 0 and 1.
    typedef typename std::conditional<kBf, __bf16, _Float16>::type elem_t;
    typedef elem_t half8_t __attribute__((ext_vector_type(8)));
    typedef float f32x4_t __attribute__((ext_vector_type(4)));
    typedef float float2_t __attribute__((ext_vector_type(2)));
    static_assert(!kBf || (kMatrixSum && MA_TILE_MFMA_AGG && HPG == 2 && CH == 32 && BW <= 24), "bf16: the matrix-unit form only");
    auto mfma16 = [](half8_t a, half8_t b, f32x4_t c) __attribute__((always_inline)) {
        if constexpr (kBf) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
        else return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    };
    // a pair of logits or weights in one register: packed halves, or packed bf16 as plain bits
    typedef typename std::conditional<kBf, uint32_t, half2_t>::type pair_t;
    auto pair_bits = [](pair_t p) __attribute__((always_inline)) { return __builtin_bit_cast(uint32_t, p); };
    auto pair_of = [](uint32_t u) __attribute__((always_inline)) { return __builtin_bit_cast(pair_t, u); };
    auto pair_lo = [](pair_t p) __attribute__((always_inline)) {
        if constexpr (kBf) return as_f32(p << 16); else return (float)p.x;
    };
    auto pair_hi = [](pair_t p) __attribute__((always_inline)) {
        if constexpr (kBf) return as_f32(p & 0xffff0000u); else return (float)p.y;
    };
    [[maybe_unused]] auto pack_bf16 = [](float lo, float hi) __attribute__((always_inline)) {   // both rounded to nearest even
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2_t{lo, hi}, bf16x2_t));
    };
    const uint32_t one_bits = (((lane_w & 15) >= 8) == (lane_w >= 32)) ? (kBf ? 0x3f803f80u : 0x3c003c00u) : 0u;
    const uint32_t ob0 = (lane_w & 3) == 0 ? one_bits : 0u, ob1 = (lane_w & 3) == 1 ? one_bits : 0u;
    [[maybe_unused]] const half8_t row_ones0 = __builtin_bit_cast(half8_t, u32x4{ob0, ob0, ob0, ob0});
    [[maybe_unused]] const half8_t row_ones1 = __builtin_bit_cast(half8_t, u32x4{ob1, ob1, ob1, ob1});
    // bf16: the subtraction q - k itself runs on the matrix unit (v_mfma_f32_16x16x16_bf16: four elements per lane and
    // operand).  With four K values of each of the 64 lanes as the B operand (lane j + 16 b: column j, rows 4 b .. 4 b + 3)
    // and an A operand that holds a single -1 per row -- A[4 b + r][4 b + r] -- result row 4 b + r of column j is minus
    // element r of lane j + 16 b's own four: every lane gets its own four K values back, widened to fp32 and negated,
    // added to the C operand, which holds the same four elements of q (unpacked once per pass).  Two instructions per
    // vector and tap replace the two unpacking and two subtracting vector instructions per word -- there is no packed
    // bf16 arithmetic -- and leave the vector ALU the rounding of the differences to bf16 and the sign mask, as in
    // fp16.  (0 x inf = NaN reaches the other lanes of a column, as with the sums: such head-queries are left to the
    // generic kernel.)
    typedef short short4v_t __attribute__((ext_vector_type(4)));
    [[maybe_unused]] short4v_t sel_neg = {0, 0, 0, 0};
    if constexpr (kBf && MA_TILE_BF16_MFMA_SUB) {
        const bool diag = (lane_w >> 4) == ((lane_w & 15) >> 2);
        const short m1 = (short)0xbf80;                  // -1.0 in bf16
        sel_neg = short4v_t{(short)(diag && (lane_w & 3) == 0 ? m1 : 0), (short)(diag && (lane_w & 3) == 1 ? m1 : 0),
                            (short)(diag && (lane_w & 3) == 2 ? m1 : 0), (short)(diag && (lane_w & 3) == 3 ? m1 : 0)};
    }
    // Lane `sub` owns the 16-byte vectors sub, sub + LPH, ... of its head, so that the lanes of one LDS read
    // touch adjacent 16-byte pieces (vectors 2 sub, 2 sub + 1 would put them 32 bytes apart: 2-way bank
    // conflicts).  With two vectors per lane, odd lane groups take theirs in the opposite order: one LDS
    // read then covers all four 32-byte bank groups of the 128-byte pixels instead of two.
    const int par = VPL == 2 ? (gi & 1) : 0;
    const uint32_t lane_lds = (uint32_t)(hslot * CH * 2 + sub * 16);
    uint32_t vec_off[VPL];                             // byte offset of this lane's vector u inside its head
#pragma unroll
    for (int u = 0; u < VPL; ++u) vec_off[u] = (uint32_t)((u ^ par) * LPH * 16);
    const float nscale = -A.scale;

    // ---- work items: (head group, chunk of at most kTileCap queries per head of one bucket) ----------
    // A fixed grid of persistent workgroups.  Workgroup ids are dealt round-robin to the 8 XCDs; XCD x takes the
    // x-th share of the work list (consecutive chunks, shares of equal cost: tile_chunks_kernel), so that one L2
    // sees one band of neighbouring tiles.  Within that share the workgroups claim items from a counter.
    const int nchunks = min(max(S.chunk_start[S.nbins], 0), S.chunk_cap);
    // Item -> (chunk, head group).  The head groups of a chunk are neighbours in the list: the items an XCD has in
    // flight then cover whole pixel rows of a block of tiles.  (With the head group as the slow index an XCD would
    // touch one 128-byte line in every 128 * nhg bytes, which its L2 maps to a fraction of its sets.)
    auto item_chunk = [&](int it) __attribute__((always_inline)) { return it / nhg; };
    auto item_hgrp = [&](int it) __attribute__((always_inline)) { return it - (it / nhg) * nhg; };
    const int xcd = blockIdx.x & 7;
    // (bounds read from scratch memory are clamped before they become indices)
    const int share_lo = clampi(S.xcd_bounds[xcd], 0, nchunks), share_hi = clampi(S.xcd_bounds[xcd + 1], share_lo, nchunks);
    const int xcd_start = share_lo * nhg, item_end = share_hi * nhg;
    const bool per_head = *S.per_head != 0;
    // Memory round trips of an item, in order: its work-list entry (fetched one item ahead), the bounds of its
    // bucket, the pixel indices of its first two passes -- issued before the staging loads, which return
    // after them -- and the first pass's offset and q row, issued while the staging loads are in flight.
    // The workgroups of an XCD claim the items of its share one by one from a counter (the static stride left
    // up to 8 % of the wave slots idle at the end of the kernel: items take two or three passes).  Thread 0
    // claims two items ahead -- the next item's work-list entry is fetched during the current one -- and hands
    // the index to the workgroup through LDS between the two barriers every item has anyway.  Every workgroup
    // sees the same indices, so all of its wavefronts leave the loop together.
    __shared__ int s_claim;
    int *const queue = S.queue + xcd;
    if (threadIdx.x == 0) s_claim = atomicAdd(queue, 2);
    if constexpr (kMatrixAgg) {                        // the zeros behind the V tile (never written again)
        for (int i = V_RECT_BYTES + threadIdx.x * 8; i < V_BYTES; i += kTileNT * 8) *(u32x2 *)(smem + V_OFF + i) = u32x2{0, 0};
    }
    __syncthreads();
    const int item0 = xcd_start + *(volatile int *)&s_claim;
    int item_next = item0 + 1;
    int2 entry = int2{0, 0};
    if (item0 < item_end) entry = S.chunk_item[item_chunk(item0)];
    for (int item = item0; item < item_end;) {
    int claim = 0;
    if (threadIdx.x == 0) claim = atomicAdd(queue, 1);
    const int hgrp = item_hgrp(item);
    const int bin = clampi(entry.x, 0, S.nbins - 1), part = max(entry.y, 0);
    // this lane group's head and its share of the bucket
    const int head = hgrp * HPG + hslot;               // (PAIRED: the half-head, i.e. the block of 32 channels)
    const int qhead = PAIRED ? hgrp : head;            // the head whose query this is: position, order, attention row, flag
    int lo, hi;
    bucket_bounds(S, per_head ? qhead : 0, bin, lo, hi);
    const int row = bin / S.bins_per_row, tx = bin - row * S.bins_per_row;
    const int b = min(row / S.rows_per_img, npix / A.N - 1), ty = row - (row / S.rows_per_img) * S.rows_per_img;
    const int box_x = tx * TW - R, box_y = ty * TH - R;

    lo = min(lo + part * kTileCap, hi);
    hi = min(hi, lo + kTileCap);
    const uint32_t chan_bytes = (uint32_t)(head * CH + sub * 8) * 2u;      // vector u adds u * LPH * 16 bytes

    auto load_pix_raw = [&](int slot) __attribute__((always_inline)) {
        return S.perm[(size_t)(per_head ? qhead : 0) * npix + min(slot, npix - 1)];
    };
    auto load_pix = [&](int slot) __attribute__((always_inline)) { return clampi(load_pix_raw(slot), 0, npix - 1); };

    // ---- stage the K and V rectangles (replicate-clamped at the image border) -----------------
    // (addresses first, then the two index loads, then the staging loads: arithmetic placed between the
    // loads may name a register an index load is still to fill, and would wait for it)
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
    __builtin_amdgcn_sched_barrier(0);                // (the wait for the pixel indices comes after these loads)
    pix = clampi(pix, 0, npix - 1);
    pix_n = clampi(pix_n, 0, npix - 1);
    uint32_t xyu = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)(pix * A.h + qhead) * 4u), 0, 0);
    u32x4 qv[VPL];
#pragma unroll
    for (int u = 0; u < VPL; ++u) qv[u] = buf_load16(rq, (uint32_t)pix * row_bytes + chan_bytes + vec_off[u]);
    // the next item's entry, behind every load this prologue waits for one by one
    const int item_n = min(item_next, item_end - 1);
    const int2 entry_n = S.chunk_item[item_chunk(item_n)];

    __syncthreads();                                  // every wave is done with the previous tiles
#pragma unroll
    for (int c = 0; c < Cfg::CPT; ++c)
        if (dst[c] != 0xffffffffu) {
            *(u32x4 *)(smem + dst[c]) = kv[0][c];
            if constexpr (kMatrixAgg) {                 // (pixel stride VSTR: 8-byte aligned pieces)
                const uint32_t dv = V_OFF + dst[c] + (dst[c] / PSTR) * (VSTR - PSTR);
                *(u32x2 *)(smem + dv) = u32x2{kv[1][c][0], kv[1][c][1]};
                *(u32x2 *)(smem + dv + 8) = u32x2{kv[1][c][2], kv[1][c][3]};
            } else {
                *(u32x4 *)(smem + Cfg::TILE_BYTES + dst[c]) = kv[1][c];
            }
        }
    if (threadIdx.x == 0) s_claim = claim;

    __syncthreads();                                  // tiles are in place
    const int item_nn = xcd_start + *(volatile int *)&s_claim;

    // Passes.  The loop is bottom-tested: the registers of the next pass are handed over in straight-line
    // code after the stores, so the wait before them covers the loads only, not the stores just issued.
    // Every load issued so far has landed before the loop starts (vmcnt(0)): otherwise the wait the first
    // pass needs for them is repeated in every pass, where it would cover the previous pass's stores.
    __builtin_amdgcn_s_waitcnt(0x0F70);
    bool valid = slot < hi;
    if (__builtin_amdgcn_ballot_w64(valid) != 0) do {
        // next pass: its pixel index is known, fetch its offset and q now; and the index after it
        const int pix_nn = load_pix(slot + 2 * QPP);
        const uint32_t xyu_n = __builtin_amdgcn_raw_buffer_load_b32(rm, (int)((uint32_t)(pix_n * A.h + qhead) * 4u), 0, 0);
        u32x4 qv_n[VPL];
#pragma unroll
        for (int u = 0; u < VPL; ++u) qv_n[u] = buf_load16(rq, (uint32_t)pix_n * row_bytes + chan_bytes + vec_off[u]);
        u32x4 gatev[VPL];                              // this pass's gate values, used at its end
#pragma unroll
        for (int u = 0; u < VPL; ++u) gatev[u] = buf_load16(rgate, (uint32_t)pix * row_bytes + chan_bytes + vec_off[u]);

        const int hq = pix * A.h + qhead;
        const float x = pair_lo(pair_of(xyu)), y = pair_hi(pair_of(xyu));
        float x0, y0, w[4];
        corner_weights<T>(x, y, x0, y0, w);
        // centres far outside the image: every tap is a border pixel whatever the distance
        const int ix = centre_index(x0), iy = centre_index(y0);
        const int cx = ix - R - box_x, cy = iy - R - box_y;
        const bool fits = cx >= 0 && cx + WN <= BW && cy >= 0 && cy + WN <= BH;
        const bool drop_last = A.row_skip && __builtin_amdgcn_ballot_w64(y != y0) == 0;
        const uint32_t tap0 = (uint32_t)(((fits ? cy : 0) * BW + (fits ? cx : 0)) * PSTR) + lane_lds;

        u32x4 buf[2][G][VPL];
        // The tiles are never written inside the loop, so nothing orders these reads for the compiler and it
        // would issue a whole phase of them at once (144 registers).  Each stage therefore takes its address
        // from an opaque copy of tap0, made where the stage is meant to start.
        auto fetch = [&](auto tile_tag, auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            constexpr int base = decltype(tile_tag)::value * Cfg::TILE_BYTES;
            uint32_t at[VPL];
#pragma unroll
            for (int u = 0; u < VPL; ++u) {
                at[u] = tap0 + vec_off[u];
                asm volatile("" : "+v"(at[u]));
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
        pair_t lgp[WN][HW];
        const pair_t ninf2 = pair_of(kBf ? 0xff80ff80u : 0xfc00fc00u);       // (-inf, -inf)
#pragma unroll
        for (int i = 0; i < HW; ++i) lgp[WN - 1][i] = ninf2;                 // stays if the row is left out
        [[maybe_unused]] float qf[VPL][8];                                   // bf16: q unpacked, once per pass
        if constexpr (kBf) {
#pragma unroll
            for (int u = 0; u < VPL; ++u)
#pragma unroll
                for (int e = 0; e < 8; ++e) qf[u][e] = vec_elem<T>(qv[u], e);
        }
        fetch(KT{}, std::integral_constant<int, 0>{});
        float held = 0.f;                               // raw sum of the even tap of a pair until its odd tap is done
        // Running sum of the raw tap sums, for one purpose: a matrix instruction multiplies the |q - k| of all four
        // 16-lane blocks of a column by 0 or 1, and 0 x inf = NaN -- a non-finite q or k value (or a difference that
        // overflows fp16) of one head-query would turn the logits of the unrelated head-query in lanes l ^ 32 into NaN
        // as well.  The sums are >= 0, so the total is finite exactly when every one of them was; head-queries whose
        // total is not are left to the generic kernel, which keeps such values local to the query that owns them.
        // (Where the aggregation runs on the matrix unit as well, only the last window row needs it: a NaN logit makes
        // every weight of its head-query NaN, hence its output, and the aggregation's own check of the results hands it
        // over -- except in the row a lane with integer y drops after the wavefront has computed it, which the generic
        // kernel would multiply by its zero weight: NaN there, lost here.)
        [[maybe_unused]] float finite_check = 0.f;
        static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
            if constexpr (s + 1 < NSR) {
                if (s + 1 < LAST0 || !drop_last) fetch(KT{}, std::integral_constant<int, s + 1>{});
            }
            if (s >= LAST0 && drop_last) return;
#pragma unroll
            for (int t = 0; t < G; ++t) {
                const int i = i0 + t;
                float sum;
                if constexpr (kMatrixSum) {
                    // The two vectors of a lane go through two matrix instructions that leave their sums in different
                    // result rows (row_ones0 / row_ones1), and the vector ALU adds the two: which of a head's vectors is a
                    // lane's vector 0 depends on its lane group (`par`), and one sum chained through both instructions
                    // would round in that order (seen once in 10^9 taps as a logit one fp16 ulp apart between two runs);
                    // an addition does not care.
                    f32x4_t acc4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int u = 0; u < VPL; ++u) {
                        u32x4 ad;
                        if constexpr (kBf && MA_TILE_BF16_MFMA_SUB) {
                            const u32x4 kw = buf[s & 1][t][u];
                            const f32x4_t d0 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(sel_neg, __builtin_bit_cast(short4v_t, u32x2{kw[0], kw[1]}),
                                                                                         f32x4_t{qf[u][0], qf[u][1], qf[u][2], qf[u][3]}, 0, 0, 0);
                            const f32x4_t d1 = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(sel_neg, __builtin_bit_cast(short4v_t, u32x2{kw[2], kw[3]}),
                                                                                         f32x4_t{qf[u][4], qf[u][5], qf[u][6], qf[u][7]}, 0, 0, 0);
                            ad[0] = pack_bf16(d0[0], d0[1]) & 0x7fff7fffu;
                            ad[1] = pack_bf16(d0[2], d0[3]) & 0x7fff7fffu;
                            ad[2] = pack_bf16(d1[0], d1[1]) & 0x7fff7fffu;
                            ad[3] = pack_bf16(d1[2], d1[3]) & 0x7fff7fffu;
                        } else
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            if constexpr (kBf) {
                                const uint32_t kw = buf[s & 1][t][u][e];
                                ad[e] = pack_bf16(qf[u][2 * e] - as_f32(kw << 16), qf[u][2 * e + 1] - as_f32(kw & 0xffff0000u)) & 0x7fff7fffu;
                            } else {
                                ad[e] = h2_as_u32(as_h2(qv[u][e]) - as_h2(buf[s & 1][t][u][e])) & 0x7fff7fffu;
                            }
                        }
                        acc4 = mfma16(u == 0 ? row_ones0 : row_ones1, __builtin_bit_cast(half8_t, ad), acc4);
                    }
                    static_assert(!kMatrixSum || VPL == 2, "one result row per vector of a lane");
                    sum = acc4[0] + acc4[1];
                    if constexpr (PAIRED) {
                        // the other half-head's sum, from the neighbouring lane (DPP quad_perm [1, 0, 3, 2]): an addition
                        // of two floats gives both lanes the same bits
                        sum += dpp_mov<0xB1>(sum);
                    }
                    if constexpr (!kMatrixAgg || j == WN - 1) finite_check += sum;
                } else {
                    sum = l1_sum<T>(qv[0], buf[s & 1][t][0]);
#pragma unroll
                    for (int u = 1; u < VPL; ++u) sum += l1_sum<T>(qv[u], buf[s & 1][t][u]);   // per vector, then added: the
                                                      // same bits whichever order the lane holds its vectors in
                    sum = group_sum<LPH>(sum);
                }
                // the two roundings of a logit (channel sum to fp16, scaled logit to fp16) on a pair of taps at a
                // time: two packed conversions and two multiplications for what took four instructions per tap
                if (!(i & 1)) {
                    held = sum;
                    asm volatile("" : "+v"(held));
                } else if constexpr (kBf) {
                    const uint32_t l16 = pack_bf16(held, sum);
                    uint32_t pinned = pack_bf16(as_f32(l16 << 16) * nscale, as_f32(l16 & 0xffff0000u) * nscale);
                    asm volatile("" : "+v"(pinned));
                    lgp[j][i >> 1] = pair_of(pinned);
                } else {
                    const half2_t l16 = __builtin_convertvector(float2_t{held, sum}, half2_t);
                    // (float)half * scale in one instruction per half: written as a fused multiply-add with a zero addend
                    // the compiler selects v_fma_mix_f32, which reads the half in place (for a plain product it converts
                    // first and multiplies then).  Not inline assembly: the compiler's hazard checks do not look into
                    // it, and its destination may be a register that a matrix instruction still in flight is going to
                    // write (the unused rows of an earlier tap's result) -- one scheduling strategy put it there.
                    const float f_lo = __builtin_fmaf((float)l16.x, nscale, 0.0f);
                    const float f_hi = __builtin_fmaf((float)l16.y, nscale, 0.0f);
                    lgp[j][i >> 1] = __builtin_convertvector(float2_t{f_lo, f_hi}, half2_t);
                    uint32_t pinned = h2_as_u32(lgp[j][i >> 1]);
                    asm volatile("" : "+v"(pinned));
                    lgp[j][i >> 1] = as_h2(pinned);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        });

        // A lane with integer y gives the last row zero weight.  Whether the row was computed depends on the
        // other lanes of the wavefront, which depends on the bucket order; dropping it per lane keeps each
        // result independent of that order.
        if (A.row_skip && y == y0) {
#pragma unroll
            for (int i = 0; i < HW; ++i) lgp[WN - 1][i] = ninf2;
        }

        // ---- window softmax (one exponential per tap around the window maximum) -------------------
        // window maximum and the maximum of the block every sub-window contains, on the packed logits
        float gmax, imax;
        if constexpr (kBf) {
            // no packed maximum for bf16: per column pair, the maxima over all rows and over the rows 1 .. 2R, unpacked
            float call_lo[HW], call_hi[HW], cin_lo[HW], cin_hi[HW];
#pragma unroll
            for (int i = 0; i < HW; ++i) {
                cin_lo[i] = pair_lo(lgp[1][i]); cin_hi[i] = pair_hi(lgp[1][i]);
#pragma unroll
                for (int j = 2; j <= 2 * R; ++j) {
                    cin_lo[i] = fmaxf(cin_lo[i], pair_lo(lgp[j][i]));
                    cin_hi[i] = fmaxf(cin_hi[i], pair_hi(lgp[j][i]));
                }
                call_lo[i] = fmaxf(cin_lo[i], fmaxf(pair_lo(lgp[0][i]), pair_lo(lgp[WN - 1][i])));
                call_hi[i] = fmaxf(cin_hi[i], fmaxf(pair_hi(lgp[0][i]), pair_hi(lgp[WN - 1][i])));
            }
            gmax = fmaxf(call_lo[0], call_hi[0]);
#pragma unroll
            for (int i = 1; i < HW; ++i) gmax = fmaxf(gmax, fmaxf(call_lo[i], call_hi[i]));
            imax = fmaxf(cin_hi[0], cin_lo[HW - 1]);                     // columns 1 and 2R
#pragma unroll
            for (int i = 1; i < HW - 1; ++i) imax = fmaxf(imax, fmaxf(cin_lo[i], cin_hi[i]));
        } else {
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
            gmax = fmaxf((float)mall.x, (float)mall.y);
            imax = fmaxf((float)min2[0].y, (float)min2[HW - 1].x);     // columns 1 and 2R
#pragma unroll
            for (int i = 1; i < HW - 1; ++i) imax = fmaxf(imax, fmaxf((float)min2[i].x, (float)min2[i].y));
        }
        int far = !(gmax - imax < kSharedExpLimit);               // needs the exact per-sub-window softmax
        if constexpr (kMatrixSum) far |= !(finite_check < __builtin_inff());   // (false for NaN too)
        asm volatile("" : "+v"(far));                             // decided here, so that the logits die with the softmax
        pair_t ap[WN][HW];
        if constexpr (kMatrixSum) {
            // Both lanes of a head-query hold all its logits.  Each takes half of the window's rows (lane `sub` rows
            // sub * HR .. sub * HR + HR - 1) through the exponentials, the row sums and the final products, and the two
            // exchange the partial sums of the sub-windows and their finished rows of weights with ds_swizzle (lane ^ 16
            // is the other lane of the pair; the crossbar of the LDS, no memory and no vector ALU cycles): half of the
            // exponentials and conversions, the most expensive instructions of the softmax, per lane.
            constexpr int HR = WN / 2;
            constexpr int kSwapHalves = 0x401f;            // ds_swizzle bit mode: and 0x1f, or 0, xor 0x10
            auto other_f = [&](float x) __attribute__((always_inline)) {
                return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, x), kSwapHalves));
            };
            const bool hi_rows = sub != 0;
            float e[HR][WN];
            const float gl = gmax * kLog2e;
#pragma unroll
            for (int jj = 0; jj < HR; ++jj)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    const pair_t l2 = hi_rows ? lgp[jj + HR][i] : lgp[jj][i];
                    e[jj][2 * i] = __builtin_amdgcn_exp2f(pair_lo(l2) * kLog2e - gl);
                    e[jj][2 * i + 1] = __builtin_amdgcn_exp2f(pair_hi(l2) * kLog2e - gl);
                }
            // row sums over columns 0 .. WN-2 (west sub-windows) and 1 .. WN-1 (east), as subwindow_sum forms them
            float rl[HR], rr[HR];
#pragma unroll
            for (int jj = 0; jj < HR; ++jj) {
                float inner = e[jj][1];
#pragma unroll
                for (int i = 2; i < WN - 1; ++i) inner += e[jj][i];
                rl[jj] = e[jj][0] + inner;
                rr[jj] = inner + e[jj][WN - 1];
            }
            // The sums over the rows every sub-window holds (1 .. WN-2) are added in subwindow_sum's order,
            // ((r1 + r2) + r3) + r4 at WN = 6, so that the result has the bits it had when one lane did it all: the lane
            // of the low rows sends its partial sum r1 + .. + r(HR-1), the lane of the high rows its rows one by one.
            float send_l[HR], send_r[HR];                  // [0 .. HR-2]: the partial sum, or inner rows; [HR-1]: my edge row
            {
                float pl = rl[1], pr = rr[1];
#pragma unroll
                for (int t = 2; t < HR; ++t) { pl += rl[t]; pr += rr[t]; }
#pragma unroll
                for (int t = 0; t < HR - 1; ++t) {
                    send_l[t] = hi_rows ? rl[t] : pl;
                    send_r[t] = hi_rows ? rr[t] : pr;
                }
                send_l[HR - 1] = hi_rows ? rl[HR - 1] : rl[0];
                send_r[HR - 1] = hi_rows ? rr[HR - 1] : rr[0];
            }
            float got_l[HR], got_r[HR];
#pragma unroll
            for (int t = 0; t < HR; ++t) { got_l[t] = other_f(send_l[t]); got_r[t] = other_f(send_r[t]); }
            // low lane: partial = mine, the high rows = theirs; high lane: partial = theirs, the high rows = mine
            float il = hi_rows ? got_l[0] : send_l[0], ir = hi_rows ? got_r[0] : send_r[0];
#pragma unroll
            for (int t = 0; t < HR - 1; ++t) {
                il += hi_rows ? rl[t] : got_l[t];
                ir += hi_rows ? rr[t] : got_r[t];
            }
            float ssum[4], c[4], c9[3][3];
            ssum[0] = (hi_rows ? got_l[HR - 1] : send_l[HR - 1]) + il;    // north-west: row 0 + rows 1 .. WN-2
            ssum[1] = (hi_rows ? got_r[HR - 1] : send_r[HR - 1]) + ir;
            ssum[2] = il + (hi_rows ? send_l[HR - 1] : got_l[HR - 1]);    // south-west: rows 1 .. WN-2 + row WN-1
            ssum[3] = ir + (hi_rows ? send_r[HR - 1] : got_r[HR - 1]);
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) c[bb] = w[bb] * __builtin_amdgcn_rcpf(ssum[bb]);
            coef9<R>(c, c9);
            pair_t mine[HR][HW], theirs[HR][HW];
#pragma unroll
            for (int jj = 0; jj < HR; ++jj) {
                // class of my row jj among the window's rows: first, last, or in between
                float cr[3];
#pragma unroll
                for (int ii = 0; ii < 3; ++ii)
                    cr[ii] = jj == 0 ? (hi_rows ? c9[1][ii] : c9[0][ii]) : (jj == HR - 1 ? (hi_rows ? c9[2][ii] : c9[1][ii]) : c9[1][ii]);
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    // product of two floats rounded once to fp16, one instruction per weight (v_fma_mixlo_f16 /
                    // v_fma_mixhi_f16, selected for a fused multiply-add with a zero addend; the plain product became a
                    // multiplication and a packed conversion: two roundings, three instructions per pair)
                    if constexpr (kBf) {
                        mine[jj][i] = pack_bf16(e[jj][2 * i] * cr[cls<R>(2 * i)], e[jj][2 * i + 1] * cr[cls<R>(2 * i + 1)]);
                    } else {
                        half2_t t2;
                        t2.x = (half_t)__builtin_fmaf(e[jj][2 * i], cr[cls<R>(2 * i)], 0.0f);
                        t2.y = (half_t)__builtin_fmaf(e[jj][2 * i + 1], cr[cls<R>(2 * i + 1)], 0.0f);
                        mine[jj][i] = t2;
                    }
                }
            }
#pragma unroll
            for (int jj = 0; jj < HR; ++jj)
#pragma unroll
                for (int i = 0; i < HW; ++i)
                    theirs[jj][i] = pair_of((uint32_t)__builtin_amdgcn_ds_swizzle((int)pair_bits(mine[jj][i]), kSwapHalves));
#pragma unroll
            for (int jj = 0; jj < HR; ++jj)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    ap[jj][i] = hi_rows ? theirs[jj][i] : mine[jj][i];
                    ap[jj + HR][i] = hi_rows ? mine[jj][i] : theirs[jj][i];
                }
        } else {
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
            for (int bb = 0; bb < 4; ++bb) c[bb] = w[bb] * __builtin_amdgcn_rcpf(ssum[bb]);
            coef9<R>(c, c9);
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    ap[j][i].x = (half_t)(e[j][2 * i] * c9[cls<R>(j)][cls<R>(2 * i)]);
                    ap[j][i].y = (half_t)(e[j][2 * i + 1] * c9[cls<R>(j)][cls<R>(2 * i + 1)]);
                }
        }
        auto store_attn = [&](bool mine) __attribute__((always_inline)) {
            // The attention row of a head-query (M/2 dwords) leaves in 16-byte pieces dealt to the LPH lanes of the
            // head-query -- piece p from lane p % LPH -- so that one store instruction covers LPH * 16 contiguous bytes per
            // head-query (8-byte stores from one lane made nine requests to L2 per row, three quarters of all the
            // requests of the kernel).  The dwords left over (2 at M = 36) follow as one 8-byte store.
            {
                constexpr int NDW = M / 2, NP = NDW / 4, REM = NDW - NP * 4;
                uint32_t dw[NDW];
#pragma unroll
                for (int m = 0; m < NDW; ++m) dw[m] = pair_bits(ap[m / HW][m % HW]);
                const uint32_t a_row = mine ? (uint32_t)pix * A.attn_row_bytes + (uint32_t)qhead * (uint32_t)(M * 2) : kDeadOffset;
#pragma unroll
                for (int t = 0; t * LPH < NP; ++t) {
                    u32x4 piece = u32x4{dw[0], dw[1], dw[2], dw[3]};
#pragma unroll
                    for (int sl = 0; sl < LPH; ++sl) {
                        const int pc = t * LPH + sl;
                        if (pc < NP && sub == sl) piece = u32x4{dw[4 * pc], dw[4 * pc + 1], dw[4 * pc + 2], dw[4 * pc + 3]};
                    }
                    const int mine_pc = t * LPH + sub;
                    buf_store16(ra, (mine && mine_pc < NP) ? a_row + (uint32_t)mine_pc * 16u : kDeadOffset, piece);
                }
                static_assert(REM == 0 || REM == 2, "attention rows are a whole number of 8-byte pieces");
                if (REM == 2)
                    buf_store8(ra, (mine && sub == NP % LPH) ? a_row + (uint32_t)NP * 16u : kDeadOffset, u32x2{dw[NP * 4], dw[NP * 4 + 1]});
            }
        };
        if constexpr (kMatrixAgg) {
            // ---- aggregation on the matrix unit ------------------------------------------------------------------
            // out^T = V^T W per head: 16 channels x 32 pixels of one row of the staged V rectangle (A operand) times the
            // weights that 16 head-queries of that head give those 32 pixels (B operand: zero except where the row crosses
            // a head-query's window), accumulated over the rows the wavefront's windows reach.  The rectangle stays
            // pixel-major: the A operand comes from ds_read_b64_tr_b16, which hands lane l of a 16-lane block the element
            // l % 4 of what lanes l / 4 + 4 e (e = 0..3) of the block address -- source lane 4 e + q reads channels
            // 8 q + 4 cb .. + 3 of pixel e, so lane l = 4 q + c receives channel 8 q + 4 cb + c of four consecutive
            // pixels.  The B operand goes through LDS: every head-query writes the weights of its window row at its
            // window's columns into its row of a 24-entry table (zeroed once per pass: a head-query always writes the
            // same entries), and lane j + 16 g reads entries 8 g .. 8 g + 7 of head-query j.  Result rows 4 b + r of the
            // two channel blocks are channels 8 b + r and 8 b + 4 + r: lane j + 16 b ends with 16 contiguous bytes of
            // head-query j's output.  The buckets are ordered by the window's row in the tile, so the 16 queries of a
            // wavefront start in neighbouring rows: the rows are walked from the first window's first row, a lane whose
            // window starts `delta` rows later takes its weights from row t - delta.  (Every delta the tile allows is
            // handled here: which queries share a wavefront depends on the arrival order inside a bucket, and a result
            // must not.)
            typedef short short4_t __attribute__((ext_vector_type(4)));
            typedef short short8_t __attribute__((ext_vector_type(8)));
            constexpr int kMaxDelta = BH - WN, NT = WN + kMaxDelta;
            const int grp_local = (lane_w & 15) + ((lane_w >> 5) << 4);       // own head-query within the wavefront
            const int qq = grp_local >> 1;                                      // its query (0..15); hslot is its head
            const int cxv = fits ? cx : 0, cyv = fits ? cy : 0;
            uint32_t cy_mask = 0;
#pragma unroll
            for (int c = 0; c <= BH - WN; ++c) cy_mask |= __builtin_amdgcn_ballot_w64(cyv == c) != 0 ? (1u << c) : 0u;
            const int cy_min = __builtin_ctz(cy_mask), spread = 31 - __builtin_clz(cy_mask) - cy_min;
            const int delta = cyv - cy_min;
            const int t_hi = min(spread, kMaxDelta) + WN - 1 - (drop_last ? 1 : 0);     // last row step with a weight in it
            const bool mine = valid && fits && !far;
            store_attn(mine && (!PAIRED || hslot == 0));   // (PAIRED: both half-heads hold the row; one writes it)
            char *const wm = smem + WM_OFF + (threadIdx.x >> 6) * WM_WAVE_BYTES;
            const int jcol = lane_w & 15, gblk = lane_w >> 4;
            // lane `sub` of a head-query writes the halves sub, 2 + sub, ... of a window row: kept in the low halves
            uint32_t wv[WN][HW];
#pragma unroll
            for (int j = 0; j < WN; ++j)
#pragma unroll
                for (int i = 0; i < HW; ++i) wv[j][i] = sub ? pair_bits(ap[j][i]) >> 16 : pair_bits(ap[j][i]);
            const uint32_t wm_write = (uint32_t)((hslot * 16 + qq) * WM_ROW_BYTES + (cxv + sub) * 2);
            // (pixels 24 .. 31 of a step lie beyond the rectangle's row: those lanes read zeros, behind the V rectangle)
            uint32_t wm_read[HPG];
#pragma unroll
            for (int hg = 0; hg < HPG; ++hg)
                wm_read[hg] = gblk < 3 ? (uint32_t)(WM_OFF + (threadIdx.x >> 6) * WM_WAVE_BYTES + (hg * 16 + jcol) * WM_ROW_BYTES + gblk * 16)
                                       : (uint32_t)V_ZERO16;
            // source address of the transposing reads: pixel 8 g + e of the first row, channels 8 q .. of head 0, block 0
            const uint32_t a_base = (uint32_t)(V_OFF + (cy_min * BW + 8 * gblk + ((lane_w & 15) >> 2)) * VSTR + (lane_w & 3) * 16);
            // owner lanes of the head-queries this lane stores (column jcol of either head), for their pixel and flags
            int pix_o[HPG], mine_o[HPG], valid_o[HPG];
#pragma unroll
            for (int hg = 0; hg < HPG; ++hg) {
                const int gl = 2 * jcol + hg, owner = (gl & 15) + ((gl >> 4) << 5);
                pix_o[hg] = __builtin_amdgcn_ds_bpermute(owner * 4, pix);
                const int fl = __builtin_amdgcn_ds_bpermute(owner * 4, (mine ? 1 : 0) | (valid ? 2 : 0));
                mine_o[hg] = fl & 1;
                valid_o[hg] = fl & 2;
            }
            u32x4 gate_o[HPG];
#pragma unroll
            for (int hg = 0; hg < HPG; ++hg)
                gate_o[hg] = buf_load16(rgate, (uint32_t)pix_o[hg] * row_bytes + (uint32_t)((hgrp * HPG + hg) * CH * 2 + gblk * 16));
            f32x4_t dacc[HPG][2];
#pragma unroll
            for (int hg = 0; hg < HPG; ++hg)
#pragma unroll
                for (int cb = 0; cb < 2; ++cb) dacc[hg][cb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            *(u32x4 *)(wm + lane_w * 16) = u32x4{0, 0, 0, 0};
            if (lane_w < (WM_WAVE_BYTES - 1024) / 16) *(u32x4 *)(wm + 1024 + lane_w * 16) = u32x4{0, 0, 0, 0};
            // One row step's operands: the transposing reads of the V rectangle, this lane's weights for the row into the
            // table, the reads of the table.  LDS instructions of a wavefront execute in order, so the table may be
            // rewritten for the next step as soon as the reads of this one are issued: the steps are issued one ahead of
            // the matrix instructions that use them.
            struct RowOps { half8_t a[HPG][2], b[HPG]; };
            RowOps ops[2];
            auto load_row = [&](auto t_tag) __attribute__((always_inline)) {
                constexpr int t = decltype(t_tag)::value;
                RowOps &o = ops[t & 1];
#pragma unroll
                for (int hg = 0; hg < HPG; ++hg)
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb) {
                        const short4_t lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) short4_t *)(smem + a_base + (uint32_t)(t * BW * VSTR + hg * CH * 2 + cb * 8)));
                        const short4_t hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                            (__attribute__((address_space(3))) short4_t *)(smem + a_base + (uint32_t)(t * BW * VSTR + hg * CH * 2 + cb * 8 + 4 * VSTR)));
                        o.a[hg][cb] = __builtin_bit_cast(half8_t, (short8_t)__builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
                    }
#pragma unroll
                for (int i = 0; i < HW; ++i) {
                    uint32_t d = 0u;                    // this lane's window row t - delta, if there is one
#pragma unroll
                    for (int dl = 0; dl <= kMaxDelta; ++dl)
                        if (t - dl >= 0 && t - dl < WN) d = delta == dl ? wv[t - dl][i] : d;
                    *(uint16_t *)(wm + wm_write + 4 * i) = (uint16_t)d;
                }
#pragma unroll
                for (int hg = 0; hg < HPG; ++hg) o.b[hg] = __builtin_bit_cast(half8_t, *(const u32x4 *)(smem + wm_read[hg]));
            };
            auto mma_row = [&](auto t_tag) __attribute__((always_inline)) {
                const RowOps &o = ops[decltype(t_tag)::value & 1];
#pragma unroll
                for (int hg = 0; hg < HPG; ++hg)
#pragma unroll
                    for (int cb = 0; cb < 2; ++cb)
                        dacc[hg][cb] = mfma16(o.a[hg][cb], o.b[hg], dacc[hg][cb]);
            };
            load_row(std::integral_constant<int, 0>{});
            static_for<0, NT>([&](auto t_tag) __attribute__((always_inline)) {
                constexpr int t = decltype(t_tag)::value;
                if (t > t_hi) return;                  // (the same in every lane)
                if constexpr (t + 1 < NT) {
                    if (t + 1 <= t_hi) load_row(std::integral_constant<int, t + 1>{});
                }
                mma_row(t_tag);
            });
            // A non-finite value in the rectangle multiplies every head-query's zeros: head-queries whose result is not
            // finite are left to the generic kernel, which keeps such values with the windows that hold them.
            u32x4 ov[HPG];
            bool ok_o[HPG];
            const unsigned long long col = 0x0001000100010001ull << jcol;     // the four lanes that hold column jcol
#pragma unroll
            for (int hg = 0; hg < HPG; ++hg) {
                float o8[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) { o8[e] = dacc[hg][0][e]; o8[4 + e] = dacc[hg][1][e]; }
                ov[hg] = vec_pack<T>(o8);
                uint32_t any = 0u;                     // bit 15 / 31 set where a half has all exponent bits set
#pragma unroll
                for (int e = 0; e < 4; ++e) any |= (ov[hg][e] & 0x7fff7fffu) + (kBf ? 0x00800080u : 0x04000400u);
                const unsigned long long bad_m = __builtin_amdgcn_ballot_w64((any & 0x80008000u) != 0u);
                ok_o[hg] = mine_o[hg] != 0 && (bad_m & col) == 0;
            }
            if constexpr (PAIRED) ok_o[0] = ok_o[1] = ok_o[0] && ok_o[1];     // one head-query: all 64 channels, or none
            if (A.gate) {
#pragma unroll
                for (int hg = 0; hg < HPG; ++hg) ov[hg] = vec_mul<T>(ov[hg], gate_o[hg]);
            }
#pragma unroll
            for (int hg = 0; hg < HPG; ++hg) {
                const int head_o = hgrp * HPG + hg;
                // the flag of the head-query (its valid owner wrote nothing: one store per head-query, from block 0's lane)
                if (!PAIRED || hg == 0)
                    __builtin_amdgcn_raw_buffer_store_b8((uint8_t)(ok_o[hg] ? 0 : 1), rd, (valid_o[hg] && gblk == 0) ? pix_o[hg] * A.h + (PAIRED ? hgrp : head_o) : (int)kDeadOffset, 0, 0);
                buf_store16(ro, ok_o[hg] ? (uint32_t)pix_o[hg] * A.out_row_bytes + (uint32_t)(head_o * CH * 2 + gblk * 16) : kDeadOffset, ov[hg]);
            }
        } else {
            __builtin_amdgcn_sched_barrier(0);
            {   // the first V stage waits for the last attention weight (keeps it below the softmax)
                uint32_t last = h2_as_u32(ap[WN - 2][HW - 1]);
                asm volatile("" : "+v"(last));
                ap[WN - 2][HW - 1] = as_h2(last);
            }
            fetch(VT{}, std::integral_constant<int, 0>{});

            // ---- aggregation -----------------------------------------------------------------------
            float acc[VPL][8];
    #pragma unroll
            for (int u = 0; u < VPL; ++u)
    #pragma unroll
                for (int e = 0; e < 8; ++e) acc[u][e] = 0.f;
            static_for<0, NSR>([&](auto s_tag) __attribute__((always_inline)) {
                constexpr int s = decltype(s_tag)::value, j = s / SPR, i0 = (s % SPR) * G;
                if constexpr (s + 1 < NSR) {
                    if (s + 1 < LAST0 || !drop_last) fetch(VT{}, std::integral_constant<int, s + 1>{});
                }
                if (s >= LAST0 && drop_last) return;
    #pragma unroll
                for (int t = 0; t < G; ++t) {
                    // One fused multiply-add per tap and channel, nothing wider: left free to contract across statements the
                    // compiler joins the two taps of one weight pair into a two-element dot product for a single channel of
                    // one vector, which rounds differently -- and which vector of the head a lane holds depends on where the
                    // bucket order puts the query.
    #pragma clang fp contract(on)
                    const int i = i0 + t;
                    const float am = (float)((i & 1) ? ap[j][i >> 1].y : ap[j][i >> 1].x);
    #pragma unroll
                    for (int u = 0; u < VPL; ++u)
    #pragma unroll
                        for (int e = 0; e < 8; ++e) acc[u][e] += am * vec_elem<T>(buf[s & 1][t][u], e);
                }
                // this stage's sums are complete before the next stage's reads are issued
    #pragma unroll
                for (int u = 0; u < VPL; ++u)
                    asm volatile("" : "+v"(acc[u][0]), "+v"(acc[u][1]), "+v"(acc[u][2]), "+v"(acc[u][3]), "+v"(acc[u][4]), "+v"(acc[u][5]), "+v"(acc[u][6]), "+v"(acc[u][7]));
                __builtin_amdgcn_sched_barrier(0);
            });

            // ---- stores; what this tile cannot serve is flagged for the generic kernel --------------------
            // (a flag per head-query, written with the results: no atomics, no zero-fill, and nothing the next
            // pass has to wait for)
            const bool mine = valid && fits && !far;
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
            store_attn(mine);
        }

        slot += QPP;
        pix = pix_n; pix_n = pix_nn; xyu = xyu_n;
#pragma unroll
        for (int u = 0; u < VPL; ++u) qv[u] = qv_n[u];
        valid = slot < hi;
    } while (__builtin_amdgcn_ballot_w64(valid) != 0);          // later passes have larger slots still
    entry = entry_n;
    item = item_next;
    item_next = item_nn;
    }   // items
}

}  // namespace ma

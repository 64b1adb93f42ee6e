// Ordering of the queries by sampling target (gfx950): a counting sort whose bins are pixels, 8-column groups or
// K/V tiles, depending on who asks.
//
//   * the direct forward may walk the queries in the order of coarse target bins (batch item, target row, 8-column
//     group) when the field is incoherent: lanes and wavefronts that run together then touch adjacent K/V lines;
//   * the LDS-tile kernels take their work from buckets of one K/V tile each (optionally cut into sub-buckets by the
//     row of the window inside the tile);
//   * the backward's per-key pass follows an exact inverse index: one bin per target pixel, the entries of a bin in
//     ascending pixel order (so that every sum runs in a fixed order), the window centres kept beside them.
// The result of a query never depends on the order, so outputs do not change with it.
//
// Kernels, in stream order (perm[hd][slot] = pixel index is what they fill):
//   probe         whether the ordering is worth using (incoherent field; skipped when it is not optional) and whether
//                 every head of every pixel falls in head 0's bin (one offset shared by the heads: one order serves all)
//   count         bin counts and the arrival rank of each pixel within its bin (a grid row per head; the rows of heads
//                 1.. leave when the heads share head 0's order)
//   rowscan,      exclusive prefix sums: the bins of a bin row by one wavefront, then the row totals
//   rowtot_scan
//   scatter       perm[hd][start[bin] + rank] = pixel (and its centre); by the way, the bucket populations the tile
//                 work list is cut from
//   bin_order,    exact index only: the entries of every bin into ascending pixel order (one thread per small bin, one
//   big_bins_*    thread per entry of the large bins along the border)
//   small         exact index of maps up to kSmallSortMaxN pixels: everything after the probe in one launch, one
//                 workgroup per image and head
#pragma once
#include "matchattn_common.h"

namespace ma {

struct SortArgs {
    const void *mo;
    int dtype;             // MATCHATTN_F32 / F16 / BF16 numbering
    int L, N, H, W, h;     // L = B*N pixels
    int bin_w;             // a bin is bin_w columns wide (1: exact inverse index; the tile width for the tile buckets)
    int force;             // 1: always sort (inverse index for the backward); 0: only when the probe finds it useful
    int bin_h;             // a bin is bin_h rows tall (1 except for the tile buckets of the LDS-tile kernels)
    int sub_h;             // 1, or bin_h: every bin is cut into bin_h sub-bins by the row inside it, numbered one after the
                           //   other (bins_per_row, nbins, count then refer to sub-bins): a tile's queries come out ordered
                           //   by the row of their window in the tile, and its bucket is still one run of the order
    int shared_perm;       // 1: when the heads share head 0's order only perm[0] is written (the consumer reads
                           //    per_head[0] and follows head 0's row); 0: every head's row is always complete
    int rows_per_img;      // ceil(H / bin_h)
    int bins_per_row;      // ceil(W / bin_w) * sub_h
    int nbins;             // nrows * bins_per_row
    int nrows;             // B * rows_per_img rows of bins
    int *count;            // [h][nbins]  (zero on entry; after the scans: start of the bin within its row)
    int *rowtot;           // [h][nrows]  (after the scans: start of the row)
    int *rank;             // [h][L]
    int *perm;             // [h][L]
    int *centre;           // optional [h][L]: centre of the entry at the same position, (cy << 16) | (cx & 0xffff),
                           //   each saturated to int16 (enough to decide which taps reach a key); or null
    int *pop;              // optional [nbins]: when the heads have their own orders, the scatter kernel leaves the largest
                           //   population of each bin over the heads here (the LDS-tile work list is cut from it); or null
    int *per_head;         // the 256-byte flag block (zero on entry, layout below): [kFlagPerHead] heads need their own
                           //     permutation, [kFlagIncoherent] number of (pixel, head) pairs whose target is not next to
                           //     their left neighbour's
};
// Words of the flag block the sort zeroes with its counters (64 ints).  The LDS-tile kernels keep their work
// counters, one per XCD, in the same block (TileSort::queue = per_head + kFlagQueue), and the work list's split among
// the XCDs (TileSort::xcd_bounds = per_head + kFlagXcdBounds).
constexpr int kFlagPerHead = 0, kFlagIncoherent = 1, kFlagQueue = 8, kFlagQueueSlots = 8, kFlagXcdBounds = 16, kFlagXcdBoundSlots = 9,
              kFlagWords = 64;
static_assert(kFlagQueue + kFlagQueueSlots <= kFlagXcdBounds && kFlagXcdBounds + kFlagXcdBoundSlots <= kFlagWords, "flag block layout");

__device__ __forceinline__ void load_xy(const void *mo, int dtype, size_t idx, float &x, float &y) {
    if (dtype == 0) {
        const float2 v = ((const float2 *)mo)[idx];
        x = v.x; y = v.y;
    } else if (dtype == 1) {
        const half2_t v = ((const half2_t *)mo)[idx];
        x = (float)v.x; y = (float)v.y;
    } else {
        const uint32_t v = ((const uint32_t *)mo)[idx];
        x = as_f32(v << 16); y = as_f32(v & 0xffff0000u);
    }
}

// The same with the element type fixed at compile time: no branch around the load, so that several loads of
// one thread stay in flight together (inside a branch the conversion waits for its load).
template <int DT>
__device__ __forceinline__ void load_xy_as(const void *mo, size_t idx, float &x, float &y) {
    if constexpr (DT == 0) {
        const float2 v = ((const float2 *)mo)[idx];
        x = v.x; y = v.y;
    } else if constexpr (DT == 1) {
        const half2_t v = ((const half2_t *)mo)[idx];
        x = (float)v.x; y = (float)v.y;
    } else {
        const uint32_t v = ((const uint32_t *)mo)[idx];
        x = as_f32(v << 16); y = as_f32(v & 0xffff0000u);
    }
}

__device__ __forceinline__ int pack_centre(float x, float y) {
    const int cx = centre_index(floorf(x)), cy = centre_index(floorf(y));
    return (int)(((uint32_t)cy << 16) | ((uint32_t)cx & 0xffffu));
}

// (row of bins within the image, column of bins) of a sampling position, packed
__device__ __forceinline__ uint32_t target_cell(const SortArgs &S, float x, float y) {
    const int ix = clampi((int)floorf(fminf(fmaxf(x, -1e6f), 1e6f)), 0, S.W - 1);
    const int iy = clampi((int)floorf(fminf(fmaxf(y, -1e6f), 1e6f)), 0, S.H - 1);
    // (unsigned division by a small run-time constant; powers of two take the shift)
    const uint32_t bw = (uint32_t)S.bin_w, bh = (uint32_t)S.bin_h;
    const uint32_t cx = (bw & (bw - 1)) == 0 ? (uint32_t)ix >> __builtin_ctz(bw) : (uint32_t)ix / bw;
    const uint32_t cy = (bh & (bh - 1)) == 0 ? (uint32_t)iy >> __builtin_ctz(bh) : (uint32_t)iy / bh;
    if (S.sub_h > 1) return (cy << 16) | (cx * (uint32_t)S.sub_h + ((uint32_t)iy - cy * bh));
    return (cy << 16) | cx;
}

__device__ __forceinline__ int target_bin(const SortArgs &S, int pix, float x, float y) {
    const uint32_t cell = target_cell(S, x, y);
    const int b = pix / S.N;
    return (b * S.rows_per_img + (int)(cell >> 16)) * S.bins_per_row + (int)(cell & 0xffffu);
}

// The ordering pays only when neighbouring queries gather from unrelated places.  A field is
// called coherent when a pixel's target sits next to its left neighbour's (per head); the ordering is
// used when more than 1/8 of the (pixel, head) pairs are not (decided on the device: no host round trip).
__device__ __forceinline__ bool sort_useful(const SortArgs &S) {
    return S.force || (long long)S.per_head[kFlagIncoherent] * 8 > (long long)S.L * S.h;
}

// One thread per (pixel, head) and step of a grid-stride loop: the loads of a wavefront are adjacent, and a
// thread compares its position with head 0's of its pixel and with the same head's of the pixel to its left.
// A workgroup adds to the two flags at most once each (every wavefront adding to one address costs about
// 13 ns each: over 100 us with one wavefront per 64 pixels at 0.5 M pixels).
constexpr int kProbeBlocks = 1024;
template <int DT>
__global__ __launch_bounds__(256) void sort_probe_kernel(SortArgs S) {
    __shared__ int part_n[4], part_d[4];
    const long long total = (long long)S.L * S.h;
    int n = 0;                 // wavefront-uniform: (pixel, head) pairs not next to their left neighbour's target
    bool differ = false;
    constexpr int UNR = 4;     // independent elements per thread and step
    // (32-bit index arithmetic, the head from a shift where the head count allows: the kernel is otherwise bound
    // by integer division, not by its loads)
    const uint32_t total32 = (uint32_t)total, stride = gridDim.x * 256u, uh = (uint32_t)S.h;
    const int hshift = (uh & (uh - 1)) == 0 ? __builtin_ctz(uh) : -1;
    const bool from_lane = hshift >= 0 && uh <= 64u;
    for (uint32_t base = blockIdx.x * 256u; base < total32; base += stride * UNR) {
        float x[UNR], y[UNR], xl[UNR], yl[UNR], x0[UNR], y0[UNR];
        bool in[UNR], other[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const uint32_t idx = base + u * stride + threadIdx.x;     // (the host checks total < 2^31, so this does not wrap)
            in[u] = idx < total32;
            const uint32_t at = in[u] ? idx : 0u;
            const uint32_t hd = hshift >= 0 ? (at & (uh - 1)) : at % uh;
            other[u] = in[u] && hd != 0;
            load_xy_as<DT>(S.mo, (size_t)at, x[u], y[u]);
            if (!from_lane) load_xy_as<DT>(S.mo, (size_t)(at - hd), x0[u], y0[u]);
            xl[u] = x[u] - 1.0f; yl[u] = y[u];
            if (!S.force) {
                const uint32_t pix = hshift >= 0 ? at >> hshift : at / uh;
                if (pix % (uint32_t)S.W != 0) load_xy_as<DT>(S.mo, (size_t)(at - uh), xl[u], yl[u]);
            }
        }
        if (from_lane) {
            // head 0 of a lane's pixel sits h-aligned in the same wavefront (indices are lane-aligned: base and stride
            // are multiples of 256): its position comes from that lane's registers, not from a second load
            const int src = (int)(threadIdx.x & 63u & ~(uh - 1u));
#pragma unroll
            for (int u = 0; u < UNR; ++u) {
                x0[u] = __shfl(x[u], src);
                y0[u] = __shfl(y[u], src);
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const bool incoherent = in[u] && (fabsf(x[u] - xl[u] - 1.0f) > 8.0f || fabsf(y[u] - yl[u]) > 2.0f);
            // exact index: heads share an index only if their (unclamped) centres coincide, because
            // the stored centre of head 0 then stands for every head; coarse ordering: same cell suffices
            // (same pixel, so the same batch item)
            // (equal positions need no cells: with shared positions, the usual case, the wavefront skips the arithmetic
            // that otherwise bounds this kernel)
            const bool unequal = other[u] && !(x[u] == x0[u] && y[u] == y0[u]);
            if (__builtin_amdgcn_ballot_w64(unequal) != 0 && unequal)
                differ = differ || (S.bin_w == 1 ? pack_centre(x[u], y[u]) != pack_centre(x0[u], y0[u])
                                                     : target_cell(S, x[u], y[u]) != target_cell(S, x0[u], y0[u]));
            if (!S.force) n += __builtin_popcountll(__builtin_amdgcn_ballot_w64(incoherent));
        }
    }
    const int wave = threadIdx.x >> 6;
    const int any_differ = __builtin_amdgcn_ballot_w64(differ) != 0 ? 1 : 0;    // (taken by all lanes together)
    if ((threadIdx.x & 63) == 0) {
        part_n[wave] = n;
        part_d[wave] = any_differ;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int tn = part_n[0] + part_n[1] + part_n[2] + part_n[3];
        if (tn) atomicAdd(&S.per_head[kFlagIncoherent], tn);
        // (the others look first: one workgroup setting the flag is enough)
        if ((part_d[0] | part_d[1] | part_d[2] | part_d[3]) &&
            __hip_atomic_load(&S.per_head[kFlagPerHead], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0)
            atomicOr(&S.per_head[kFlagPerHead], 1);
    }
}

// Bin counts and ranks.  A workgroup first counts its entries in an LDS table keyed by the low bits of
// the bin (neighbouring pixels mostly share a handful of bins), then adds each occupied table entry to
// the global counter once; an entry whose table slot is taken by another bin goes to the global counter
// directly.  Ranks inside a bin are arbitrary, as with one atomic per entry, but far fewer contend.
constexpr int kCountTable = 2048, kCountPerThread = 4;
// One workgroup counts 1024 pixels of one head, four per thread (grid.y = heads; the rows of heads 1.. exit when the
// heads share their offsets: head 0 then stands for all of them).  The more entries a workgroup sees, the more of
// them share a bin: with the sub-buckets of the tile sort 256 entries hardly ever did, and every one of them cost a
// global atomic.
__global__ __launch_bounds__(256) void sort_count_kernel(SortArgs S) {
    __shared__ int tag[kCountTable], cnt[kCountTable], base[kCountTable];
    const int hd = blockIdx.y;
    if (!sort_useful(S) || (hd > 0 && *S.per_head == 0)) return;    // uniform over the workgroup
    for (int i = threadIdx.x; i < kCountTable; i += blockDim.x) { tag[i] = -1; cnt[i] = 0; }
    int *const count = S.count + (size_t)hd * S.nbins;
    int *const rank = S.rank + (size_t)hd * S.L;
    int pix[kCountPerThread], bin[kCountPerThread], local[kCountPerThread];
    float x[kCountPerThread], y[kCountPerThread];
#pragma unroll
    for (int u = 0; u < kCountPerThread; ++u) {
        pix[u] = (blockIdx.x * kCountPerThread + u) * (int)blockDim.x + (int)threadIdx.x;
        load_xy(S.mo, S.dtype, (size_t)min(pix[u], S.L - 1) * S.h + hd, x[u], y[u]);
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kCountPerThread; ++u) {
        local[u] = -1;
        bin[u] = 0;
        if (pix[u] < S.L) {
            bin[u] = target_bin(S, pix[u], x[u], y[u]);
            const int idx = bin[u] & (kCountTable - 1);
            const int old = atomicCAS(&tag[idx], -1, bin[u]);
            if (old == -1 || old == bin[u]) local[u] = atomicAdd(&cnt[idx], 1);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kCountTable; i += blockDim.x)
        if (tag[i] >= 0) base[i] = atomicAdd(&count[tag[i]], cnt[i]);
    __syncthreads();
#pragma unroll
    for (int u = 0; u < kCountPerThread; ++u)
        if (pix[u] < S.L) rank[pix[u]] = local[u] >= 0 ? base[bin[u] & (kCountTable - 1)] + local[u] : atomicAdd(&count[bin[u]], 1);
}

// Two-level exclusive scan of the bin counts: bins are (target row, column group), so one
// wavefront scans the bins of one target row (in place) and leaves the row total; a second
// tiny kernel scans the row totals.  Both are fully parallel (a single-block scan of all
// bins was latency-bound at over 100 us).
__global__ __launch_bounds__(64) void sort_rowscan_kernel(SortArgs S) {
    const int row = blockIdx.x, hd = blockIdx.y;
    if (!sort_useful(S) || (hd > 0 && *S.per_head == 0)) return;
    int *c = S.count + (size_t)hd * S.nbins + (size_t)row * S.bins_per_row;
    const int per = (S.bins_per_row + 63) / 64;
    const int lo = min((int)threadIdx.x * per, S.bins_per_row), hi = min(lo + per, S.bins_per_row);
    int s = 0;
    for (int i = lo; i < hi; ++i) s += c[i];
    int incl = s;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(incl, d, 64);
        if ((int)threadIdx.x >= d) incl += v;
    }
    int run = incl - s;
    for (int i = lo; i < hi; ++i) { const int v = c[i]; c[i] = run; run += v; }
    if (threadIdx.x == 63) S.rowtot[hd * S.nrows + row] = incl;
}

__global__ __launch_bounds__(1024) void sort_rowtot_scan_kernel(SortArgs S) {
    const int hd = blockIdx.x;
    if (!sort_useful(S) || (hd > 0 && *S.per_head == 0)) return;
    __shared__ int part[1024];
    int *c = S.rowtot + (size_t)hd * S.nrows;
    const int per = (S.nrows + 1023) / 1024;
    const int lo = min((int)threadIdx.x * per, S.nrows), hi = min(lo + per, S.nrows);
    int s = 0;
    for (int i = lo; i < hi; ++i) s += c[i];
    part[threadIdx.x] = s;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {          // Hillis-Steele inclusive scan of the partials
        const int v = (int)threadIdx.x >= d ? part[threadIdx.x - d] : 0;
        __syncthreads();
        part[threadIdx.x] += v;
        __syncthreads();
    }
    int run = part[threadIdx.x] - s;
    for (int i = lo; i < hi; ++i) { const int v = c[i]; c[i] = run; run += v; }
}

// Writes a complete permutation for every head, so that the forward kernel can follow
// perm[head][slot] without consulting any flag: the identity when the field is coherent, head
// 0's order for every head when the heads share their bins, each head's own order otherwise.
// With S.shared_perm the copies of head 0's order are left out.
__global__ __launch_bounds__(256) void sort_scatter_kernel(SortArgs S) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // head * L + pix
    // By the way, for the consumer that cuts the bins into chunks (one workgroup, which would otherwise fetch the
    // bounds of every bin once per head through one CU): the largest population of bin `idx` over the heads.
    // (per whole bin: the sub_h sub-bins of a tile together)
    if (S.pop && idx < S.nbins / S.sub_h && sort_useful(S) && *S.per_head) {
        const int tiles_per_row = S.bins_per_row / S.sub_h;
        const int row = idx / tiles_per_row, tx = idx - row * tiles_per_row;
        const int row_n = min(row + 1, S.nrows - 1);
        const int first = row * S.bins_per_row + tx * S.sub_h, first_n = min(first + S.sub_h, S.nbins - 1);
        int n = 0;
#pragma unroll 4
        for (int hd = 0; hd < S.h; ++hd) {
            const int row_start = S.rowtot[hd * S.nrows + row], next_row = S.rowtot[hd * S.nrows + row_n];
            const int start = S.count[hd * S.nbins + first], next = S.count[hd * S.nbins + first_n];
            const int lo = clampi(row_start + start, 0, S.L);
            const int hi = clampi(tx + 1 < tiles_per_row ? row_start + next : (row + 1 < S.nrows ? next_row : S.L), lo, S.L);
            n = max(n, hi - lo);
        }
        S.pop[idx] = n;
    }
    if (idx >= S.h * S.L) return;
    const int hd = idx / S.L, pix = idx - hd * S.L;
    if (!sort_useful(S)) {
        S.perm[idx] = pix;
        if (S.centre) {
            float x0, y0;
            load_xy(S.mo, S.dtype, (size_t)pix * S.h + hd, x0, y0);
            S.centre[idx] = pack_centre(x0, y0);
        }
        return;
    }
    const int src = *S.per_head ? hd : 0;                        // whose bins and ranks to use
    if (S.shared_perm && hd != src) return;                      // the consumer follows head 0's row
    float x, y;
    load_xy(S.mo, S.dtype, (size_t)pix * S.h + src, x, y);
    const int bin = target_bin(S, pix, x, y);
    const int start = S.rowtot[src * S.nrows + bin / S.bins_per_row] + S.count[src * S.nbins + bin];
    const int pos = min(max(start + S.rank[src * S.L + pix], 0), S.L - 1);
    S.perm[hd * S.L + pos] = pix;
    if (S.centre) S.centre[hd * S.L + pos] = pack_centre(x, y);
}

// Makes the order inside each bin independent of the arrival order of the counting atomics:
// one thread per bin sorts its (few) entries by pixel index.  With it, every consumer that
// walks a bin sums in a fixed order and the backward is bit-reproducible.  Bins with more than
// kMaxSortedBin entries (border bins collecting clamped centres) are ordered by the two kernels
// that follow instead, one thread per entry.
constexpr int kMaxSortedBin = 8;
// Bins beyond this size keep the arrival order (ordering them costs n reads per entry; such a bin means that
// thousands of queries sample one pixel, and the sums over it are then not bit-reproducible).
constexpr int kMaxRankedBin = 2048;
__global__ __launch_bounds__(256) void sort_bin_order_kernel(SortArgs S) {
    if (!sort_useful(S)) return;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // head * nbins + bin
    const int nh = *S.per_head ? S.h : 1;
    if (idx >= nh * S.nbins) return;
    const int hd = idx / S.nbins, bin = idx - hd * S.nbins;
    const bool last_in_row = (bin + 1) % S.bins_per_row == 0;
    const int lo_rel = S.count[idx];
    int n;
    const int row = bin / S.bins_per_row;
    const int base = S.rowtot[hd * S.nrows + row];
    if (!last_in_row) n = S.count[idx + 1] - lo_rel;
    else n = (row + 1 < S.nrows ? S.rowtot[hd * S.nrows + row + 1] : S.L) - base - lo_rel;
    const int lo = base + lo_rel;
    if (n < 2 || n > kMaxSortedBin || lo < 0 || lo + n > S.L) return;
    int *p = S.perm + (size_t)hd * S.L + lo;
    int *c = S.centre ? S.centre + (size_t)hd * S.L + lo : nullptr;
    if (n == 2) {                                   // by far the most common case
        const int a0 = p[0], a1 = p[1];
        if (a0 > a1) {
            p[0] = a1; p[1] = a0;
            if (c) { const int c0 = c[0], c1 = c[1]; c[0] = c1; c[1] = c0; }
        }
        return;
    }
    for (int a = 1; a < n; ++a) {                   // insertion sort, ascending pixel index
        const int v = p[a], cv = c ? c[a] : 0;
        int k = a - 1;
        while (k >= 0 && p[k] > v) { p[k + 1] = p[k]; if (c) c[k + 1] = c[k]; --k; }
        p[k + 1] = v;
        if (c) c[k + 1] = cv;
    }
}


// [lo, lo + n) of the bin the entry at `pos` of head `hd`'s order lies in (from the pixel stored there).
__device__ __forceinline__ void bin_of_entry(const SortArgs &S, int hd, int pix, int &lo, int &n) {
    float x, y;
    load_xy(S.mo, S.dtype, (size_t)pix * S.h + hd, x, y);
    const int bin = target_bin(S, pix, x, y);
    const int row = bin / S.bins_per_row;
    const int base = S.rowtot[hd * S.nrows + row];
    const int rel = S.count[hd * S.nbins + bin];
    const bool last_in_row = (bin + 1) % S.bins_per_row == 0;
    const int end = last_in_row ? (row + 1 < S.nrows ? S.rowtot[hd * S.nrows + row + 1] : S.L)
                                : base + S.count[hd * S.nbins + bin + 1];
    lo = min(max(base + rel, 0), S.L);
    n = min(max(end - lo, 0), S.L - lo);
}

// Large bins, step 1: every entry of a bin with more than kMaxSortedBin entries counts the entries of its bin
// with a smaller pixel index -- its final place -- and writes itself there in `rank` (free after the scatter).
__global__ __launch_bounds__(256) void sort_big_bins_rank_kernel(SortArgs S) {
    if (!sort_useful(S)) return;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // head * L + position
    const int nh = *S.per_head ? S.h : 1;
    if (idx >= nh * S.L) return;
    const int hd = idx / S.L, pos = idx - hd * S.L;
    const int *p = S.perm + (size_t)hd * S.L;
    const int mine = min(max(p[pos], 0), S.L - 1);
    int lo, n;
    bin_of_entry(S, hd, mine, lo, n);
    if (n <= kMaxSortedBin || n > kMaxRankedBin || pos < lo || pos >= lo + n) return;
    int r = 0;
    for (int j = 0; j < n; ++j) r += p[lo + j] < mine ? 1 : 0;
    S.rank[(size_t)hd * S.L + lo + min(r, n - 1)] = mine;
}

// Large bins, step 2: the ordered entries go back into the order of every head that uses it, with their
// centres.  A thread finds its bin from the entry at its own position, which may already be the reordered
// one when the head shares head 0's order -- another pixel of the same bin, so the bounds are the same.
__global__ __launch_bounds__(256) void sort_big_bins_store_kernel(SortArgs S) {
    if (!sort_useful(S)) return;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // head * L + position
    if (idx >= S.h * S.L) return;
    const int hd = idx / S.L, pos = idx - hd * S.L;
    const int src = *S.per_head ? hd : 0;
    const int cur = min(max(S.perm[(size_t)src * S.L + pos], 0), S.L - 1);
    int lo, n;
    bin_of_entry(S, src, cur, lo, n);
    if (n <= kMaxSortedBin || n > kMaxRankedBin || pos < lo || pos >= lo + n) return;
    const int v = min(max(S.rank[(size_t)src * S.L + pos], 0), S.L - 1);
    S.perm[idx] = v;
    if (S.centre) {
        float x, y;
        load_xy(S.mo, S.dtype, (size_t)v * S.h + src, x, y);
        S.centre[idx] = pack_centre(x, y);
    }
}

// Small maps: the exact inverse index (bins of one pixel, entries of a bin in ascending pixel order, centres) of one
// image and head from ONE workgroup, in place of the count, scan, scatter and ordering kernels above -- at a few
// thousand pixels each of those is a launch that lasts longer than its work.  The workgroup counts the image's bins
// in LDS, scans them there, places the entries (in arrival order) in an LDS copy of the order, and every entry then
// finds its final place by counting the entries of its bin with a smaller pixel index: the result does not depend on
// the order of the atomics.  Bins with more than kMaxRankedBin entries keep the arrival order, as above.
// Grid (batch items, heads); the workgroups of heads 1.. leave when the heads share head 0's index (the probe has
// run).  Writes count, rowtot, perm and centre exactly as the kernels above leave them (rank is not used).
// (Letting every workgroup do the probe's work itself -- read all positions of the call, so that all come to the same
// answer without exchanging a word -- saves the zeroing and the probe launches, but one CU reads the positions at a
// fraction of the chip's rate: measured equal at 2 x 48 x 48 x 4 heads, 12 us slower at 2 x 96 x 96 x 4.  And the
// limit is where one CU stops being faster than seven launches over the whole chip: a variant for images of up to
// 40 448 pixels -- 16-bit counters, two per LDS word, the positions read three times -- took 90 us at 2 x 192 x 192
// where the kernels above take 43.)
constexpr int kSmallSortMaxN = 16384, kSmallSortThreads = 1024;
template <int DT>
__global__ __launch_bounds__(kSmallSortThreads) void sort_small_kernel(SortArgs S) {
    __shared__ int tab[kSmallSortMaxN];              // bin counts, then bin starts
    __shared__ uint16_t order[kSmallSortMaxN];       // pixel (within the image) at each position, arrival order
    __shared__ int wave_tot[kSmallSortThreads / 64];
    const int b = blockIdx.x, hd = blockIdx.y, N = S.N, tid = threadIdx.x;
    if (hd > 0 && *S.per_head == 0) return;          // uniform over the workgroup
    constexpr int PER = kSmallSortMaxN / kSmallSortThreads;
    for (int i = tid; i < N; i += kSmallSortThreads) tab[i] = 0;
    float x[PER], y[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int p = min(tid + u * kSmallSortThreads, N - 1);
        load_xy_as<DT>(S.mo, ((size_t)b * N + p) * S.h + hd, x[u], y[u]);
    }
    __syncthreads();
    int bin[PER], arrival[PER], ctr[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const uint32_t cell = target_cell(S, x[u], y[u]);        // bins of one pixel: (row << 16) | column
        bin[u] = (int)(cell >> 16) * S.W + (int)(cell & 0xffffu);
        ctr[u] = pack_centre(x[u], y[u]);
        arrival[u] = tid + u * kSmallSortThreads < N ? atomicAdd(&tab[bin[u]], 1) : 0;
    }
    __syncthreads();
    // exclusive scan of the counts, in place: a run of bins per thread, the runs' totals over the wavefront and the
    // wavefronts' totals through LDS
    {
        const int per = (N + kSmallSortThreads - 1) / kSmallSortThreads;
        const int lo = min(tid * per, N), hi = min(lo + per, N);
        int s = 0;
        for (int i = lo; i < hi; ++i) s += tab[i];
        int incl = s;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int v = __shfl_up(incl, d, 64);
            if ((tid & 63) >= d) incl += v;
        }
        if ((tid & 63) == 63) wave_tot[tid >> 6] = incl;
        __syncthreads();
        int run = incl - s;
        for (int w = 0; w < (tid >> 6); ++w) run += wave_tot[w];
        for (int i = lo; i < hi; ++i) { const int v = tab[i]; tab[i] = run; run += v; }
    }
    __syncthreads();
    int *const count = S.count + (size_t)hd * S.nbins + (size_t)b * N;
    for (int i = tid; i < N; i += kSmallSortThreads) {
        const int row = i / S.W;
        count[i] = tab[i] - tab[row * S.W];
        if (i == row * S.W) S.rowtot[hd * S.nrows + b * S.H + row] = b * N + tab[i];
    }
#pragma unroll
    for (int u = 0; u < PER; ++u)
        if (tid + u * kSmallSortThreads < N) order[tab[bin[u]] + arrival[u]] = (uint16_t)(tid + u * kSmallSortThreads);
    __syncthreads();
    int *const perm = S.perm + (size_t)hd * S.L + (size_t)b * N;
    int *const centre = S.centre ? S.centre + (size_t)hd * S.L + (size_t)b * N : nullptr;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
        const int p = tid + u * kSmallSortThreads;
        if (p >= N) continue;
        const int lo = tab[bin[u]], n = (bin[u] + 1 < N ? tab[bin[u] + 1] : N) - lo;
        int r = arrival[u];
        if (n > 1 && n <= kMaxRankedBin) {
            r = 0;
            for (int j = 0; j < n; ++j) r += (int)order[lo + j] < p ? 1 : 0;
        }
        perm[lo + r] = b * N + p;
        if (centre) centre[lo + r] = ctr[u];
    }
}

}  // namespace ma

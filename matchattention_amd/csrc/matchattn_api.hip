// C ABI of libmatchattn_hip.so: argument checks, kernel selection, launches.
// Declarations and the reference interfaces they replace: include/matchattn_hip.h.
#include "../../include/matchattn_hip.h"

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <vector>
#include <atomic>

#include "matchattn_bwd.h"
#include "matchattn_launch.h"
#include "matchattn_sort.h"

namespace ma {

// ---- helpers around the scatter: zero the accumulators, narrow them to the output dtype ------
// (a fill kernel rather than hipMemsetAsync so that callers may capture the call in a HIP graph)
__global__ __launch_bounds__(256) void fill_zero_kernel(float *p, size_t n) {
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nth = (size_t)gridDim.x * blockDim.x;
    if ((reinterpret_cast<uintptr_t>(p) & 15u) == 0) {
        const size_t n4 = n >> 2;
        for (size_t i = tid; i < n4; i += nth) ((u32x4 *)p)[i] = u32x4{0, 0, 0, 0};
        for (size_t i = (n4 << 2) + tid; i < n; i += nth) p[i] = 0.f;
    } else {
        for (size_t i = tid; i < n; i += nth) p[i] = 0.f;
    }
}

// dst0 = T(src0), dst1 = T(src1), n elements each (16-bit T).
template <typename T>
__global__ __launch_bounds__(256) void narrow_kernel(const float *src0, const float *src1, T *dst0, T *dst1, size_t n) {
    const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x, nth = (size_t)gridDim.x * blockDim.x;
    const bool aligned = ((reinterpret_cast<uintptr_t>(src0) | reinterpret_cast<uintptr_t>(src1)) & 15u) == 0 &&
                         ((reinterpret_cast<uintptr_t>(dst0) | reinterpret_cast<uintptr_t>(dst1)) & 7u) == 0;
    const size_t n4 = aligned ? (n >> 2) : 0;
    for (size_t i = tid; i < n4; i += nth) {
        const float4 a = ((const float4 *)src0)[i], c = ((const float4 *)src1)[i];
        T ta[4] = {Traits<T>::from_f(a.x), Traits<T>::from_f(a.y), Traits<T>::from_f(a.z), Traits<T>::from_f(a.w)};
        T tc[4] = {Traits<T>::from_f(c.x), Traits<T>::from_f(c.y), Traits<T>::from_f(c.z), Traits<T>::from_f(c.w)};
        ((u32x2 *)dst0)[i] = __builtin_bit_cast(u32x2, ta);
        ((u32x2 *)dst1)[i] = __builtin_bit_cast(u32x2, tc);
    }
    for (size_t i = (n4 << 2) + tid; i < n; i += nth) {
        dst0[i] = Traits<T>::from_f(src0[i]);
        dst1[i] = Traits<T>::from_f(src1[i]);
    }
}

// Sampling positions from relative ones, in one pass: what the attention layer and module do with four
// elementwise launches before the operator (models/attention_blocks.py:149-151 or 162-163: the pixel's own
// coordinates, in the tensor dtype, are added; :45-59, :79: clamp to [r, size-1-r-1e-3] with bounds rounded
// to the tensor dtype).  rel is [L][rel_heads][2] with rel_heads == h, or 1 for a position every head shares.
template <typename T>
__global__ __launch_bounds__(256) void make_offsets_kernel(const T *rel, T *mo, int nhq, int h, int rel_heads, int W, int N,
                                                           float lo_x, float hi_x, float lo_y, float hi_y) {
    typedef Traits<T> Tr;
    const long long gid = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= nhq) return;
    const int hq = (int)gid, pix = hq / h, head = hq - pix * h;
    const int n = pix % N, py = n / W, px = n - py * W;
    const T *r = rel + ((size_t)pix * rel_heads + (rel_heads == 1 ? 0 : head)) * 2;
    // (coordinates beyond the dtype's exact integers round as torch.arange in that dtype does)
    const float x = Tr::round(Tr::to_f(r[0]) + Tr::round((float)px)), y = Tr::round(Tr::to_f(r[1]) + Tr::round((float)py));
    const float cx = x != x ? x : fminf(fmaxf(x, Tr::round(lo_x)), Tr::round(hi_x));      // torch.clamp keeps NaN
    const float cy = y != y ? y : fminf(fmaxf(y, Tr::round(lo_y)), Tr::round(hi_y));
    mo[(size_t)hq * 2] = Tr::from_f(cx);
    mo[(size_t)hq * 2 + 1] = Tr::from_f(cy);
}

KernelTimer g_fwd_timer = {{false}, nullptr, nullptr};

unsigned tile_grid(unsigned per_cu) {
    static std::atomic<int> cus[64];                   // compute units per device index, 0 = not asked yet
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 64) n = cus[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        if (dev >= 0 && dev < 64) cus[dev].store(n, std::memory_order_relaxed);
    }
    return (((unsigned)n * per_cu + 7u) / 8u) * 8u;
}

}  // namespace ma

namespace {

thread_local char g_err[512] = "";
// names of the last kernels launched (process-wide: autograd calls backward on another thread)
std::atomic<const char *> g_last_fwd{""};
std::atomic<const char *> g_last_bwd{""};
std::atomic<int> g_forward_variant{-1};
std::atomic<int> g_row_skip{1};
std::atomic<int> g_xcd_swizzle{1};
std::atomic<int> g_forward_lds{-1};
std::atomic<int> g_backward_mode{-1};    // -1 auto (gather when possible), 0 scatter (atomics), 1 gather, 2 gather with the direct pass A

// The options as one entry point sees them: read once per call, so that a matchattn_set_option on another thread
// cannot make the workspace size a call checks differ from the one its kernels use.
struct Options {
    int forward_variant, row_skip, xcd_swizzle, forward_lds, backward_mode;
};
Options options_now() {
    return Options{g_forward_variant.load(), g_row_skip.load(), g_xcd_swizzle.load(), g_forward_lds.load(), g_backward_mode.load()};
}

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

size_t elem_size(int dtype) { return dtype == MATCHATTN_F32 ? 4 : 2; }

int check_common(const char *fn, int B, int H, int W, int C, int h, int rx, int ry, int dtype) {
    if (dtype != MATCHATTN_F32 && dtype != MATCHATTN_F16 && dtype != MATCHATTN_BF16)
        return fail(MATCHATTN_ERR_ARG, "%s: unknown dtype %d (0 f32, 1 f16, 2 bf16)", fn, dtype);
    if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || h <= 0)
        return fail(MATCHATTN_ERR_ARG, "%s: B, H, W, C, h must be positive (got %d %d %d %d %d)", fn, B, H, W, C, h);
    if (C % h) return fail(MATCHATTN_ERR_ARG, "%s: C=%d is not a multiple of h=%d", fn, C, h);
    if (rx != ry)
        return fail(MATCHATTN_ERR_ARG, "%s: only square windows are defined (win_r = [%d, %d])", fn, rx, ry);
    if (rx < 1 || rx > ma::kMaxR)
        return fail(MATCHATTN_ERR_ARG, "%s: window radius %d outside 1..%d", fn, rx, ma::kMaxR);
    if (2 * rx + 2 > W || 2 * ry + 2 > H)   // models/attention_blocks.py:64
        return fail(MATCHATTN_ERR_ARG, "%s: window %dx%d does not fit the %dx%d map", fn, 2 * rx + 2, 2 * ry + 2, W, H);
    if (H > 29000 || W > 29000)             // window centres are bounded to +-30000 before any index arithmetic
        return fail(MATCHATTN_ERR_ARG, "%s: maps beyond 29000 pixels a side are not supported (got %dx%d)", fn, H, W);
    const long long nhq = (long long)B * H * W * h;
    if (nhq >= (1ll << 31)) return fail(MATCHATTN_ERR_ARG, "%s: B*H*W*h = %lld exceeds 2^31-1", fn, nhq);
    return 0;
}

// The tiled kernels address K/V with 32-bit byte offsets through buffer descriptors and
// need whole 16-byte vectors per head.
bool tiled_ok(const void *const *ptrs, int nptr, long long L, int C, int CH, int dtype) {
    const size_t es = elem_size(dtype);
    if ((CH * es) % 16) return false;
    if ((unsigned long long)L * C * es >= 0xFFFFFF00ull) return false;
    for (int i = 0; i < nptr; ++i)
        if (reinterpret_cast<uintptr_t>(ptrs[i]) & 15u) return false;
    return true;
}

bool bwd_tiled_shape(int CH, int rx, int dtype) {
    if (rx > 2) return false;
    const int f16set[] = {8, 16, 32, 40, 64, 80, 96, 128, 192}, f32set[] = {8, 16, 32, 40, 64, 80, 96, 128, 192};
    if (dtype == MATCHATTN_F32) { for (int c : f32set) if (c == CH) return true; return false; }
    for (int c : f16set) if (c == CH) return true;
    return false;
}

}  // namespace

extern "C" {

int matchattn_abi_version(void) { return 4; }

const char *matchattn_last_error(void) { return g_err; }

const char *matchattn_last_forward_kernel(void) { return g_last_fwd.load(); }

const char *matchattn_last_backward_kernel(void) { return g_last_bwd.load(); }

int matchattn_set_option(const char *name, int value) {
    if (!name) return fail(MATCHATTN_ERR_ARG, "matchattn_set_option: null name");
    if (!strcmp(name, "forward_variant")) {
        if (value != -1 && value != 0 && value != 1 && value != 2)
            return fail(MATCHATTN_ERR_ARG, "matchattn_set_option: forward_variant must be -1, 0, 1 or 2");
        g_forward_variant = value;
        return 0;
    }
    if (!strcmp(name, "stereo_row_skip")) { g_row_skip = value ? 1 : 0; return 0; }
    if (!strcmp(name, "xcd_swizzle")) { g_xcd_swizzle = value ? 1 : 0; return 0; }
    if (!strcmp(name, "forward_lds")) { g_forward_lds = value < 0 ? -1 : (value ? 1 : 0); return 0; }
    if (!strcmp(name, "backward_mode")) {
        if (value < -1 || value > 2) return fail(MATCHATTN_ERR_ARG, "matchattn_set_option: backward_mode must be -1, 0, 1 or 2");
        g_backward_mode = value;
        return 0;
    }
    if (!strcmp(name, "time_kernels")) {
        if (value && !ma::g_fwd_timer.before) {
            if (hipEventCreate(&ma::g_fwd_timer.before) != hipSuccess || hipEventCreate(&ma::g_fwd_timer.after) != hipSuccess)
                return fail(MATCHATTN_ERR_LAUNCH, "matchattn_set_option: time_kernels: cannot create events");
        }
        ma::g_fwd_timer.on = value != 0;
        return 0;
    }
    return fail(MATCHATTN_ERR_ARG, "matchattn_set_option: unknown option '%s'", name);
}

namespace {
struct SortLayout { size_t count_off, rowtot_off, rank_off, perm_off, flag_off, total; int nbins, bins_per_row, nrows, rows_per_img; };
SortLayout sort_layout(int B, int H, int W, int h, int bin_w, int bin_h = 1, int sub_h = 1) {
    SortLayout s;
    s.bins_per_row = (W + bin_w - 1) / bin_w * sub_h;
    s.rows_per_img = (H + bin_h - 1) / bin_h;
    s.nrows = B * s.rows_per_img;
    s.nbins = s.nrows * s.bins_per_row;
    const size_t L = (size_t)B * H * W;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    s.flag_off = 0;                                   // flag + counters are zeroed together
    s.count_off = 256;
    s.rowtot_off = s.count_off + up((size_t)h * s.nbins * 4);
    s.rank_off = s.rowtot_off + up((size_t)h * s.nrows * 4);
    s.perm_off = s.rank_off + up(L * h * 4);
    s.total = s.perm_off + up(L * h * 4);
    return s;
}
// LDS-tile forward: buckets of the tile sort, then one flag byte per head-query (left for the generic kernel).
struct TileLayout { SortLayout sl; size_t defer_off, chunk_off, item_off, total; int chunk_cap; };
// `by_row`: the buckets are ordered by the window's row inside the tile (one sub-bucket per row), which the fp16
// forward with 32 channels per head wants: its aggregation walks the rows the 16 queries of a wavefront reach.
bool tile_rows_wanted(int C, int h, int rx, int dtype) {
    // (64 channels with the 6x6 window: as two half-heads of 32 on the same kernel)
    return (dtype == MATCHATTN_F16 || dtype == MATCHATTN_BF16) && (C / h == 32 || (C / h == 64 && rx == 2));
}
TileLayout tile_layout(int B, int H, int W, int h, bool by_row) {
    TileLayout t;
    const int sub = by_row ? ma::kTileDims[1] : 1;
    t.sl = sort_layout(B, H, W, h, ma::kTileDims[0], ma::kTileDims[1], sub);
    t.defer_off = t.sl.total;
    t.chunk_off = t.defer_off + (((size_t)B * H * W * h + 255) & ~(size_t)255);   // one flag byte per head-query
    const int ntiles = t.sl.nbins / sub;
    t.item_off = t.chunk_off + (((size_t)(ntiles + 1) * 4 + 255) & ~(size_t)255);
    // a bucket has ceil(max over heads of its population / cap) chunks: at most nbins + h * L / cap in all
    t.chunk_cap = (int)std::min<size_t>((size_t)ntiles + (size_t)B * H * W * h / ma::kTileCapHost + 1, (size_t)1 << 30);
    t.total = t.item_off + (((size_t)t.chunk_cap * 8 + 255) & ~(size_t)255);
    return t;
}
// The counting sort of the queries on their target bucket (matchattn_sort.h): the kernels in stream order.
// `shared_known`: the caller states that all heads of a pixel have the same sampling position (and the ordering is
// not optional, S.force): the probe that would find that out, and the per-head counts, are not launched -- the
// zeroed flags already say "shared".
void launch_sort(const ma::SortArgs &S, const SortLayout &sl, long long L, int h, char *ws, bool bin_order, hipStream_t s,
                 bool shared_known = false) {
    // Small maps, exact index: one workgroup per image and head builds it whole (the counters need no zeroing then)
    const bool small = bin_order && S.force && S.bin_w == 1 && S.bin_h == 1 && S.sub_h == 1 && !S.pop && !S.shared_perm &&
                       S.N <= ma::kSmallSortMaxN && S.W < 65536 && S.H < 65536;
    const size_t nzero = small ? (size_t)ma::kFlagWords : sl.rowtot_off / 4;            // flags (+ counters)
    const size_t zb = nzero / 4 / 256 + 1;
    shared_known = (shared_known && S.force) || (small && h == 1);
    hipLaunchKernelGGL(ma::fill_zero_kernel, dim3((unsigned)(zb < 8192 ? zb : 8192)), dim3(256), 0, s, (float *)ws, nzero);
    if (!shared_known) {
        const dim3 pg((unsigned)std::min<long long>((L * h + 255) / 256, ma::kProbeBlocks));
        if (S.dtype == MATCHATTN_F32) hipLaunchKernelGGL(ma::sort_probe_kernel<0>, pg, dim3(256), 0, s, S);
        else if (S.dtype == MATCHATTN_F16) hipLaunchKernelGGL(ma::sort_probe_kernel<1>, pg, dim3(256), 0, s, S);
        else hipLaunchKernelGGL(ma::sort_probe_kernel<2>, pg, dim3(256), 0, s, S);
    }
    if (small) {
        const dim3 g((unsigned)(L / S.N), (unsigned)h), t(ma::kSmallSortThreads);
        if (S.dtype == MATCHATTN_F32) hipLaunchKernelGGL(ma::sort_small_kernel<0>, g, t, 0, s, S);
        else if (S.dtype == MATCHATTN_F16) hipLaunchKernelGGL(ma::sort_small_kernel<1>, g, t, 0, s, S);
        else hipLaunchKernelGGL(ma::sort_small_kernel<2>, g, t, 0, s, S);
        return;
    }
    // (grid.x a multiple of the 8 XCDs, workgroup ids being dealt to them round-robin: the workgroups that count the
    // same pixels for the other heads -- one grid row each -- then run on the same XCD and find the lines of positions,
    // which hold all heads of a pixel side by side, in its L2; the workgroups past the map leave at once)
    const unsigned count_blocks = (unsigned)((L + 256 * ma::kCountPerThread - 1) / (256 * ma::kCountPerThread));
    hipLaunchKernelGGL(ma::sort_count_kernel, dim3((count_blocks + 7u) / 8u * 8u, (unsigned)(shared_known ? 1 : h)),
                       dim3(256), 0, s, S);
    hipLaunchKernelGGL(ma::sort_rowscan_kernel, dim3((unsigned)sl.nrows, (unsigned)h), dim3(64), 0, s, S);
    hipLaunchKernelGGL(ma::sort_rowtot_scan_kernel, dim3((unsigned)h), dim3(1024), 0, s, S);
    hipLaunchKernelGGL(ma::sort_scatter_kernel, dim3((unsigned)(((long long)h * L + 255) / 256)), dim3(256), 0, s, S);
    if (bin_order) {
        hipLaunchKernelGGL(ma::sort_bin_order_kernel, dim3((unsigned)(((long long)h * sl.nbins + 255) / 256)), dim3(256), 0, s, S);
        hipLaunchKernelGGL(ma::sort_big_bins_rank_kernel, dim3((unsigned)(((long long)h * L + 255) / 256)), dim3(256), 0, s, S);
        hipLaunchKernelGGL(ma::sort_big_bins_store_kernel, dim3((unsigned)(((long long)h * L + 255) / 256)), dim3(256), 0, s, S);
    }
}

// Sort arguments over a workspace laid out by sort_layout at `ws`.
ma::SortArgs sort_args(const void *max_offset, int dtype, int B, int H, int W, int h, const SortLayout &sl, char *ws,
                       int bin_w, int bin_h, int force) {
    ma::SortArgs S;
    S.mo = max_offset; S.dtype = dtype; S.L = B * H * W; S.N = H * W; S.H = H; S.W = W; S.h = h;
    S.bin_w = bin_w; S.bin_h = bin_h; S.sub_h = sl.bins_per_row / ((W + bin_w - 1) / bin_w); S.rows_per_img = sl.rows_per_img; S.force = force; S.centre = nullptr;
    S.shared_perm = 0; S.pop = nullptr;
    S.bins_per_row = sl.bins_per_row; S.nbins = sl.nbins; S.nrows = sl.nrows;
    S.rowtot = (int *)(ws + sl.rowtot_off); S.per_head = (int *)(ws + sl.flag_off); S.count = (int *)(ws + sl.count_off);
    S.rank = (int *)(ws + sl.rank_off); S.perm = (int *)(ws + sl.perm_off);
    return S;
}

// Tile buckets + work list for the LDS-tile kernels, over a workspace laid out by tile_layout at `ws`.
ma::TileSort tile_sort_args(const ma::SortArgs &S, const TileLayout &tl, char *ws) {
    ma::TileSort T;
    T.count = S.count; T.rowtot = S.rowtot; T.per_head = S.per_head; T.perm = S.perm;
    T.defer = (uint8_t *)(ws + tl.defer_off); T.chunk_start = (int *)(ws + tl.chunk_off);
    T.chunk_item = (int2 *)(ws + tl.item_off); T.chunk_cap = tl.chunk_cap;
    T.queue = S.per_head + ma::kFlagQueue;             // inside the 256-byte flag block the sort zeroes
    T.xcd_bounds = S.per_head + ma::kFlagXcdBounds;
    T.sub = S.sub_h;
    T.bins_per_row = tl.sl.bins_per_row / T.sub; T.nbins = tl.sl.nbins / T.sub; T.nrows = tl.sl.nrows; T.rows_per_img = tl.sl.rows_per_img;
    T.L = S.L;
    return T;
}

// Whether the forward would use the LDS-tile kernel for these sizes (it needs the workspace).
bool tile_wanted(const Options &O, int B, int H, int W, int C, int h, int rx, int ry, int dtype) {
    const int CH = C / h, mode = O.forward_lds;
    if (mode == 0 || rx != ry || rx > 2 || O.forward_variant == 0) return false;
    // head sizes with an instance (a head group is the heads that fill a 128-byte line per pixel; 64 fp32
    // channels are 256-byte pixels: one workgroup of 512 threads per CU instead of two of 256)
    const int head_bytes = CH * (int)elem_size(dtype);
    if (!(CH == 16 || CH == 32 || CH == 64)) return false;
    if (h % (head_bytes >= 128 ? 1 : 128 / head_bytes) != 0) return false;
    if (mode == 1) return true;
    // auto: the sizes from which the tiles win.  Measured against the direct gather in one process on five fields per
    // size -- i.i.d. stereo (x - U(0, W/4), y exact), i.i.d. per-head 2-D (sigma 8), and three smooth ones as a model
    // produces them (blurred stereo, a synthetic scene's disparity, blurred per-head) -- with 4 and 8 heads, 2^18 to
    // 2^22 head-queries; the limit is where the geometric mean over the five crosses 1.  The smooth fields decide it:
    // their gathers hit L1 and L2 and the direct kernel needs no bucketing, so the tiles win later than on the i.i.d.
    // fields (and on the i.i.d. 2-D field they win 1.2x to 2x already one step below every limit given here).
    //   fp16, 32 channels per head (the kernel with the matrix-unit phases):
    //     6x6 window: 0.71x to 1.29x at 2^19, 1.16x to 2.1x at 2^20, 1.28x to 2.7x at 2^21, 1.43x to 3.2x at 2^22
    //     4x4 window: 0.68x to 1.36x at 2^20, 0.77x to 1.78x at 2^21 (mean 1.0), 0.87x to 2.2x at 2^22
    //   fp16, 64 channels: 6x6 0.73x to 0.88x at 2^18, 1.13x to 1.50x at 2^19; 4x4 0.78x to 1.13x at 2^19, 0.89x to
    //     1.56x at 2^20;  16 channels: 6x6 0.66x to 1.94x at 2^20 (mean 0.86), 1.05x to 3.0x at 2^21; 4x4 not below 2^21
    //   bf16, 32 channels: 6x6 0.78x to 1.48x at 2^19 (mean 0.95), 1.05x to 2.45x at 2^20; 4x4 0.73x to 1.9x at 2^20,
    //     0.86x to 2.2x at 2^21 (mean 1.07);  64 channels: 6x6 0.89x to 1.04x at 2^18, 1.15x to 1.66x at 2^19; 4x4 and
    //     16 channels: only the i.i.d. 2-D field wins below 2^21 (6x6 from 2^21, 4x4 not by default)
    //   fp32 (whose direct kernel moves twice the bytes through L2), 16 and 32 channels: 6x6 0.61x to 1.24x at 2^18,
    //     0.84x to 2.1x at 2^19 (mean 1.03 and 1.4); 4x4 32 channels 0.79x to 1.46x at 2^19, 0.91x to 2.1x at 2^20, 16
    //     channels 0.80x to 1.31x at 2^20, 0.95x to 2.5x at 2^21;  64 channels (one workgroup of 512 threads per CU):
    //     6x6 1.3x to 2.3x at 2^18, 4x4 0.88x to 1.62x at 2^18 (mean 1.03), 1.01x to 2.4x at 2^19
    const long long nhq = (long long)B * H * W * h, k19 = 1ll << 19, k20 = 1ll << 20, k21 = 1ll << 21;
    if (dtype == MATCHATTN_F32) {
        if (CH == 64) return nhq >= (rx == 2 ? (1ll << 17) : (1ll << 18));
        if (rx == 2) return nhq >= k19;
        return nhq >= (CH == 32 ? k20 : k20 + k19);
    }
    if (dtype == MATCHATTN_F16) {
        if (CH == 64) return nhq >= (rx == 2 ? k19 : k20);
        if (CH == 32) return nhq >= (rx == 2 ? k20 : k21);
        return nhq >= (rx == 2 ? k20 + k19 : k21);
    }
    if (CH == 32) return nhq >= (rx == 2 ? k20 : k21);
    if (CH == 64) return rx == 2 && nhq >= k19;            // (as two half-heads of 32 on the same kernel: 1.15x to 1.66x at 2^19)
    return rx == 2 && nhq >= k21;
}
}  // namespace

namespace {
size_t forward_workspace_bytes(const Options &O, int B, int H, int W, int C, int h, int rx, int ry, int dtype) {
    if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || h <= 0) return 0;
    return tile_wanted(O, B, H, W, C, h, rx, ry, dtype) ? tile_layout(B, H, W, h, tile_rows_wanted(C, h, rx, dtype)).total : 0;
}
}  // namespace

size_t matchattn_forward_workspace_bytes(int B, int H, int W, int C, int h, int rx, int ry, int dtype) {
    return forward_workspace_bytes(options_now(), B, H, W, C, h, rx, ry, dtype);
}

namespace {
// Where the forward puts its results: row strides in elements (0: contiguous) and the optional gate.
struct Placement {
    long long out_stride = 0, attn_stride = 0;
    const void *gate = nullptr;
    bool shared_offsets = false;    // every head of a pixel is known to have the same sampling position
    // `max_offset` holds positions relative to the query pixels, [B,N,rel_heads,2] (0: the sampling positions
    // themselves); set only for calls that take a kernel which adds the pixel grid and clamps in its own prologue
    int rel_heads = 0;
};

int forward_impl(const Options &O, const void *max_offset, const void *q, const void *k, const void *v, void *out, void *attn,
                 const Placement &P, void *workspace, size_t workspace_bytes,
                 int B, int H, int W, int C, int h, int rx, int ry, float scale, int dtype, void *stream) {
    if (!max_offset || !q || !k || !v || !out || !attn)
        return fail(MATCHATTN_ERR_ARG, "matchattn_forward: null tensor pointer");
    hipStream_t s = (hipStream_t)stream;
    const long long L = (long long)B * H * W;
    const int CH = C / h;
    const long long M = (long long)(2 * rx + 2) * (2 * ry + 2), es = (long long)elem_size(dtype);
    const long long out_stride = P.out_stride ? P.out_stride : C, attn_stride = P.attn_stride ? P.attn_stride : h * M;
    if (out_stride < C || attn_stride < h * M)
        return fail(MATCHATTN_ERR_ARG, "matchattn_forward: row strides %lld, %lld are shorter than the rows (%d, %lld)",
                    out_stride, attn_stride, C, h * M);
    if (out_stride * es >= (1ll << 31) || attn_stride * es >= (1ll << 31))
        return fail(MATCHATTN_ERR_ARG, "matchattn_forward: row strides of 2 GiB or more are not supported");
    // (the tiled kernels address the outputs with 32-bit byte offsets)
    const bool small_views = (L - 1) * out_stride * es + C * es < 0xFFFFFF00ll && (L - 1) * attn_stride * es + h * M * es < 0xFFFFFF00ll;
    ma::FwdArgs A;
    A.mo = max_offset; A.q = q; A.k = k; A.v = v; A.out = out; A.attn = attn;
    A.nhq = (int)(L * h); A.N = H * W; A.H = H; A.W = W; A.C = C; A.h = h;
    A.h_log2 = (h & (h - 1)) == 0 ? __builtin_ctz((unsigned)h) : -1;
    A.scale = scale; A.row_skip = O.row_skip; A.xcd_swizzle = O.xcd_swizzle;
    A.defer = nullptr;
    A.out_row_bytes = (uint32_t)(out_stride * es); A.attn_row_bytes = (uint32_t)(attn_stride * es); A.gate = P.gate;
    A.rel_heads = P.rel_heads;
    A.lo_x = (float)rx; A.hi_x = (float)((double)(W - 1 - rx) - 1e-3); A.lo_y = (float)ry; A.hi_y = (float)((double)(H - 1 - ry) - 1e-3);

    const int variant = O.forward_variant;
    const char *kname = "";
    const void *ptrs[] = {q, k, v, out, P.gate, attn, max_offset};      // (a null gate is aligned)
    int rc = -1;
    if (variant != 0 && rx <= 2 && tiled_ok(ptrs, 5, L, C, CH, dtype) &&
        (reinterpret_cast<uintptr_t>(attn) & 7u) == 0 && A.out_row_bytes % 16 == 0 && A.attn_row_bytes % 8 == 0 && small_views) {
        const int vpl = variant > 0 ? variant : 1;      // vectors per lane of the direct kernels
        // LDS-tile path: bucket the queries by K/V tile, one workgroup per tile and head group, then the
        // generic kernel for the (normally empty) list of queries a tile could not serve
        if (workspace && P.rel_heads == 0 && tile_wanted(O, B, H, W, C, h, rx, ry, dtype) && (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0) {
            const TileLayout tl = tile_layout(B, H, W, h, tile_rows_wanted(C, h, rx, dtype));
            const SortLayout &sl = tl.sl;
            if (workspace_bytes < tl.total)
                return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_forward_ws: workspace of %zu bytes needed, %zu given",
                            tl.total, workspace_bytes);
            char *ws = (char *)workspace;
            ma::SortArgs S = sort_args(max_offset, dtype, B, H, W, h, sl, ws, ma::kTileDims[0], ma::kTileDims[1], 1);
            S.shared_perm = 1;
            S.pop = (int *)(ws + tl.chunk_off);          // (the work list's own array: populations first, chunk starts later)
            launch_sort(S, sl, L, h, ws, false, s, P.shared_offsets);
            if (hipError_t e = hipGetLastError())
                return fail(MATCHATTN_ERR_LAUNCH, "matchattn_forward_ws: sort launch failed: %s", hipGetErrorString(e));
            const ma::TileSort T = tile_sort_args(S, tl, ws);
            uint8_t *defer = T.defer;
            switch (dtype) {
            case MATCHATTN_F32: rc = ma::launch_fwd_tile_f32(A, T, CH, rx, s, &kname); break;
            case MATCHATTN_F16: rc = ma::launch_fwd_tile_f16(A, T, CH, rx, s, &kname); break;
            default: rc = ma::launch_fwd_tile_bf16(A, T, CH, rx, s, &kname); break;
            }
            if (rc == 0) {
                ma::FwdArgs D = A;
                D.defer = defer;
                const char *dname = "";
                switch (dtype) {
                case MATCHATTN_F32: rc = ma::launch_fwd_generic_f32(D, rx, s, &dname); break;
                case MATCHATTN_F16: rc = ma::launch_fwd_generic_f16(D, rx, s, &dname); break;
                default: rc = ma::launch_fwd_generic_bf16(D, rx, s, &dname); break;
                }
            }
            if (rc == 0) { g_last_fwd = kname; return MATCHATTN_OK; }
            if (rc != -1)
                return fail(MATCHATTN_ERR_LAUNCH, "matchattn_forward_ws: launch of %s failed: %s", kname,
                            hipGetErrorString((hipError_t)rc));
        }
        ma::timer_mark(false, s);
        // (auto: one vector per lane; head sizes of more than 16 vectors -- 80, 96, 128 fp32 channels, 192 in the 16-bit
        // types -- only exist with two)
        for (int v = vpl; v <= (variant > 0 ? vpl : 2); ++v) {
            switch (dtype) {
            case MATCHATTN_F32: rc = ma::launch_fwd_tiled_f32(A, CH, rx, v, s, &kname); break;
            case MATCHATTN_F16: rc = ma::launch_fwd_tiled_f16(A, CH, rx, v, s, &kname); break;
            default: rc = ma::launch_fwd_tiled_bf16(A, CH, rx, v, s, &kname); break;
            }
            if (rc != -1) break;
        }
        ma::timer_mark(true, s);
        if (rc == -1 && variant > 0)
            return fail(MATCHATTN_ERR_ARG, "matchattn_forward: no tiled kernel for Ch=%d r=%d vectors/lane=%d", CH, rx, vpl);
    }
    if (rc == -1) {
        ma::timer_mark(false, s);
        switch (dtype) {
        case MATCHATTN_F32: rc = ma::launch_fwd_generic_f32(A, rx, s, &kname); break;
        case MATCHATTN_F16: rc = ma::launch_fwd_generic_f16(A, rx, s, &kname); break;
        default: rc = ma::launch_fwd_generic_bf16(A, rx, s, &kname); break;
        }
        ma::timer_mark(true, s);
    }
    g_last_fwd = kname;
    if (rc != 0)
        return fail(MATCHATTN_ERR_LAUNCH, "matchattn_forward: launch of %s failed: %s", kname,
                    rc > 0 ? hipGetErrorString((hipError_t)rc) : "no kernel");
    return MATCHATTN_OK;
}

size_t offsets_bytes(int B, int H, int W, int h, int dtype) {
    return (((size_t)B * H * W * h * 2 * elem_size(dtype)) + 255) & ~(size_t)255;
}
}  // namespace

int matchattn_forward(const void *max_offset, const void *q, const void *k, const void *v, void *out, void *attn,
                      int B, int H, int W, int C, int h, int rx, int ry, float scale, int dtype, void *stream) {
    return matchattn_forward_ws(max_offset, q, k, v, out, attn, nullptr, 0, B, H, W, C, h, rx, ry, scale, dtype, stream);
}

int matchattn_forward_ws(const void *max_offset, const void *q, const void *k, const void *v, void *out, void *attn,
                         void *workspace, size_t workspace_bytes,
                         int B, int H, int W, int C, int h, int rx, int ry, float scale, int dtype, void *stream) {
    g_err[0] = 0;
    if (int rc = check_common("matchattn_forward", B, H, W, C, h, rx, ry, dtype)) return rc;
    return forward_impl(options_now(), max_offset, q, k, v, out, attn, Placement(), workspace, workspace_bytes, B, H, W, C, h, rx, ry,
                        scale, dtype, stream);
}

// ---- forward on the library's own scratch: nothing is allocated by the caller or by the call ------------------
// One array per GPU (each device that loads the library holds its own copy at its own address, until the process
// ends).  In host code the array's name is only a handle for hipGetSymbolAddress: kernels, fills and copies take
// the device address that call returns, kept per device below.
}  // extern "C"

namespace {
constexpr size_t kStaticScratchBytes = (size_t)40 << 20;
constexpr int kMaxDevices = 64;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
namespace {
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up once per device), or null with the error set.
void *static_scratch(const char *fn) {
    int dev = -1;
    if (hipError_t e = hipGetDevice(&dev)) {
        fail(MATCHATTN_ERR_LAUNCH, "%s: hipGetDevice failed: %s", fn, hipGetErrorString(e));
        return nullptr;
    }
    if (dev < 0 || dev >= kMaxDevices) {
        fail(MATCHATTN_ERR_ARG, "%s: device index %d beyond the %d this entry point keeps scratch for", fn, dev, kMaxDevices);
        return nullptr;
    }
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (p) return p;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) {
        fail(MATCHATTN_ERR_LAUNCH, "%s: hipGetSymbolAddress failed on device %d: %s", fn, dev, hipGetErrorString(e));
        return nullptr;
    }
    if (!p || (reinterpret_cast<uintptr_t>(p) & 255u)) {
        fail(MATCHATTN_ERR_LAUNCH, "%s: scratch array at %p on device %d is not 256-byte aligned", fn, p, dev);
        return nullptr;
    }
    g_scratch_ptr[dev].store(p, std::memory_order_release);   // (two threads racing here store the same address)
    return p;
}
}  // namespace

extern "C" {

size_t matchattn_static_scratch_bytes(void) {
    g_err[0] = 0;
    return static_scratch("matchattn_static_scratch_bytes") ? kStaticScratchBytes : 0;
}

int matchattn_forward_static(const void *max_offset, const void *q, const void *k, const void *v, void *out, void *attn,
                             int B, int H, int W, int C, int h, int rx, int ry, float scale, int dtype, void *stream) {
    g_err[0] = 0;
    if (int rc = check_common("matchattn_forward_static", B, H, W, C, h, rx, ry, dtype)) return rc;
    const Options O = options_now();
    const size_t need = forward_workspace_bytes(O, B, H, W, C, h, rx, ry, dtype);
    if (need > kStaticScratchBytes)
        return fail(MATCHATTN_ERR_WORKSPACE,
                    "matchattn_forward_static: these sizes need %zu bytes of scratch, the library's own array holds %zu "
                    "(B*H*W*h = %lld head-queries; use matchattn_forward_ws with a caller-provided workspace)",
                    need, kStaticScratchBytes, (long long)B * H * W * h);
    void *ws = nullptr;
    if (need) {
        ws = static_scratch("matchattn_forward_static");
        if (!ws) return MATCHATTN_ERR_LAUNCH;
    }
    return forward_impl(O, max_offset, q, k, v, out, attn, Placement(), ws, need, B, H, W, C, h, rx, ry, scale, dtype, stream);
}

float matchattn_last_forward_kernel_ms(void) {
    if (!ma::g_fwd_timer.on || !ma::g_fwd_timer.after) return -1.f;
    float ms = -1.f;
    if (hipEventSynchronize(ma::g_fwd_timer.after) != hipSuccess) return -1.f;
    if (hipEventElapsedTime(&ms, ma::g_fwd_timer.before, ma::g_fwd_timer.after) != hipSuccess) return -1.f;
    return ms;
}

int matchattn_forward_deferred(const void *workspace, size_t workspace_bytes,
                               int B, int H, int W, int C, int h, int rx, int ry, int dtype,
                               void *stream, long long *count) {
    g_err[0] = 0;
    if (int rc = check_common("matchattn_forward_deferred", B, H, W, C, h, rx, ry, dtype)) return rc;
    if (!count) return fail(MATCHATTN_ERR_ARG, "matchattn_forward_deferred: null count pointer");
    *count = -1;
    if (!workspace || !tile_wanted(options_now(), B, H, W, C, h, rx, ry, dtype)) return MATCHATTN_OK;
    const TileLayout tl = tile_layout(B, H, W, h, tile_rows_wanted(C, h, rx, dtype));
    if (workspace_bytes < tl.total)
        return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_forward_deferred: workspace of %zu bytes needed, %zu given",
                    tl.total, workspace_bytes);
    const size_t nhq = (size_t)B * H * W * h;
    std::vector<uint8_t> flags(nhq);
    hipStream_t s = (hipStream_t)stream;
    hipError_t e = hipMemcpyAsync(flags.data(), (const char *)workspace + tl.defer_off, nhq, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess)
        return fail(MATCHATTN_ERR_LAUNCH, "matchattn_forward_deferred: copy failed: %s", hipGetErrorString(e));
    long long n = 0;
    for (uint8_t f : flags) n += f != 0;
    *count = n;
    return MATCHATTN_OK;
}

size_t matchattn_forward_fused_workspace_bytes(int B, int H, int W, int C, int h, int rx, int ry, int dtype) {
    if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || h <= 0) return 0;
    // only the LDS-tile path wants scratch: the sampling positions (a pass of their own prepares them for the bucketing,
    // which reads every position three times) and the buckets; the other kernels take relative positions as they are
    const size_t fw = forward_workspace_bytes(options_now(), B, H, W, C, h, rx, ry, dtype);
    return fw ? offsets_bytes(B, H, W, h, dtype) + fw : 0;
}

int matchattn_forward_fused(const void *position, int position_heads, const void *q, const void *k, const void *v,
                            const void *gate, void *out, long long out_row_stride, void *attn, long long attn_row_stride,
                            void *workspace, size_t workspace_bytes,
                            int B, int H, int W, int C, int h, int rx, int ry, float scale, int dtype, void *stream) {
    g_err[0] = 0;
    if (int rc = check_common("matchattn_forward_fused", B, H, W, C, h, rx, ry, dtype)) return rc;
    if (!position) return fail(MATCHATTN_ERR_ARG, "matchattn_forward_fused: null tensor pointer");
    if (position_heads != 0 && position_heads != 1 && position_heads != h)
        return fail(MATCHATTN_ERR_ARG, "matchattn_forward_fused: position_heads must be 0 (sampling positions given), 1 or h=%d, got %d",
                    h, position_heads);
    if (out_row_stride < 0 || attn_row_stride < 0)
        return fail(MATCHATTN_ERR_ARG, "matchattn_forward_fused: negative row stride");
    const Options O = options_now();
    Placement P;
    P.out_stride = out_row_stride; P.attn_stride = attn_row_stride; P.gate = gate;
    P.shared_offsets = position_heads == 1;
    if (position_heads == 0)
        return forward_impl(O, position, q, k, v, out, attn, P, workspace, workspace_bytes, B, H, W, C, h, rx, ry, scale, dtype, stream);
    // Relative positions.  Without the LDS-tile path (small maps, or no workspace) the kernel that runs adds the pixel grid
    // and clamps in its own prologue: no launch beside it.  (Element-aligned positions are all that path needs.)
    const size_t ob = offsets_bytes(B, H, W, h, dtype);
    const size_t fw = forward_workspace_bytes(O, B, H, W, C, h, rx, ry, dtype);
    if (!fw || !workspace) {
        if (reinterpret_cast<uintptr_t>(position) & (elem_size(dtype) - 1))
            return fail(MATCHATTN_ERR_ARG, "matchattn_forward_fused: position is not aligned to its element size");
        P.rel_heads = position_heads;
        return forward_impl(O, position, q, k, v, out, attn, P, nullptr, 0, B, H, W, C, h, rx, ry, scale, dtype, stream);
    }
    // LDS-tile path: the sampling positions go to the head of the workspace, the rest serves the kernels
    if (workspace_bytes < ob + fw || (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_forward_fused: a 16-byte aligned workspace of %zu bytes is needed, %zu given",
                    ob + fw, workspace_bytes);
    const int nhq = B * H * W * h;
    const float lo_x = (float)rx, hi_x = (float)((double)(W - 1 - rx) - 1e-3), lo_y = (float)ry, hi_y = (float)((double)(H - 1 - ry) - 1e-3);
    const dim3 grid((unsigned)((nhq + 255) / 256)), block(256);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
    case MATCHATTN_F32:
        hipLaunchKernelGGL((ma::make_offsets_kernel<float>), grid, block, 0, s, (const float *)position, (float *)workspace, nhq, h,
                           position_heads, W, H * W, lo_x, hi_x, lo_y, hi_y);
        break;
    case MATCHATTN_F16:
        hipLaunchKernelGGL((ma::make_offsets_kernel<ma::half_t>), grid, block, 0, s, (const ma::half_t *)position,
                           (ma::half_t *)workspace, nhq, h, position_heads, W, H * W, lo_x, hi_x, lo_y, hi_y);
        break;
    default:
        hipLaunchKernelGGL((ma::make_offsets_kernel<ma::bf16_t>), grid, block, 0, s, (const ma::bf16_t *)position,
                           (ma::bf16_t *)workspace, nhq, h, position_heads, W, H * W, lo_x, hi_x, lo_y, hi_y);
        break;
    }
    if (hipError_t e = hipGetLastError())
        return fail(MATCHATTN_ERR_LAUNCH, "matchattn_forward_fused: launch failed: %s", hipGetErrorString(e));
    const size_t rest = workspace_bytes - ob;
    return forward_impl(O, workspace, q, k, v, out, attn, P, (char *)workspace + ob, rest, B, H, W, C, h, rx, ry, scale,
                        dtype, stream);
}

namespace {
struct BwdLayout { size_t sort_off, centre_off, dl_off, tile_off, total; SortLayout sl; bool tile; TileLayout tl; };
// bytes of one (logit gradient, attention value) pair: two floats for fp32 tensors, two halves otherwise (PairOf<T>)
size_t pair_bytes(int dtype) { return dtype == MATCHATTN_F32 ? 8 : 4; }
// Whether pass A of the gather backward would run on LDS tiles (shapes the tile kernels have; the (dl, a)
// scratch must fit the 32-bit offsets of a buffer descriptor).
bool bwd_tile_wanted(const Options &O, int B, int H, int W, int C, int h, int rx, int dtype) {
    const int CH = C / h, M = (2 * rx + 2) * (2 * rx + 2), mode = O.backward_mode;
    if (mode == 2 || mode == 0) return false;
    const int head_bytes = CH * (int)elem_size(dtype);
    if (!(rx <= 2 && (CH == 16 || CH == 32 || CH == 64) &&
          h % (head_bytes >= 128 ? 1 : 128 / head_bytes) == 0 &&
          (unsigned long long)B * H * W * h * M * pair_bytes(dtype) < 0xFFFFF000ull))
        return false;
    if (mode == 1) return true;
    // auto: maps large enough to pay for the second bucketing.  Whole backward with pass A on tiles against the direct
    // pass A, heads of 16 and 32 channels, i.i.d. and smooth fields, shared and per-head offsets (one process):
    //   fp16  6x6 window: 0.91x to 1.02x at 2^18 head-queries, 0.98x to 1.27x at 2^19, 1.06x to 1.42x at 2^20;
    //         4x4 window: 0.85x to 0.93x at 2^18, 0.92x to 1.08x at 2^19, 0.97x to 1.22x at 2^20
    //   fp32  6x6: 0.89x to 1.14x at 2^18, 1.00x to 1.25x at 2^19;  4x4: 0.82x to 0.93x at 2^18, 0.88x to 1.12x at 2^19
    //   bf16  6x6: 0.80x to 0.90x at 2^18, 0.85x to 1.12x at 2^19, 0.93x to 1.28x at 2^20;
    //         4x4: 0.82x to 0.97x at 2^19, 0.87x to 1.08x at 2^20, 0.92x to 1.27x at 2^21
    // (the smooth per-head field is the low end everywhere: its gathers already hit L1).  Heads of 64 channels, twice
    // the bytes per head-query, pay one step earlier: fp32 1.1x to 1.4x at 2^17; fp16 6x6 1.00x to 1.17x at 2^18, 4x4
    // 0.89x to 1.00x at 2^18 and 1.00x to 1.17x at 2^19; bf16 6x6 0.88x to 1.01x at 2^18 and 0.99x to 1.10x at 2^19, 4x4
    // 0.94x to 1.04x at 2^19 and 0.98x to 1.10x at 2^20.
    const long long nhq = (long long)B * H * W * h;
    if (dtype == MATCHATTN_F32) return nhq >= (CH == 64 ? (1ll << 17) : rx == 2 ? (1ll << 18) : (1ll << 19));
    if (dtype == MATCHATTN_F16) return nhq >= (rx == 2 && CH == 64 ? (1ll << 18) : (1ll << 19));
    if (CH == 64) return nhq >= (rx == 2 ? (1ll << 19) : (1ll << 20));
    return nhq >= (rx == 2 ? (1ll << 20) : (3ll << 19));
}
BwdLayout bwd_gather_layout(const Options &O, int B, int H, int W, int C, int h, int rx, int dtype) {
    BwdLayout l;
    l.sl = sort_layout(B, H, W, h, 1);              // one bin per target pixel
    const size_t nhq = (size_t)B * H * W * h, M = (size_t)(2 * rx + 2) * (2 * rx + 2);
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    l.sort_off = 0;
    l.centre_off = up(l.sl.total);
    l.dl_off = l.centre_off + up((size_t)B * H * W * h * 4);
    l.tile_off = l.dl_off + up(nhq * M * pair_bytes(dtype));
    l.total = l.tile_off;
    l.tile = bwd_tile_wanted(O, B, H, W, C, h, rx, dtype);
    if (l.tile) {
        l.tl = tile_layout(B, H, W, h, false);
        l.total += up(l.tl.total);
    }
    return l;
}
size_t bwd_scatter_bytes(int B, int H, int W, int C, int dtype) {
    if (dtype == MATCHATTN_F32) return 0;
    const size_t n = (size_t)B * H * W * C;
    return 2 * (((n * sizeof(float)) + 255) & ~(size_t)255);
}
bool bwd_gather_possible(const Options &O, int B, int H, int W, int C, int h, int rx, int dtype) {
    if (O.backward_mode == 0 || O.forward_variant == 0 || C % h) return false;
    const int CH = C / h;
    const long long L = (long long)B * H * W;
    const unsigned long long M = (unsigned long long)(2 * rx + 2) * (2 * rx + 2);
    // (the pair array is indexed with 32 bits, PairLayout::at: at most 2^32 - 1 (dl, a) pairs)
    return bwd_tiled_shape(CH, rx, dtype) && (CH * elem_size(dtype)) % 16 == 0 && H < 30000 && W < 30000 &&
           (unsigned long long)L * C * elem_size(dtype) < 0xFFFFFF00ull && (unsigned long long)L * h * M < 0xFFFFFF00ull;
}
}  // namespace

namespace {
size_t backward_workspace_bytes(const Options &O, int B, int H, int W, int C, int h, int rx, int dtype) {
    if (B <= 0 || H <= 0 || W <= 0 || C <= 0 || h <= 0) return 0;
    size_t need = bwd_scatter_bytes(B, H, W, C, dtype);
    if (bwd_gather_possible(O, B, H, W, C, h, rx, dtype)) {
        const size_t g = bwd_gather_layout(O, B, H, W, C, h, rx, dtype).total;
        if (g > need) need = g;
    }
    return need;
}
}  // namespace

size_t matchattn_backward_workspace_bytes(int B, int H, int W, int C, int h, int rx, int ry, int dtype) {
    (void)ry;
    return backward_workspace_bytes(options_now(), B, H, W, C, h, rx, dtype);
}

int matchattn_backward(const void *max_offset, const void *q, const void *k, const void *v, const void *d_out,
                       const void *d_attn, void *dq, void *dk, void *dv, void *d_max_offset, void *workspace,
                       size_t workspace_bytes, int B, int H, int W, int C, int h, int rx, int ry, float scale,
                       int dtype, void *stream) {
    g_err[0] = 0;
    if (int rc = check_common("matchattn_backward", B, H, W, C, h, rx, ry, dtype)) return rc;
    if (!max_offset || !q || !k || !v || !d_out || !dq || !dk || !dv || !d_max_offset)
        return fail(MATCHATTN_ERR_ARG, "matchattn_backward: null tensor pointer");
    const Options O = options_now();
    const size_t need = backward_workspace_bytes(O, B, H, W, C, h, rx, dtype);
    if (need && (!workspace || workspace_bytes < need))
        return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_backward: workspace of %zu bytes needed, %zu given", need,
                    workspace ? workspace_bytes : (size_t)0);
    if (need && (reinterpret_cast<uintptr_t>(workspace) & 15u))
        return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_backward: workspace must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const long long L = (long long)B * H * W;
    const size_t n = (size_t)L * C;
    const int CH = C / h;

    ma::BwdArgs A;
    A.mo = max_offset; A.q = q; A.k = k; A.v = v; A.d_out = d_out; A.d_attn = d_attn;
    A.dq = dq; A.dmo = d_max_offset;
    A.dl_ws = nullptr; A.dk = dk; A.dv = dv;
    A.perm = nullptr; A.centre = nullptr; A.bin_start = nullptr; A.row_start = nullptr; A.per_head = nullptr; A.nrows = B * H;
    A.only_flagged = nullptr;
    A.nhq = (int)(L * h); A.N = H * W; A.H = H; A.W = W; A.C = C; A.h = h;
    A.scale = scale; A.xcd_swizzle = O.xcd_swizzle;

    // ---- gather mode: deterministic, no atomics (pass A per query, inverse index, pass B per key) ----
    {
        const void *gp[] = {q, k, v, d_out, dq, dk, dv};
        if (bwd_gather_possible(O, B, H, W, C, h, rx, dtype) && tiled_ok(gp, 7, L, C, CH, dtype) &&
            (!d_attn || (reinterpret_cast<uintptr_t>(d_attn) & (elem_size(dtype) - 1)) == 0)) {
            const BwdLayout bl = bwd_gather_layout(O, B, H, W, C, h, rx, dtype);
            if (!workspace || workspace_bytes < bl.total)
                return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_backward: workspace of %zu bytes needed, %zu given",
                            bl.total, workspace ? workspace_bytes : (size_t)0);
            char *ws = (char *)workspace;
            const SortLayout &sl = bl.sl;
            ma::SortArgs S = sort_args(max_offset, dtype, B, H, W, h, sl, ws, 1, 1, 1);
            S.centre = (int *)(ws + bl.centre_off);
            launch_sort(S, sl, L, h, ws, true, s);
            if (hipError_t e = hipGetLastError())
                return fail(MATCHATTN_ERR_LAUNCH, "matchattn_backward: index launch failed: %s", hipGetErrorString(e));
            A.dl_ws = ws + bl.dl_off;                                       // (dl, a) pairs
            A.dk_acc = nullptr; A.dv_acc = nullptr;
            A.perm = S.perm; A.centre = S.centre; A.bin_start = S.count; A.row_start = S.rowtot; A.per_head = S.per_head;
            const char *kname = "";
            int rc = -1;
            if (bl.tile) {
                // pass A on LDS tiles: a second bucketing (by K/V tile), the tile kernel, then the direct kernel
                // for the head-queries the tile kernel flagged
                char *tws = ws + bl.tile_off;
                ma::SortArgs TS = sort_args(max_offset, dtype, B, H, W, h, bl.tl.sl, tws, ma::kTileDims[0], ma::kTileDims[1], 1);
                TS.shared_perm = 1;
                TS.pop = (int *)(tws + bl.tl.chunk_off);
                launch_sort(TS, bl.tl.sl, L, h, tws, false, s);
                const ma::TileSort T = tile_sort_args(TS, bl.tl, tws);
                switch (dtype) {
                case MATCHATTN_F32: rc = ma::launch_bwd_tile_f32(A, T, CH, rx, s); break;
                case MATCHATTN_F16: rc = ma::launch_bwd_tile_f16(A, T, CH, rx, s); break;
                default: rc = ma::launch_bwd_tile_bf16(A, T, CH, rx, s); break;
                }
                if (rc == 0) {
                    ma::BwdArgs F = A;
                    F.only_flagged = T.defer;
                    switch (dtype) {
                    case MATCHATTN_F32: rc = ma::launch_bwd_tiled_f32(F, CH, rx, s, &kname); kname = "bwd_tile_f32"; break;
                    case MATCHATTN_F16: rc = ma::launch_bwd_tiled_f16(F, CH, rx, s, &kname); kname = "bwd_tile_f16"; break;
                    default: rc = ma::launch_bwd_tiled_bf16(F, CH, rx, s, &kname); kname = "bwd_tile_bf16"; break;
                    }
                }
            }
            if (rc == -1) {
                switch (dtype) {
                case MATCHATTN_F32: rc = ma::launch_bwd_tiled_f32(A, CH, rx, s, &kname); break;
                case MATCHATTN_F16: rc = ma::launch_bwd_tiled_f16(A, CH, rx, s, &kname); break;
                default: rc = ma::launch_bwd_tiled_bf16(A, CH, rx, s, &kname); break;
                }
            }
            if (rc == 0) {
                switch (dtype) {
                case MATCHATTN_F32: rc = ma::launch_bwd_key_f32(A, CH, rx, s); break;
                case MATCHATTN_F16: rc = ma::launch_bwd_key_f16(A, CH, rx, s); break;
                default: rc = ma::launch_bwd_key_bf16(A, CH, rx, s); break;
                }
            }
            g_last_bwd = kname;
            if (rc != 0)
                return fail(MATCHATTN_ERR_LAUNCH, "matchattn_backward: launch of %s (gather) failed: %s", kname,
                            rc > 0 ? hipGetErrorString((hipError_t)rc) : "no kernel");
            return MATCHATTN_OK;
        }
    }

    // ---- scatter mode: fp32 atomics (any shape) ----
    const size_t need_scatter = bwd_scatter_bytes(B, H, W, C, dtype);
    if (need_scatter && (!workspace || workspace_bytes < need_scatter))
        return fail(MATCHATTN_ERR_WORKSPACE, "matchattn_backward: workspace of %zu bytes needed, %zu given", need_scatter,
                    workspace ? workspace_bytes : (size_t)0);
    if (dtype == MATCHATTN_F32) {
        A.dk_acc = (float *)dk;
        A.dv_acc = (float *)dv;
    } else {
        A.dk_acc = (float *)workspace;
        A.dv_acc = (float *)((char *)workspace + need_scatter / 2);
    }

    const size_t want_blocks = (n / 4 + 255) / 256 + 1;
    const unsigned fill_blocks = (unsigned)(want_blocks < 8192 ? want_blocks : 8192);
    hipLaunchKernelGGL(ma::fill_zero_kernel, dim3(fill_blocks), dim3(256), 0, s, A.dk_acc, n);
    hipLaunchKernelGGL(ma::fill_zero_kernel, dim3(fill_blocks), dim3(256), 0, s, A.dv_acc, n);
    if (hipError_t e = hipGetLastError())
        return fail(MATCHATTN_ERR_LAUNCH, "matchattn_backward: fill launch failed: %s", hipGetErrorString(e));

    const void *ptrs[] = {q, k, v, d_out, dq};
    const char *kname = "";
    int rc = -1;
    if (O.forward_variant != 0 && rx <= 2 && tiled_ok(ptrs, 5, L, C, CH, dtype) &&
        (!d_attn || (reinterpret_cast<uintptr_t>(d_attn) & (elem_size(dtype) - 1)) == 0)) {
        switch (dtype) {
        case MATCHATTN_F32: rc = ma::launch_bwd_tiled_f32(A, CH, rx, s, &kname); break;
        case MATCHATTN_F16: rc = ma::launch_bwd_tiled_f16(A, CH, rx, s, &kname); break;
        default: rc = ma::launch_bwd_tiled_bf16(A, CH, rx, s, &kname); break;
        }
    }
    if (rc == -1) {
        switch (dtype) {
        case MATCHATTN_F32: rc = ma::launch_bwd_generic_f32(A, rx, s, &kname); break;
        case MATCHATTN_F16: rc = ma::launch_bwd_generic_f16(A, rx, s, &kname); break;
        default: rc = ma::launch_bwd_generic_bf16(A, rx, s, &kname); break;
        }
    }
    g_last_bwd = kname;
    if (rc != 0)
        return fail(MATCHATTN_ERR_LAUNCH, "matchattn_backward: launch of %s failed: %s", kname,
                    rc > 0 ? hipGetErrorString((hipError_t)rc) : "no kernel");

    if (dtype != MATCHATTN_F32) {
        const unsigned nb = fill_blocks;
        if (dtype == MATCHATTN_F16)
            hipLaunchKernelGGL((ma::narrow_kernel<ma::half_t>), dim3(nb), dim3(256), 0, s, A.dk_acc, A.dv_acc,
                               (ma::half_t *)dk, (ma::half_t *)dv, n);
        else
            hipLaunchKernelGGL((ma::narrow_kernel<ma::bf16_t>), dim3(nb), dim3(256), 0, s, A.dk_acc, A.dv_acc,
                               (ma::bf16_t *)dk, (ma::bf16_t *)dv, n);
        if (hipError_t e = hipGetLastError())
            return fail(MATCHATTN_ERR_LAUNCH, "matchattn_backward: narrow launch failed: %s", hipGetErrorString(e));
    }
    return MATCHATTN_OK;
}

}  // extern "C"

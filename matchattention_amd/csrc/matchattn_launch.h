// Host-side launch entry points, one set per storage dtype (each compiled in its own
// translation unit so that the build parallelises).
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>

namespace ma {

struct FwdArgs;
struct BwdArgs;
struct TileSort;

// Returns hipSuccess (0) or the launch error; -1 when no tiled kernel exists for
// (CH, R, VPL) in this dtype -- the caller then uses the generic kernel.
// *name receives a static string naming the kernel that was launched.
int launch_fwd_tiled_f32(const FwdArgs &A, int CH, int R, int VPL, hipStream_t s, const char **name);
int launch_fwd_tiled_f16(const FwdArgs &A, int CH, int R, int VPL, hipStream_t s, const char **name);
int launch_fwd_tiled_bf16(const FwdArgs &A, int CH, int R, int VPL, hipStream_t s, const char **name);
int launch_fwd_generic_f32(const FwdArgs &A, int R, hipStream_t s, const char **name);
int launch_fwd_generic_f16(const FwdArgs &A, int R, hipStream_t s, const char **name);
int launch_fwd_generic_bf16(const FwdArgs &A, int R, hipStream_t s, const char **name);

// LDS-tile forward (fp16 only); -1 when no instance exists for (CH, R) or h is not a multiple of the head group.
int launch_fwd_tile_f16(const FwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s, const char **name);
// the same for fp32 (head size 16 or 32) and bf16 storage (matchattn_fwd_tile_t.h)
int launch_fwd_tile_f32(const FwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s, const char **name);
int launch_fwd_tile_bf16(const FwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s, const char **name);

// Optional timing of the dominant kernel of a forward call (option "time_kernels"): when `on`, the launcher of
// that kernel records the two events on the stream either side of the launch.
struct KernelTimer { std::atomic<bool> on; hipEvent_t before, after; };
extern KernelTimer g_fwd_timer;
inline void timer_mark(bool end, hipStream_t s) {
    if (g_fwd_timer.on) (void)hipEventRecord(end ? g_fwd_timer.after : g_fwd_timer.before, s);
}
// Size of the persistent grid of the LDS-tile kernels: `per_cu` workgroups for every compute unit of the current device
// (asked from the runtime once per device), rounded up to a multiple of the 8 XCDs the kernels' work split assumes
// (workgroup i runs on XCD i mod 8; on a part with another XCD count the split still covers every item, each
// workgroup claiming from the counter of "its" eighth, only the L2 locality it aims for is lost).
unsigned tile_grid(unsigned per_cu);
// Builds the work list of the LDS-tile kernels (tile_chunks_kernel); queries_per_pass is the number of queries per head the
// consuming kernel takes from a chunk at a time (prices a chunk for the split of the list among the XCDs).  Defined once, beside the fp16 forward tile kernel:
// a second copy in another translation unit would be a second device kernel of the same name.
void launch_tile_chunks(const TileSort &S, int h, int queries_per_pass, hipStream_t s);
extern const int kTileDims[2];       // tile width and height (key pixels) the kernels were built for
extern const int kTileCapHost;       // queries per head in one work item of that kernel

int launch_bwd_tiled_f32(const BwdArgs &A, int CH, int R, hipStream_t s, const char **name);
int launch_bwd_tiled_f16(const BwdArgs &A, int CH, int R, hipStream_t s, const char **name);
int launch_bwd_tiled_bf16(const BwdArgs &A, int CH, int R, hipStream_t s, const char **name);
int launch_bwd_key_f32(const BwdArgs &A, int CH, int R, hipStream_t s);
int launch_bwd_key_f16(const BwdArgs &A, int CH, int R, hipStream_t s);
int launch_bwd_key_bf16(const BwdArgs &A, int CH, int R, hipStream_t s);
// LDS-tile pass A of the gather-mode backward (fp16 only); -1 when no instance exists
int launch_bwd_tile_f16(const BwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s);
// the same for fp32 (head size 16 or 32) and bf16 storage (matchattn_bwd_tile_t.h)
int launch_bwd_tile_f32(const BwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s);
int launch_bwd_tile_bf16(const BwdArgs &A, const TileSort &S, int CH, int R, hipStream_t s);
int launch_bwd_generic_f32(const BwdArgs &A, int R, hipStream_t s, const char **name);
int launch_bwd_generic_f16(const BwdArgs &A, int R, hipStream_t s, const char **name);
int launch_bwd_generic_bf16(const BwdArgs &A, int R, hipStream_t s, const char **name);

}  // namespace ma

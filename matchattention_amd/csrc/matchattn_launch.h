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
extern const int kTileLog2[2];       // log2 of the tile width and height the kernel was built for
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

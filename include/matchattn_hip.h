/*
 * C ABI of libmatchattn_hip.so -- the gfx950 (MI355X) MatchAttention operator.
 *
 * These entry points are what a binding of the reference's fused operator would
 * bind.  They replace, for mat_impl='hip':
 *   - the compiled module behind `match_attention.fused_forward(...)`
 *     (reference models/src/match_former_cuda.cpp:24-49, host driver
 *     models/src/match_former_fused_forward.cu:461-628), called from
 *     models/match_former_ops.py:28-39;
 *   - and, for training, the autograd that the reference only has through its
 *     pure-PyTorch path (models/mat_pytorch_impl.py:1-178 via
 *     models/attention_blocks.py:82-91).
 * Semantics follow the PyTorch definition (per-tap replicate clamp, one softmax
 * per (2r+1)^2 sub-window), not the reference's CUDA kernels where the two differ.
 *
 * Conventions
 *   - plain device pointers and sizes, no framework types; all tensors contiguous;
 *   - max_offset [B,N,h,2] (x = column, y = row), q/k/v/out [B,N,C],
 *     attn [B,N,h,M], N = H*W, C = h*Ch, M = (2*rx+2)*(2*ry+2);
 *   - all tensors of one call share `dtype`;
 *   - work is enqueued on `stream` (a hipStream_t; NULL = the null stream) of the
 *     current device; nothing is synchronised and nothing is allocated;
 *   - outputs need not be zeroed by the caller;
 *   - return 0 on success; otherwise a non-zero code, with a message available
 *     from matchattn_last_error() (thread-local).
 */
#ifndef MATCHATTN_HIP_H_
#define MATCHATTN_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { MATCHATTN_F32 = 0, MATCHATTN_F16 = 1, MATCHATTN_BF16 = 2 };

enum {
    MATCHATTN_OK = 0,
    MATCHATTN_ERR_ARG = 1,        /* bad shape / dtype / null pointer / unsupported window */
    MATCHATTN_ERR_WORKSPACE = 2,  /* workspace missing or too small */
    MATCHATTN_ERR_LAUNCH = 3      /* the HIP runtime reported an error at launch */
};

/* ABI version of this header (bumped on any signature change). */
int matchattn_abi_version(void);

/* Message of the last failing call on this thread ("" if none). */
const char *matchattn_last_error(void);

/*
 * Forward: out, attn = MatchAttention(max_offset, q, k, v).
 * Replaces match_former_fused_forward (models/src/match_former_fused_forward.cu:461-628)
 * with attn_type == "l1_norm"; `scale` multiplies the negative-L1 logits
 * (models/attention_blocks.py:86).  rx must equal ry (the reference's window is
 * always square, models/attention_blocks.py:115,118), 1 <= rx <= 3.
 */
int matchattn_forward(const void *max_offset, const void *q, const void *k, const void *v,
                      void *out, void *attn,
                      int B, int H, int W, int C, int h, int rx, int ry,
                      float scale, int dtype, void *stream);

/*
 * Forward with scratch memory.  For large, spatially incoherent offset fields the forward is
 * faster when it may first order the queries by sampling target (a counting sort into a
 * permutation held in `workspace`); results are identical.  matchattn_forward_workspace_bytes
 * returns the bytes that would be used for these sizes (0 when the ordering would not be used);
 * a NULL workspace makes this call the same as matchattn_forward.  No counterpart in the
 * reference (its driver allocates its temporaries itself, match_former_fused_forward.cu:492-527).
 */
size_t matchattn_forward_workspace_bytes(int B, int H, int W, int C, int h, int rx, int ry, int dtype);
int matchattn_forward_ws(const void *max_offset, const void *q, const void *k, const void *v,
                         void *out, void *attn, void *workspace, size_t workspace_bytes,
                         int B, int H, int W, int C, int h, int rx, int ry,
                         float scale, int dtype, void *stream);

/*
 * matchattn_forward_ws on scratch memory the library owns.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory around the call -- code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  The scratch is one static device array of matchattn_static_scratch_bytes()
 * = 40 MiB per GPU (held by every GPU the library is used on until the process ends), enough for 4.6 M
 * head-queries (B*H*W*h; the 544x960, 8-head map needs 36.2 MiB); larger sizes are rejected with
 * MATCHATTN_ERR_WORKSPACE.  Neither call allocates or frees anything; results are bit-identical to
 * matchattn_forward_ws.  Every call on a GPU uses that GPU's one array, so two calls that overlap on one GPU
 * (two streams, two threads) race: serialise them.  matchattn_static_scratch_bytes looks the array's device
 * address up for the current device (once per device; matchattn_forward_static does the same on its first call
 * there) and returns the capacity, or 0 with the error set: call it once per device before a stream capture.
 */
size_t matchattn_static_scratch_bytes(void);
int matchattn_forward_static(const void *max_offset, const void *q, const void *k, const void *v,
                             void *out, void *attn,
                             int B, int H, int W, int C, int h, int rx, int ry,
                             float scale, int dtype, void *stream);

/*
 * Forward fused with the steps the attention module runs either side of the operator.
 *
 * Before (replaces the elementwise passes of models/attention_blocks.py:149-151 / 162-163 and the module's
 * clamp_max_offset, :45-59, :79): `position` holds positions RELATIVE to each query pixel,
 * [B,N,position_heads,2] with position_heads == h, or 1 for one position shared by all heads (the
 * cross-attention field, :162).  The pixel's own (x, y), in the tensor dtype, is added and the sum clamped
 * to [r, size-1-r-1e-3] with the bounds rounded to the tensor dtype, bit for bit what those lines compute.
 * position_heads == 0 means `position` already holds the clamped sampling positions [B,N,h,2], as
 * matchattn_forward takes them.
 *
 * After (replaces :96-98 of the cross-attention module): with `gate` ([B,N,C], or NULL) the stored output is
 * round(gate * round(out)); `out` rows start every out_row_stride elements and `attn` rows (h*M values per
 * pixel) every attn_row_stride elements (0: contiguous), so both can be column ranges of the [B,N,C+h*M]
 * input of the output projection: out = buf, attn = buf + C, both strides C + h*M.
 *
 * Workspace: matchattn_forward_fused_workspace_bytes returns what these sizes would use (16-byte aligned scratch), 0 for
 * maps that do not take the LDS-tile path: there the kernel that runs adds the pixel grid and clamps in its own prologue
 * and the call is a single launch.  On the LDS-tile path the sampling positions are first written to the head of the
 * workspace by a pass of their own (the bucketing reads every position three times); a NULL workspace selects the
 * single-launch kernels at any size.
 * matchattn_backward differentiates the operator itself; a binding that trains through this call applies the gate's
 * and the clamp's own gradients around it (matchattention_amd/match_former_ops.py does).
 */
size_t matchattn_forward_fused_workspace_bytes(int B, int H, int W, int C, int h, int rx, int ry, int dtype);
int matchattn_forward_fused(const void *position, int position_heads,
                            const void *q, const void *k, const void *v, const void *gate,
                            void *out, long long out_row_stride, void *attn, long long attn_row_stride,
                            void *workspace, size_t workspace_bytes,
                            int B, int H, int W, int C, int h, int rx, int ry,
                            float scale, int dtype, void *stream);

/*
 * Bytes of scratch the backward needs for these sizes (per-tap logit gradients and attention
 * weights plus an inverse index of the sampling centres for the gather mode; fp32 staging of dK
 * and dV for the atomic mode with 16-bit dtypes).  The binding allocates it from its own
 * allocator and passes it in; contents on entry are irrelevant.
 */
size_t matchattn_backward_workspace_bytes(int B, int H, int W, int C, int h, int rx, int ry, int dtype);

/*
 * Backward of matchattn_forward.  Counterpart in the reference: autograd through
 * models/mat_pytorch_impl.py (the reference's fused op registers no backward,
 * models/match_former_ops.py:6).
 *   d_out  [B,N,C]    gradient of out
 *   d_attn [B,N,h,M]  gradient of attn, or NULL when attn is not used downstream
 *   dq, dk, dv [B,N,C], d_max_offset [B,N,h,2]: overwritten.
 * The forward is recomputed from q and k; nothing is saved between the two calls.
 */
int matchattn_backward(const void *max_offset, const void *q, const void *k, const void *v,
                       const void *d_out, const void *d_attn,
                       void *dq, void *dk, void *dv, void *d_max_offset,
                       void *workspace, size_t workspace_bytes,
                       int B, int H, int W, int C, int h, int rx, int ry,
                       float scale, int dtype, void *stream);

/*
 * Test/benchmark knob: choose a kernel variant instead of the built-in heuristic.
 *   name "forward_variant":  -1 auto, 0 generic (one lane per head-query, any Ch),
 *                            1/2 tiled kernel with that many 16-byte vectors per lane
 *   name "stereo_row_skip":   1 (default) skip the last window row when every lane of a
 *                            wavefront has an integer y (its weights are exactly 0), 0 never
 *   name "forward_lds":      -1 (default) auto, 1 always, 0 never: r <= 2, head size 16/32/64, workspace given --
 *                            bucket the queries by the 16x8 tile of K/V their window centre falls in, stage
 *                            each tile with its halo in LDS once and read every tap from LDS.  Auto uses it
 *                            from the map sizes at which it measured faster than the direct kernel over
 *                            i.i.d. and smooth offset fields (geometric mean), in head-queries B*H*W*h:
 *                              fp16  r = 2: 2^20 (32 channels per head), 2^19 (64), 1.5 * 2^20 (16);
 *                                    r = 1: 2^21 (32 and 16), 2^20 (64)
 *                              bf16  r = 2: 2^20 (32), 2^19 (64), 2^21 (16); r = 1: 2^21 (32), never (16, 64)
 *                              fp32  r = 2: 2^19 (16 and 32), 2^17 (64); r = 1: 2^20 (32), 1.5 * 2^20 (16), 2^18 (64)
 *   name "backward_mode":     -1 auto (default: gather where a tiled kernel exists), 0 scatter dK/dV with
 *                            fp32 atomics, 1 / 2 gather them per key through an inverse index
 *                            (deterministic) with the per-query pass on LDS tiles wherever that kernel
 *                            exists (1: head size 16/32/64) or always on the direct kernel (2); auto
 *                            takes the tiles from the sizes at which the whole backward measured faster with
 *                            them: fp32 from 2^18 head-queries with r = 2, 2^19 with r = 1, 2^17 for heads of
 *                            64 channels; fp16 from 2^19 (2^18 for 64 channels and r = 2); bf16 from 2^20
 *                            with r = 2 and 1.5 * 2^20 with r = 1 (64 channels: 2^19 and 2^20)
 *   name "time_kernels":      0 (default) / 1: see matchattn_last_forward_kernel_ms
 *   name "xcd_swizzle":       1 (default) give each XCD a contiguous band of the image, 0 keep
 *                            the hardware's round-robin workgroup order
 * Returns 0, or MATCHATTN_ERR_ARG for an unknown name/value.  Process-wide.
 */
int matchattn_set_option(const char *name, int value);

/* Name of the kernel variant the last forward / backward call of this process launched. */
const char *matchattn_last_forward_kernel(void);
const char *matchattn_last_backward_kernel(void);

/*
 * Diagnostic (no counterpart in the reference): with option "time_kernels" = 1 a forward call records two HIP
 * events on the caller's stream, either side of the launch of its dominant kernel (the one
 * matchattn_last_forward_kernel names; not the bucketing kernels before it nor the scan after it).  This waits for
 * the second event and returns the time between them in milliseconds for the last forward call of the process;
 * negative when the option is off or nothing was recorded.  One pair of events per process: not for concurrent
 * callers, and not inside a stream capture.
 */
float matchattn_last_forward_kernel_ms(void);

/*
 * Diagnostic (no counterpart in the reference): after a matchattn_forward_ws call with the same sizes and this
 * `workspace` took the LDS-tile path, *count = the number of (pixel, head) pairs the tile kernel left to the
 * direct kernel (window outside the staged tile, or sub-windows that need the exact softmax); *count = -1
 * when these sizes do not take the tile path.  The results are the same either way; a large count means the
 * call ran at the direct kernel's speed.  Waits for `stream`, copies one byte per pair to the host.
 */
int matchattn_forward_deferred(const void *workspace, size_t workspace_bytes,
                               int B, int H, int W, int C, int h, int rx, int ry, int dtype,
                               void *stream, long long *count);

#ifdef __cplusplus
}
#endif
#endif /* MATCHATTN_HIP_H_ */

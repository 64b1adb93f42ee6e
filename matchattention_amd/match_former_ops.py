"""mat_impl='hip': the MatchAttention fused operator on MI355X.

Host-side mirror of the reference's operator boundary, models/match_former_ops.py:
  * ``MF_FusedForwardOps`` -- same constructor and ``forward`` signature
    (models/match_former_ops.py:65-121), so ``MatchAttention`` in
    models/attention_blocks.py:43,93 can use it unchanged;
  * ``fused_forward`` -- the 12-argument in-place call the reference's custom op makes
    into its compiled module (models/match_former_ops.py:30-33,
    models/src/match_former_cuda.cpp:24-49).
Unlike the reference's fused path this one is differentiable: the backward kernel is
registered with autograd (the reference trains only through mat_impl='pytorch').

Everything here is plumbing around libmatchattn_hip.so; tensors must be on the GPU.
"""
from typing import List, Optional, Tuple

import torch
import torch.nn as nn

from . import _cabi

_DTYPES = {torch.float32: _cabi.F32, torch.float16: _cabi.F16, torch.bfloat16: _cabi.BF16}


def _check_inputs(max_offset, q, k, v, H, W, win_r, attn_num, attn_type):
    if attn_type != "l1_norm":
        # The reference's other option ("dot_product", models/src/match_former_fused_forward.cu:560)
        # is never selected by the model (models/attention_blocks.py:93).
        raise ValueError(f"mat_impl='hip' implements attn_type='l1_norm' only, got {attn_type!r}")
    if q.dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {q.dtype}")
    if q.dim() != 3 or max_offset.dim() != 4 or max_offset.size(-1) != 2:
        raise ValueError("expected q [B,N,C] and max_offset [B,N,h,2]")
    B, N, C = q.shape
    h = max_offset.size(2)
    for name, t in (("max_offset", max_offset), ("q", q), ("k", k), ("v", v)):
        if not t.is_cuda:
            raise ValueError(f"{name} must be a GPU tensor (mat_impl='hip' has no CPU path)")
        if t.dtype != q.dtype or t.device != q.device:
            raise TypeError(f"{name}: dtype/device differ from q ({t.dtype}, {t.device})")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    if k.shape != q.shape or v.shape != q.shape or max_offset.shape[:2] != (B, N):
        raise ValueError("q, k, v must share [B,N,C]; max_offset must be [B,N,h,2]")
    if N != H * W:
        raise ValueError(f"N={N} != H*W={H * W}")
    if len(win_r) != 2 or attn_num != (2 * win_r[0] + 2) * (2 * win_r[1] + 2):
        raise ValueError(f"attn_num={attn_num} does not match win_r={list(win_r)}")
    return B, N, C, h


def _stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def fused_forward(max_offset, q, k, v, output, attn_out, H, W, win_r, attn_num, attn_type, scale) -> None:
    """In-place forward with the reference's native signature
    (models/src/match_former_cuda.cpp:24-39): fills ``output`` [B,N,C] and ``attn_out``
    [B,N,h,attn_num].  The outputs need not be zeroed."""
    B, N, C, h = _check_inputs(max_offset, q, k, v, H, W, win_r, attn_num, attn_type)
    if output.shape != (B, N, C) or attn_out.shape != (B, N, h, attn_num):
        raise ValueError("output / attn_out have the wrong shape")
    for t in (output, attn_out):
        if t.dtype != q.dtype or t.device != q.device or not t.is_contiguous():
            raise TypeError("output / attn_out must match q's dtype and device and be contiguous")
    lib = _cabi.load()
    dt = _DTYPES[q.dtype]
    with torch.cuda.device(q.device):
        # scratch for the optional ordering of queries by sampling target (0 bytes when not used)
        ws_bytes = lib.matchattn_forward_workspace_bytes(B, H, W, C, h, int(win_r[0]), int(win_r[1]), dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        _cabi.check(lib.matchattn_forward_ws(
            max_offset.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), output.data_ptr(), attn_out.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes,
            B, H, W, C, h, int(win_r[0]), int(win_r[1]), float(scale), dt, _stream_ptr(q.device)))


# Dispatcher route.  When ``import match_attention`` fails, the reference's operator falls back to
# ``torch.ops.match_attention.fused_forward`` (models/match_former_ops.py:34-39), which its extension registers with
# the schema of models/src/match_former_cuda.cpp:46-49.  The same name and schema are defined here (as a fragment: the
# reference's own file defines ``match_attention::fused_forward_ops`` in that namespace), so that branch lands in
# this library as well once ``matchattention_amd`` has been imported.
_DISPATCH_LIB = torch.library.Library("match_attention", "FRAGMENT")
_DISPATCH_LIB.define("fused_forward(Tensor max_offset, Tensor q, Tensor k, Tensor v, Tensor(a!) output, "
                     "Tensor(b!) attn_out, int H, int W, int[] win_r, int attn_num, str attn_type, float scale) -> ()")
_DISPATCH_LIB.impl("fused_forward", fused_forward, "CUDA")


@torch.library.custom_op("matchattention_amd::fused_forward_ops", mutates_args={"output", "attn_out"})
def fused_forward_ops(max_offset: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      output: torch.Tensor, attn_out: torch.Tensor, H: int, W: int, win_r: List[int],
                      attn_num: int, attn_type: str, scale: float) -> None:
    """Opaque (to torch.compile) in-place op; same schema as the reference's
    ``match_attention::fused_forward_ops`` (models/match_former_ops.py:6-20)."""
    fused_forward(max_offset, q, k, v, output, attn_out, H, W, win_r, attn_num, attn_type, scale)


@fused_forward_ops.register_fake
def _(max_offset, q, k, v, output, attn_out, H, W, win_r, attn_num, attn_type, scale):
    B, N, C = q.shape
    h = max_offset.size(2)
    torch._check(output.shape == (B, N, C), lambda: f"output shape {tuple(output.shape)} != {(B, N, C)}")
    torch._check(attn_out.shape == (B, N, h, attn_num),
                 lambda: f"attn_out shape {tuple(attn_out.shape)} != {(B, N, h, attn_num)}")
    torch._check(output.dtype == q.dtype and attn_out.dtype == q.dtype, lambda: "output dtypes must match q")
    torch._check(output.device == q.device and attn_out.device == q.device, lambda: "output devices must match q")
    return None


@torch.library.custom_op("matchattention_amd::match_attention", mutates_args=())
def match_attention(max_offset: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                    H: int, W: int, win_r: List[int], attn_num: int, attn_type: str,
                    scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Functional form (allocates its outputs); this is the differentiable entry."""
    B, N, C, h = _check_inputs(max_offset, q, k, v, H, W, win_r, attn_num, attn_type)
    output = torch.empty_like(q)
    attn_out = q.new_empty((B, N, h, attn_num))
    fused_forward(max_offset, q, k, v, output, attn_out, H, W, win_r, attn_num, attn_type, scale)
    return output, attn_out


@match_attention.register_fake
def _(max_offset, q, k, v, H, W, win_r, attn_num, attn_type, scale):
    B, N, C = q.shape
    return torch.empty_like(q), q.new_empty((B, N, max_offset.size(2), attn_num))


@torch.library.custom_op("matchattention_amd::match_attention_backward", mutates_args=())
def match_attention_backward(max_offset: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                             d_out: torch.Tensor, d_attn: Optional[torch.Tensor], H: int, W: int,
                             win_r: List[int], scale: float
                             ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """(dq, dk, dv, d_max_offset) for upstream gradients d_out and (optionally) d_attn."""
    attn_num = (2 * win_r[0] + 2) * (2 * win_r[1] + 2)
    B, N, C, h = _check_inputs(max_offset, q, k, v, H, W, win_r, attn_num, "l1_norm")
    d_out = d_out.contiguous()
    if d_attn is not None:
        d_attn = d_attn.contiguous()
    lib = _cabi.load()
    dt = _DTYPES[q.dtype]
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    dmo = torch.empty_like(max_offset)
    ws_bytes = lib.matchattn_backward_workspace_bytes(B, H, W, C, h, int(win_r[0]), int(win_r[1]), dt)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    with torch.cuda.device(q.device):
        _cabi.check(lib.matchattn_backward(
            max_offset.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(),
            d_attn.data_ptr() if d_attn is not None else None,
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dmo.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes,
            B, H, W, C, h, int(win_r[0]), int(win_r[1]), float(scale), dt, _stream_ptr(q.device)))
    return dq, dk, dv, dmo


@match_attention_backward.register_fake
def _(max_offset, q, k, v, d_out, d_attn, H, W, win_r, scale):
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(max_offset)


def _setup_context(ctx, inputs, output):
    max_offset, q, k, v, H, W, win_r, attn_num, attn_type, scale = inputs
    ctx.save_for_backward(max_offset, q, k, v)
    ctx.geom = (H, W, list(win_r), scale)


def _backward(ctx, d_out, d_attn):
    max_offset, q, k, v = ctx.saved_tensors
    H, W, win_r, scale = ctx.geom
    if d_out is None:
        d_out = torch.zeros_like(q)
    dq, dk, dv, dmo = match_attention_backward(max_offset, q, k, v, d_out, d_attn, H, W, win_r, scale)
    return dmo, dq, dk, dv, None, None, None, None, None, None


match_attention.register_autograd(_backward, setup_context=_setup_context)


class MF_FusedForwardOps(nn.Module):
    """Drop-in for the reference's ``MF_FusedForwardOps`` (models/match_former_ops.py:65-121):
    same call signature and return values; parameter-free.  When any input requires grad
    the differentiable functional op is used, otherwise the in-place one."""

    def __init__(self):
        super().__init__()

    def forward(self, max_offset: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                H: int, W: int, win_r: List[int], attn_num: int, attn_type: str = 'l1_norm',
                scale: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
        if torch.is_grad_enabled() and any(t.requires_grad for t in (max_offset, q, k, v)):
            return match_attention(max_offset, q, k, v, H, W, list(win_r), attn_num, attn_type, float(scale))
        B, N, C = q.shape
        h = max_offset.size(2)
        output = torch.empty_like(v)
        attn_out = q.new_empty([B, N, h, attn_num])
        fused_forward_ops(max_offset, q, k, v, output, attn_out, H, W, list(win_r), attn_num, attn_type, float(scale))
        return output, attn_out


@torch.library.custom_op("matchattention_amd::fused_module_step", mutates_args=())
def fused_module_step(position: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                      gate: Optional[torch.Tensor], H: int, W: int, win_r: List[int], num_head: int, scale: float,
                      relative: bool, concat: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Opaque (to torch.compile) form of ``fused_module_forward``: returns (buffer [B,N,C+h*M], empty) with
    ``concat``, else (out [B,N,C], attn [B,N,h,M])."""
    h = int(num_head)
    attn_num = (2 * win_r[0] + 2) * (2 * win_r[1] + 2)
    if position.dim() != 4 or position.size(-1) != 2 or position.size(2) not in ((1, h) if relative else (h,)):
        raise ValueError(f"position must be [B,N,{'1 or ' if relative else ''}{h},2], got {tuple(position.shape)}")
    B, N, C, _ = _check_inputs(position, q, k, v, H, W, win_r, attn_num, "l1_norm")
    if C % h:
        raise ValueError(f"C={C} is not a multiple of num_head={h}")
    if gate is not None and (gate.shape != q.shape or gate.dtype != q.dtype or gate.device != q.device or not gate.is_contiguous()):
        raise ValueError("gate must match q (shape, dtype, device) and be contiguous")
    lib = _cabi.load()
    dt = _DTYPES[q.dtype]
    if concat:
        width = C + h * attn_num
        first = q.new_empty((B, N, width))
        second = q.new_empty((0,))
        out_ptr, attn_ptr = first.data_ptr(), first.data_ptr() + C * first.element_size()
        out_stride = attn_stride = width
    else:
        first = torch.empty_like(q)
        second = q.new_empty((B, N, h, attn_num))
        out_ptr, attn_ptr, out_stride, attn_stride = first.data_ptr(), second.data_ptr(), 0, 0
    with torch.cuda.device(q.device):
        ws_bytes = lib.matchattn_forward_fused_workspace_bytes(B, H, W, C, h, int(win_r[0]), int(win_r[1]), dt)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
        _cabi.check(lib.matchattn_forward_fused(
            position.data_ptr(), position.size(2) if relative else 0,
            q.data_ptr(), k.data_ptr(), v.data_ptr(), gate.data_ptr() if gate is not None else None,
            out_ptr, out_stride, attn_ptr, attn_stride,
            ws.data_ptr() if ws is not None else None, ws_bytes,
            B, H, W, C, h, int(win_r[0]), int(win_r[1]), float(scale), dt, _stream_ptr(q.device)))
    return first, second


@fused_module_step.register_fake
def _(position, q, k, v, gate, H, W, win_r, num_head, scale, relative, concat):
    B, N, C = q.shape
    M = (2 * win_r[0] + 2) * (2 * win_r[1] + 2)
    if concat:
        return q.new_empty((B, N, C + num_head * M)), q.new_empty((0,))
    return torch.empty_like(q), q.new_empty((B, N, num_head, M))


def _sampling_positions(position: torch.Tensor, H: int, W: int, r: int, h: int, relative: bool):
    """What the fused call computes before the operator, in torch ops: pixel grid add and clamp with the bounds
    rounded to the tensor dtype (models/attention_blocks.py:149-151, 162-163, 45-59).  Returns the sampling
    positions [B,N,h,2] and the mask of the components the clamp let through (its gradient)."""
    B, N = position.shape[:2]
    if not relative:
        return position, None
    dt, dev = position.dtype, position.device
    ys, xs = torch.meshgrid(torch.arange(H, device=dev, dtype=dt), torch.arange(W, device=dev, dtype=dt), indexing="ij")
    grid = torch.stack((xs, ys), -1).view(1, N, 1, 2)
    raw = (position + grid).expand(B, N, h, 2)
    lo = torch.full((), float(r), dtype=dt, device=dev)
    hi = torch.stack((torch.full((), W - 1 - r - 1e-3, dtype=dt, device=dev), torch.full((), H - 1 - r - 1e-3, dtype=dt, device=dev)))
    mo = torch.minimum(torch.maximum(raw, lo), hi)
    return mo.contiguous(), (raw >= lo) & (raw <= hi)


def _fused_setup_context(ctx, inputs, output):
    position, q, k, v, gate, H, W, win_r, num_head, scale, relative, concat = inputs
    ctx.save_for_backward(position, q, k, v, gate)
    ctx.cfg = (H, W, list(win_r), int(num_head), float(scale), bool(relative), bool(concat))


def _fused_backward(ctx, d_first, d_second):
    """Gradient of the fused module step: the column ranges of the projection input are split back into the
    gradient of the gated output and of the attention weights, the gate takes d(gate * out) -- `out` is recomputed
    by one forward call, the fused forward stores only the product --, the operator's backward kernel does the
    rest, and the clamp's mask and the broadcast over heads turn d max_offset into d position."""
    position, q, k, v, gate = ctx.saved_tensors
    H, W, win_r, h, scale, relative, concat = ctx.cfg
    B, N, C = q.shape
    M = (2 * win_r[0] + 2) * (2 * win_r[1] + 2)
    mo, passed = _sampling_positions(position, H, W, win_r[0], h, relative)
    if concat:
        d_res = None if d_first is None else d_first[..., :C]
        d_attn = None if d_first is None else d_first[..., C:].reshape(B, N, h, M).contiguous()
    else:
        d_res, d_attn = d_first, d_second
    if d_res is None:
        d_res = torch.zeros_like(q)
    d_gate = None
    if gate is not None:
        out = torch.empty_like(q)
        attn = q.new_empty((B, N, h, M))
        fused_forward_ops(mo, q, k, v, out, attn, H, W, win_r, M, "l1_norm", scale)
        d_gate = d_res * out
        d_res = d_res * gate
    dq, dk, dv, dmo = match_attention_backward(mo, q, k, v, d_res.contiguous(), d_attn, H, W, win_r, scale)
    if relative:
        dmo = dmo * passed
        if position.size(2) == 1 and h > 1:
            dmo = dmo.sum(2, keepdim=True)
    return dmo, dq, dk, dv, d_gate, None, None, None, None, None, None, None


fused_module_step.register_autograd(_fused_backward, setup_context=_fused_setup_context)


def fused_module_forward(position: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                         H: int, W: int, win_r: List[int], num_head: int, scale: float,
                         gate: Optional[torch.Tensor] = None, relative: bool = True, concat: bool = False):
    """The operator together with the elementwise steps the attention module runs either side of it, in
    one native call (``matchattn_forward_fused`` of the C ABI); differentiable.

    ``position`` [B,N,hp,2]: with ``relative`` the positions relative to each query pixel, hp = num_head or
    1 (shared by all heads) -- the pixel coordinates are added and the sum clamped inside the call, as
    models/attention_blocks.py:149-151 / 162-163 and :45-59 do; otherwise the clamped sampling positions
    (hp = num_head).  ``gate`` [B,N,C] multiplies the output (:96).  With ``concat`` the result is the single
    [B,N,C + h*attn_num] tensor the cross-attention projection consumes (:97-98); otherwise (out, attn).
    Under autograd the backward recomputes the ungated output with one forward call and runs the operator's
    backward kernel; gradients flow to position (through the clamp's mask), q, k, v and gate."""
    first, second = fused_module_step(position, q, k, v, gate, H, W, list(win_r), int(num_head), float(scale),
                                      bool(relative), bool(concat))
    return first if concat else (first, second)

"""The MatchAttention operator in plain PyTorch ops: the `mat_impl='pytorch'` choice beside `'hip'`.

Same definition as the reference's PyTorch path (models/mat_pytorch_impl.py:3-178 sequenced by
models/attention_blocks.py:82-91) -- floor, bilinear corner weights, gathered negative-L1 logits, scale, one softmax
per (2r+1)^2 sub-window merged with the corner weights, aggregation -- with the same rounding points in 16-bit
types, but walked tap by tap: the (2r+2)^2 taps are gathered one at a time, so the largest temporary is [B,N,C]
instead of [B,N,h,M,Ch] (9.6 GB at 544x960, C=256, r=2).  Runs on any device, differentiable by autograd.
It is what `--mat_impl pytorch` selects in `matchattention_amd.run_img` and what the end-to-end baseline leg of
the benchmark times; the HIP path never calls it.
"""
from typing import Sequence, Tuple

import torch


def _corner_weights(max_offset: torch.Tensor) -> Tuple[torch.Tensor, ...]:
    """(nw, ne, sw, se) weights of the four integer-centre windows, in the tensor dtype
    (models/mat_pytorch_impl.py:3-27)."""
    fx = max_offset[..., 0] - torch.floor(max_offset[..., 0])
    fy = max_offset[..., 1] - torch.floor(max_offset[..., 1])
    gx, gy = 1 - fx, 1 - fy
    return gx * gy, fx * gy, gx * fy, fx * fy


def match_attention_torch(max_offset: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                          H: int, W: int, win_r: Sequence[int], scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """max_offset [B,N,h,2] (x, y; already clamped by the module), q/k/v [B,N,C] -> out [B,N,C], attn [B,N,h,M]."""
    B, N, C = q.shape
    h = max_offset.size(2)
    rx, ry = int(win_r[0]), int(win_r[1])
    nx, ny = 2 * rx + 2, 2 * ry + 2
    q4, k4, v4 = (t.view(B, N, h, C // h) for t in (q, k, v))
    centre = torch.floor(max_offset).long()
    bsel = torch.arange(B, device=q.device).view(B, 1, 1)
    hsel = torch.arange(h, device=q.device).view(1, 1, h)
    # per-tap replicate clamp (models/mat_pytorch_impl.py:58-59), taps row by row (y-major, :45-48)
    cols = [(centre[..., 0] + (i - rx)).clamp(0, W - 1) for i in range(nx)]
    rows = [(centre[..., 1] + (j - ry)).clamp(0, H - 1) * W for j in range(ny)]
    index = [[rows[j] + cols[i] for i in range(nx)] for j in range(ny)]            # [ny][nx] of [B,N,h]
    logits = torch.stack([torch.stack([-(q4 - k4[bsel, index[j][i], hsel]).abs().sum(-1) for i in range(nx)], -1)
                          for j in range(ny)], -2)                                   # [B,N,h,ny,nx]
    logits = logits * scale
    # BilinearSoftmax: independent softmax over the four sub-windows, merged in the order nw, ne, sw, se (:78-165)
    attn = torch.zeros_like(logits)
    for wgt, (dx, dy) in zip(_corner_weights(max_offset), ((0, 0), (1, 0), (0, 1), (1, 1))):
        sub = logits[..., dy:dy + ny - 1, dx:dx + nx - 1]
        p = sub.reshape(B, N, h, -1).softmax(-1).view_as(sub)
        attn[..., dy:dy + ny - 1, dx:dx + nx - 1] += wgt[..., None, None] * p
    # aggregation: products in the tensor dtype, summed over the window in fp32 as torch sums half tensors (:167-178)
    acc = torch.zeros(B, N, h, C // h, dtype=torch.float32 if q.dtype != torch.float64 else torch.float64, device=q.device)
    for j in range(ny):
        for i in range(nx):
            acc = acc + (attn[..., j, i, None] * v4[bsel, index[j][i], hsel]).to(acc.dtype)
    return acc.to(q.dtype).reshape(B, N, C), attn.reshape(B, N, h, ny * nx)


def attend_torch(max_offset, q, k, v, H, W, win_r, attn_num, scale):
    """The harness's operator signature (matchattention_amd.stereo_harness) on the PyTorch definition."""
    assert attn_num == (2 * win_r[0] + 2) * (2 * win_r[1] + 2)
    return match_attention_torch(max_offset, q, k, v, H, W, win_r, scale)

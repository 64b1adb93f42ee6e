"""MatchStereo harness: the callers on either side of the MatchAttention operator.

A compact PyTorch restatement of the network that drives the operator in the reference
(architecture after models/match_stereo.py:11-130, models/attention_blocks.py:12-210,
models/convformer.py:65-358, models/cost_volume.py:8-179, models/common.py:5-48), written
to measure the operator end to end: same tensor shapes into the operator, same data flow
around it, random-init weights from a seed.  It is not a product model: there is no
checkpoint loading and only the stereo branch of the initial correlation is present.

The operator is injected: ``attend(max_offset, q, k, v, H, W, win_r, attn_num, scale) ->
(out [B,N,C], attn [B,N,h,M])``.  ``matchattention_amd.MF_FusedForwardOps`` is the 'hip'
choice; tests plug a PyTorch definition for the 'pytorch' one.  Optionally a second callable,
``fused(position, q, k, v, H, W, win_r, num_head, scale, gate=, relative=True, concat=)``
(``matchattention_amd.fused_module_forward``), takes over the elementwise steps either side of the
operator: the pixel-coordinate add and clamp before it, the gate and the concatenation after it.
"""
import math
from typing import Callable, List, Optional, Sequence

import torch
import torch.nn as nn
import torch.nn.functional as F

VARIANTS = {"tiny": [32, 64, 128, 160], "small": [64, 128, 160, 320], "base": [128, 256, 320, 512]}


def pixel_grid(B, H, W, dtype, device):
    """(x, y) coordinates of every pixel, [B,H,W,2] (utils/utils.py:31-36)."""
    ys, xs = torch.meshgrid(torch.arange(H, device=device, dtype=dtype),
                            torch.arange(W, device=device, dtype=dtype), indexing="ij")
    return torch.stack((xs, ys), -1).expand(B, H, W, 2)


def depthwise_nhwc(conv: nn.Conv2d, x: torch.Tensor) -> torch.Tensor:
    """Depthwise 3x3 convolution of a channels-last activation [B,H,W,C] -> [B,H,W,C].  MIOpen has no tuned
    fp16 solver for these on channels-last views and falls back to its generic kernel, whose cost barely depends
    on the map size (0.25-0.3 ms per call on an MI355X); below 1/4 scale an explicit NCHW copy and the NCHW
    solver are 2-4x faster (measured: 92x160x128 0.28 -> 0.16 ms, 46x80x256 0.25 -> 0.07 ms)."""
    t = x.permute(0, 3, 1, 2)
    if x.shape[1] * x.shape[2] <= 128 * 192:
        t = t.contiguous()
    return conv(t).permute(0, 2, 3, 1)


class ScaleOnlyLayerNorm(nn.Module):
    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        return F.layer_norm(x, self.weight.shape, self.weight, None, self.eps)


# ---------------------------------------------------------------- encoder (ConvFormer) ----
class MixerBlock(nn.Module):
    """x + SepConv(norm(x)); x + MLP(norm(x)), channels-last (convformer.py:136-258)."""

    def __init__(self, dim, has_res_scale):
        super().__init__()
        self.norm_a, self.norm_b = ScaleOnlyLayerNorm(dim, 1e-6), ScaleOnlyLayerNorm(dim, 1e-6)
        self.pw_in = nn.Linear(dim, 2 * dim, bias=False)
        self.dw = nn.Conv2d(2 * dim, 2 * dim, 3, padding=1, groups=2 * dim, bias=False)
        self.pw_out = nn.Linear(2 * dim, dim, bias=False)
        self.fc_in = nn.Linear(dim, 2 * dim, bias=False)
        self.fc_out = nn.Linear(2 * dim, dim, bias=False)
        # the reference creates residual scales for the last two stages and never applies them
        # (convformer.py:215-225,228-231); kept only so that the parameter count can be compared
        self.unused_res_scale = nn.Parameter(torch.ones(2, dim)) if has_res_scale else None

    def forward(self, x):
        x = x + self.pw_out(depthwise_nhwc(self.dw, F.gelu(self.pw_in(self.norm_a(x)))))
        return x + self.fc_out(F.gelu(self.fc_in(self.norm_b(x))))


class Encoder(nn.Module):
    def __init__(self, dims: Sequence[int], depths=(2, 2, 6, 2)):
        super().__init__()
        self.dims = list(dims)
        d0 = dims[0]
        self.stem = nn.Sequential(nn.Conv2d(3, d0 // 2, 3, 2, 1), nn.InstanceNorm2d(d0 // 2), nn.GELU(),
                                  nn.Conv2d(d0 // 2, d0, 3, 2, 1), nn.InstanceNorm2d(d0), nn.GELU())
        self.down_norm = nn.ModuleList([ScaleOnlyLayerNorm(dims[i], 1e-6) for i in range(3)])
        self.down_conv = nn.ModuleList([nn.Conv2d(dims[i], dims[i + 1], 3, 2, 1) for i in range(3)])
        self.stages = nn.ModuleList([nn.ModuleList([MixerBlock(dims[i], i >= 2) for _ in range(depths[i])])
                                     for i in range(4)])
        self.unused_head = nn.Linear(dims[-1], 1000)   # classification head of the backbone, never called

    def forward(self, img):
        feats = []
        x = self.stem(img).permute(0, 2, 3, 1).contiguous()
        for i in range(4):
            if i > 0:
                x = self.down_conv[i - 1](self.down_norm[i - 1](x).permute(0, 3, 1, 2)).permute(0, 2, 3, 1).contiguous()
            for blk in self.stages[i]:
                x = blk(x)
            feats.append(x)
        return feats   # 1/4, 1/8, 1/16, 1/32, each [B,H,W,C]


# -------------------------------------------------------- initial correlation (stereo) ----
class RowCorrelation(nn.Module):
    """All-pairs correlation along rows at 1/32 scale -> initial disparity for both views
    (cost_volume.py:8-54,123-179).  The volume is built with one gather instead of the
    reference's per-disparity Python loops; values are the same."""

    def __init__(self, dim):
        super().__init__()
        self.norm = ScaleOnlyLayerNorm(dim)
        self.q = nn.Linear(dim, dim, bias=False)
        self.k = nn.Linear(dim, dim, bias=False)
        self.scale = dim ** -0.5

    def forward(self, x):
        x = self.norm(x)
        left, right = x.chunk(2, 0)
        corr = torch.matmul(self.q(left), self.k(right).transpose(-2, -1)) * self.scale   # [B,H,W(left),W(right)]
        B, H, W, _ = corr.shape
        d = torch.arange(W, device=x.device).view(W, 1)
        w = torch.arange(W, device=x.device).view(1, W)
        # left view: volume[d, w] = corr[w, w-d] for w >= d; right view: corr[w+d, w] for w+d < W; else 0
        il = (w - d).clamp(min=0).expand(B, H, W, W)                       # [.., d, w] -> right column
        vol_l = torch.gather(corr.unsqueeze(2).expand(B, H, W, W, W), 4, il.unsqueeze(-1)).squeeze(-1)
        vol_l = torch.where((w >= d), vol_l, torch.zeros_like(vol_l))      # [B,H,d,w]
        corr_t = corr.transpose(-2, -1)                                     # [B,H,W(right),W(left)]
        ir = (w + d).clamp(max=W - 1).expand(B, H, W, W)
        vol_r = torch.gather(corr_t.unsqueeze(2).expand(B, H, W, W, W), 4, ir.unsqueeze(-1)).squeeze(-1)
        vol_r = torch.where((w + d <= W - 1), vol_r, torch.zeros_like(vol_r))
        vol = torch.cat((vol_l, vol_r), 0).permute(0, 2, 1, 3)              # [2B, D, H, W]
        vol = F.softmax(vol, dim=1).to(vol.dtype)
        # out-of-view columns copy the nearest in-view probability of the same disparity
        edge_l = torch.gather(vol[:B], 3, d.view(1, W, 1, 1).expand(B, W, H, 1))           # value at w = d
        edge_r = torch.gather(vol[B:], 3, (W - 1 - d).view(1, W, 1, 1).expand(B, W, H, 1)) # value at w = W-1-d
        wv, dv = w.view(1, 1, 1, W), d.view(1, W, 1, 1)
        vol = torch.cat((torch.where(wv < dv, edge_l, vol[:B]), torch.where(wv > W - 1 - dv, edge_r, vol[B:])), 0)
        return self._soft_argmax(vol)

    @staticmethod
    def _soft_argmax(vol, k=5):
        B2, D, H, W = vol.shape
        r = k // 2
        blur = F.avg_pool1d(vol.permute(0, 2, 3, 1).reshape(B2, H * W, D), k, 1, r).view(B2, H, W, D)
        peak = blur.argmax(-1).clamp(r, D - 1 - r)                                     # [2B,H,W]
        idx = (peak.unsqueeze(-1) + torch.arange(-r, r + 1, device=vol.device)).clamp(0, D - 1)   # [2B,H,W,k]
        p = torch.gather(vol.permute(0, 2, 3, 1), 3, idx)
        p = torch.where(p < 1.0 / D, torch.zeros_like(p), p)
        s = p.sum(-1, keepdim=True).clamp(min=torch.finfo(p.dtype).tiny)
        disp = ((p / s) * idx.to(p.dtype)).sum(-1, keepdim=True).to(p.dtype)
        sign = torch.ones(B2, 1, 1, 1, device=vol.device, dtype=p.dtype)
        sign[: B2 // 2] = -1                                                          # left view: negative x-flow
        return torch.cat((disp * sign, torch.zeros_like(disp)), -1).contiguous()      # [2B,H,W,2]


# ------------------------------------------------------------------- attention blocks ----
class ConvGLU(nn.Module):
    def __init__(self, dim, ratio=2):
        super().__init__()
        hid = int(ratio * dim)
        self.fc1 = nn.Linear(dim, 2 * hid)
        self.dw = nn.Conv2d(hid, hid, 3, padding=1, groups=hid)
        self.fc2 = nn.Linear(hid, dim)

    def forward(self, x):
        a, gate = self.fc1(x).chunk(2, -1)
        a = F.gelu(depthwise_nhwc(self.dw, a).contiguous())
        return self.fc2(a * gate)


class MatchAttention(nn.Module):
    """Projections around the operator (attention_blocks.py:12-101)."""

    def __init__(self, attend, dim, r, heads, head_dim, cross, fused=None):
        super().__init__()
        self.attend, self.fused, self.r, self.h, self.cross = attend, fused, r, heads, cross
        self.scale = head_dim ** -0.5
        self.M = (2 * r + 2) ** 2
        inner = heads * head_dim
        emb = dim if cross else dim + 1                     # self-attention sees the consistency mask too
        self.q, self.k, self.v = (nn.Linear(emb, inner, bias=False) for _ in range(3))
        if cross:
            self.g = nn.Linear(emb, inner, bias=False)
            self.proj = nn.Linear(inner + heads * self.M, dim, bias=False)
        else:
            self.proj = nn.Linear(inner, dim, bias=False)

    def forward(self, x, rel, noc_mask=None):
        """rel [B,N,hp,2]: sampling positions relative to each query pixel, hp = heads, or 1 when all heads
        share one (the layer adds the pixel grid itself in the reference, attention_blocks.py:149-151,162-163)."""
        B, H, W, _ = x.shape
        N, r = H * W, self.r
        assert 2 * r + 2 <= min(H, W)
        x = x.reshape(B, N, -1)
        if self.cross:
            a, b = x.chunk(2, 0)
            ref, tgt = x, torch.cat((b, a), 0)
            gate = F.silu(self.g(ref))
        else:
            ref = tgt = torch.cat((x, noc_mask.reshape(B, N, 1)), -1)
        q, k, v = self.q(ref).contiguous(), self.k(tgt).contiguous(), self.v(tgt).contiguous()
        if self.fused is not None:
            res = self.fused(rel.contiguous(), q, k, v, H, W, [r, r], self.h, self.scale,
                             gate=gate.contiguous() if self.cross else None, relative=True, concat=self.cross)
            return self.proj(res if self.cross else res[0]).view(B, H, W, -1)
        max_offset = (rel + pixel_grid(B, H, W, rel.dtype, rel.device).reshape(B, N, 1, 2)).expand(B, N, self.h, 2)
        # clamp with the bounds rounded to the tensor dtype as the reference does (:45-59); the bounds are filled on
        # the device (no host-to-device copy, no host read-back: the forward stays capturable in a HIP graph and
        # traces under torch.compile without a graph break)
        dt, dev = max_offset.dtype, max_offset.device
        lo = torch.full((), float(r), dtype=dt, device=dev)
        hi_x = torch.full((), W - 1 - r - 1e-3, dtype=dt, device=dev)
        hi_y = torch.full((), H - 1 - r - 1e-3, dtype=dt, device=dev)
        mx = torch.clamp(max_offset[..., 0:1], min=lo, max=hi_x)
        my = torch.clamp(max_offset[..., 1:2], min=lo, max=hi_y)
        out, attn = self.attend(torch.cat((mx, my), -1).contiguous(), q, k, v, H, W, [r, r], self.M, self.scale)
        if self.cross:
            out = torch.cat((gate * out, attn.reshape(B, N, -1)), -1)
        return self.proj(out).view(B, H, W, -1)


class MatchLayer(nn.Module):
    """self-attention -> cross-attention -> ConvGLU with the field carried in the features
    (attention_blocks.py:104-175)."""

    def __init__(self, attend, dim, r, heads, head_dim, fused=None):
        super().__init__()
        self.h = heads
        self.self_attn = MatchAttention(attend, dim + 2 + 2 * heads, r, heads, head_dim, cross=False, fused=fused)
        self.cross_attn = MatchAttention(attend, dim + 2, r, heads, head_dim, cross=True, fused=fused)
        self.n0, self.n1, self.n2 = (ScaleOnlyLayerNorm(d) for d in (dim + 2 + 2 * heads, dim + 2, dim))
        self.mlp = ConvGLU(dim)
        self.field_scale = nn.Parameter(0.1 * torch.ones(1, 1, 1, 2))

    @staticmethod
    def consistency(field, A=2):
        B, H, W, _ = field.shape
        pos = field + pixel_grid(B, H, W, field.dtype, field.device)
        other = torch.cat(field.chunk(2, 0)[::-1], 0).permute(0, 3, 1, 2)
        grid = torch.stack((2 * pos[..., 0] / (W - 1) - 1, 2 * pos[..., 1] / (H - 1) - 1), -1)
        warped = F.grid_sample(other, grid, mode="bilinear", align_corners=True).permute(0, 2, 3, 1)
        return ((field + warped).abs().sum(-1, keepdim=True) < A).to(field.dtype)

    def forward(self, x, self_rpos, field, stereo=True):
        B, H, W, _ = x.shape
        h, fs = self.h, self.field_scale.to(field.dtype)
        noc = self.consistency(field.detach())
        x = torch.cat((x, field * fs, self_rpos), -1)
        x = x + self.self_attn(self.n0(x), self_rpos.view(B, H * W, h, 2), noc)
        self_rpos, x = x[..., -2 * h:].contiguous(), x[..., :-2 * h].contiguous()
        if stereo:
            x[..., -1] = 0
        field = x[..., -2:] / fs
        x = x + self.cross_attn(self.n1(x), field.reshape(B, H * W, 1, 2))
        if stereo:
            x[..., -1] = 0
        field = x[..., -2:] / fs
        x = x[..., :-2].contiguous()
        return x + self.mlp(self.n2(x)), self_rpos, field.contiguous()


class UpFuse(nn.Module):
    def __init__(self, cin, cout):
        super().__init__()
        self.up = nn.ConvTranspose2d(cin, cout, 2, 2)
        self.mix = nn.Sequential(nn.Conv2d(2 * cout, cout, 1), nn.ReLU(inplace=True), nn.Conv2d(cout, cout, 3, padding=1))

    def forward(self, coarse, fine):
        c = self.up(coarse.permute(0, 3, 1, 2))
        return self.mix(torch.cat((fine.permute(0, 3, 1, 2), c), 1)).permute(0, 2, 3, 1).contiguous()


def convex_upsample(field, mask, f):
    """RAFT-style convex combination of the 3x3 neighbourhood (match_stereo.py:73-84)."""
    B, H, W, D = field.shape
    m = torch.softmax(mask.view(B, 1, 9, f, f, H, W), 2).to(mask.dtype)
    nb = F.unfold(field.permute(0, 3, 1, 2) * f, 3, padding=1).view(B, D, 9, 1, 1, H, W)
    up = (m * nb).sum(2).to(mask.dtype)                       # [B,D,f,f,H,W]
    return up.permute(0, 4, 2, 5, 3, 1).reshape(B, f * H, f * W, D).contiguous()


class MatchStereoHarness(nn.Module):
    def __init__(self, attend: Callable, variant="tiny", win_rs=(2, 2, 1, 1), depths=(8, 8, 8, 2), heads=(4, 4, 4, 4),
                 seed: Optional[int] = 0, fused: Optional[Callable] = None):
        super().__init__()
        self.encoder = Encoder(VARIANTS[variant])
        ch = self.encoder.dims[::-1]                           # 1/32 ... 1/4
        self.ch = ch
        self.init_corr = RowCorrelation(ch[0])
        self.fuse = nn.ModuleList([UpFuse(ch[i - 1], ch[i]) for i in range(1, 4)])
        self.masks = nn.ModuleList([nn.Sequential(nn.Conv2d(ch[i - 1], ch[i - 1], 3, padding=1), nn.ReLU(inplace=True),
                                                  nn.Conv2d(ch[i - 1], 4 * 9, 1)) for i in range(1, 4)])
        self.final_mask = nn.Sequential(nn.Conv2d(ch[-1], 2 * ch[-1], 3, padding=1), nn.ReLU(inplace=True),
                                        nn.Conv2d(2 * ch[-1], 16 * 9, 1))
        self.blocks = nn.ModuleList([nn.ModuleList([MatchLayer(attend, ch[i], win_rs[i], heads[i], ch[i] // heads[i], fused)
                                                    for _ in range(depths[i])]) for i in range(4)])
        self.heads = heads
        if seed is not None:
            self.reset(seed)

    def reset(self, seed):
        """trunc_normal(std=0.02) on every Conv2d / Linear weight, zero bias (match_stereo.py:66-70)."""
        g = torch.Generator().manual_seed(seed)
        for m in self.modules():
            if isinstance(m, (nn.Conv2d, nn.Linear)):
                with torch.no_grad():
                    w = torch.empty(m.weight.shape)
                    nn.init.trunc_normal_(w, std=0.02, generator=g)
                    m.weight.copy_(w)
                    if m.bias is not None:
                        m.bias.zero_()

    def forward(self, left, right, init_field=None, return_rpos=False):
        """left, right: [B,3,H,W] in 0..255, H and W multiples of 32.  Returns the full-resolution
        field [2B,H,W,2] (x-disparity of the left view in the first half, of the right view in the
        second) and the list of per-scale fields; with `return_rpos` also the self-attention's relative
        positions at 1/4 scale [2B,H/4,W/4,2].  `init_field` [2B,H/32,W/32,2] replaces the initial
        correlation (the low-resolution initialisation of the reference's script, match_stereo.py:96-103)."""
        x = torch.cat((2 * (left / 255.0) - 1, 2 * (right / 255.0) - 1), 0).contiguous()
        feats = self.encoder(x)[::-1]
        fields = []
        for i in range(4):
            if i == 0:
                field = self.init_corr(feats[0]) if init_field is None else init_field.to(feats[0].dtype).clone()
                rpos = torch.zeros_like(field)
            else:
                feats[i] = self.fuse[i - 1](feats[i - 1], feats[i])
                mask = self.masks[i - 1](feats[i - 1].permute(0, 3, 1, 2))
                rpos, field = convex_upsample(rpos, mask, 2), convex_upsample(field, mask, 2)
            h = self.heads[i]
            rp = rpos.repeat(1, 1, 1, h)
            f = feats[i]
            for layer in self.blocks[i]:
                f, rp, field = layer(f, rp, field)
            feats[i] = f
            B2, H, W, _ = f.shape
            rpos = rp.view(B2, H, W, h, 2).mean(-2)
            fields.append(field)
        full = convex_upsample(field, self.final_mask(feats[-1].permute(0, 3, 1, 2)), 4)
        if return_rpos:
            return full, fields, rpos
        return full, fields

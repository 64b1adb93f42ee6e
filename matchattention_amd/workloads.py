"""Synthetic operator workloads: the shapes and offset distributions the benchmark and
the full-size tests use.  Inputs are i.i.d. per pixel as specified (no spatial coherence),
which is the hardest case for tap reuse; `smooth=True` blurs the offset field instead (same amplitude, correlated over
about 8 px: still several pixels of offset change per pixel), `smooth="scene"` makes a stereo field as a scene gives it
(slanted surfaces with discontinuities: a fraction of a pixel of change per pixel).  """
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    dtype: torch.dtype
    B: int
    H: int
    W: int
    C: int
    h: int
    r: int
    offsets: str          # "stereo:<max_disp>" | "gauss:<sigma>"
    per_head: bool        # self-attention: one offset per head; cross: one shared by all heads
    backward: bool

    @property
    def N(self):
        return self.H * self.W

    @property
    def M(self):
        return (2 * self.r + 2) ** 2

    @property
    def scale(self):
        return (self.C // self.h) ** -0.5

    def forward_bytes(self) -> int:
        """Algorithmic bytes of one forward: read q,k,v + write out (4C), read max_offset (2h),
        write attn (hM), per query pixel."""
        s = torch.finfo(self.dtype).bits // 8
        return self.B * self.N * s * (4 * self.C + 2 * self.h + self.h * self.M)

    def backward_bytes(self, with_dattn: bool) -> int:
        """read q,k,v,dOut + write dq,dk,dv (7C), read dAttn (hM, cross only), read offsets +
        write their gradient (4h), per query pixel."""
        s = torch.finfo(self.dtype).bits // 8
        return self.B * self.N * s * (7 * self.C + (self.h * self.M if with_dattn else 0) + 4 * self.h)


WORKLOADS = {
    "cfg1_cross": Workload("cfg1_cross", torch.float32, 1, 104, 208, 128, 4, 1, "stereo:40", False, False),
    "cfg2_cross": Workload("cfg2_cross", torch.float16, 1, 384, 384, 128, 4, 1, "stereo:96", False, True),
    "cfg3_cross": Workload("cfg3_cross", torch.float16, 1, 544, 960, 256, 8, 2, "stereo:240", False, False),
    "cfg3_self": Workload("cfg3_self", torch.float16, 1, 544, 960, 256, 8, 2, "gauss:2", True, False),
    "cfg4_cross": Workload("cfg4_cross", torch.float16, 2, 384, 384, 256, 8, 2, "gauss:24", False, True),
    "cfg4_self": Workload("cfg4_self", torch.float16, 2, 384, 384, 256, 8, 2, "gauss:24", True, True),
}


# The operator calls of one MatchStereo-T frame at 1536 x 1536 (reference models/match_stereo.py:13-15,24 and
# models/convformer.py:353: four levels at 1/32 .. 1/4 of the padded input, both views in the batch, 4 heads), each as
# the cross-attention call (one position shared by the heads, attention gradient present) and the self-attention call
# (a position per head).  The fields are spatially smooth, as a model's are.
MODEL_SHAPES = {
    f"tiny1536_{hw}x{hw}_c{c}_r{r}_{kind}": Workload(f"tiny1536_{hw}x{hw}_c{c}_r{r}_{kind}", torch.float16, 2, hw, hw, c, 4, r,
                                                    f"stereo:{hw // 4}" if kind == "cross" else "gauss:2", kind == "self", True)
    for hw, c, r in ((48, 160, 2), (96, 128, 2), (192, 64, 1), (384, 32, 1)) for kind in ("cross", "self")
}

# The same frame through the `base` variant in the precision the reference's script defaults to (run_img.py:195-196,
# models/convformer.py:372-380: channels 128, 256, 320, 512 from the finest level; fp32): heads of 32, 64, 80 and 128
# channels.
MODEL_SHAPES_BASE_F32 = {
    f"base1536_{hw}x{hw}_c{c}_r{r}_{kind}": Workload(f"base1536_{hw}x{hw}_c{c}_r{r}_{kind}", torch.float32, 2, hw, hw, c, 4, r,
                                                    f"stereo:{hw // 4}" if kind == "cross" else "gauss:2", kind == "self", True)
    for hw, c, r in ((48, 512, 2), (96, 320, 2), (192, 256, 1), (384, 128, 1)) for kind in ("cross", "self")
}


def clamp_max_offset(max_offset: torch.Tensor, H: int, W: int, r: int) -> torch.Tensor:
    """The clamp the attention module applies before calling the operator
    (reference models/attention_blocks.py:45-59); bounds are rounded to the tensor dtype."""
    dt, dev = max_offset.dtype, max_offset.device
    lo = torch.tensor(float(r), dtype=dt, device=dev)
    hx = torch.tensor(W - 1 - r - 1e-3, dtype=dt, device=dev)
    hy = torch.tensor(H - 1 - r - 1e-3, dtype=dt, device=dev)
    x = torch.clamp(max_offset[..., 0:1], min=lo, max=hx)
    y = torch.clamp(max_offset[..., 1:2], min=lo, max=hy)
    return torch.cat((x, y), dim=-1).contiguous()


def make_inputs(wl: Workload, device="cuda", seed: Optional[int] = None, smooth: bool = False,
                rows: Optional[int] = None):
    """Returns dict(max_offset, q, k, v, d_out, d_attn) on `device`, seeded.
    `rows` limits the map to its first rows (a bounded sample of the same workload)."""
    H = wl.H if rows is None else min(rows, wl.H)
    if seed is None:
        seed = (list(WORKLOADS).index(wl.name) if wl.name in WORKLOADS else
                100 + list(MODEL_SHAPES).index(wl.name) if wl.name in MODEL_SHAPES else
                200 + list(MODEL_SHAPES_BASE_F32).index(wl.name))
    g = torch.Generator(device=device).manual_seed(1000 + seed)
    N = H * wl.W

    def randn(*shape):
        return torch.randn(*shape, generator=g, device=device, dtype=torch.float32)

    q, k, v = (randn(wl.B, N, wl.C).to(wl.dtype) for _ in range(3))
    ys, xs = torch.meshgrid(torch.arange(H, device=device, dtype=torch.float32),
                            torch.arange(wl.W, device=device, dtype=torch.float32), indexing="ij")
    coords = torch.stack((xs, ys), -1).view(1, N, 1, 2)
    hh = wl.h if wl.per_head else 1
    kind, val = wl.offsets.split(":")
    if kind == "stereo":
        rpos = torch.zeros(wl.B, N, hh, 2, device=device)
        rpos[..., 0] = -torch.rand(wl.B, N, hh, generator=g, device=device) * float(val)
    else:
        rpos = randn(wl.B, N, hh, 2) * float(val)
    if smooth == "scene" and kind == "stereo":
        # a field as a stereo scene gives it: disparity a coarse random grid (cells of 256 px) upsampled bicubically to
        # the map (mean |d disparity / dx| about 0.35 px per px) with three foreground boxes 25-40 px nearer on top
        # (discontinuities); the same for every head and image
        cell = 256
        coarse = torch.rand(1, 1, H // cell + 2, wl.W // cell + 2, generator=g, device=device)
        d = torch.nn.functional.interpolate(coarse, size=(H, wl.W), mode="bicubic", align_corners=True).clamp(0, 1)[0, 0]
        d = d * (float(val) * 5.0 / 6.0)
        for fy0, fy1, fx0, fx1, dd in ((0.18, 0.55, 0.21, 0.44, 1 / 6), (0.64, 0.92, 0.62, 0.83, 5 / 48), (0.09, 0.28, 0.73, 0.94, 1 / 8)):
            d[int(fy0 * H):int(fy1 * H), int(fx0 * wl.W):int(fx1 * wl.W)] += dd * float(val)
        rpos = torch.zeros(wl.B, N, hh, 2, device=device)
        rpos[..., 0] = -d.reshape(1, N, 1)
    elif smooth:  # spatially correlated field: box-blur the i.i.d. one a few times (about sigma 8 px)
        f = rpos.view(wl.B, H, wl.W, hh * 2).permute(0, 3, 1, 2)
        amp = f.std().clamp_min(1e-6)
        for _ in range(3):
            f = torch.nn.functional.avg_pool2d(f, 17, stride=1, padding=8, count_include_pad=False)
        f = f * (amp / f.std().clamp_min(1e-6))
        rpos = f.permute(0, 2, 3, 1).reshape(wl.B, N, hh, 2)
        if kind == "stereo":
            rpos[..., 1] = 0
            rpos[..., 0] = -rpos[..., 0].abs()
    mo = (coords + rpos).expand(wl.B, N, wl.h, 2).to(wl.dtype).contiguous()
    mo = clamp_max_offset(mo, H, wl.W, wl.r)
    d_out = randn(wl.B, N, wl.C).to(wl.dtype)
    d_attn = None if wl.per_head else randn(wl.B, N, wl.h, wl.M).to(wl.dtype)
    return dict(max_offset=mo, q=q, k=k, v=v, d_out=d_out, d_attn=d_attn, H=H, W=wl.W)


def make_stereo_pair(H=720, W=1280, max_disp=64.0, seed=5, device="cuda", dtype=torch.float32, pad_to=32):
    """Synthetic stereo pair for the end-to-end harness: left ~ U(0,255); right = left shifted by a
    smooth random disparity field in [0, max_disp] px plus N(0,2) noise; both replicate-padded at the
    top/right to multiples of `pad_to` (the reference pads the same way, utils/utils.py:9-23).
    Returns left, right [1,3,Hp,Wp] and the disparity [1,1,H,W]."""
    g = torch.Generator(device=device).manual_seed(seed)
    left = torch.rand(1, 3, H, W, generator=g, device=device) * 255.0
    coarse = torch.rand(1, 1, H // 40 + 2, W // 40 + 2, generator=g, device=device)
    disp = torch.nn.functional.interpolate(coarse, size=(H, W), mode="bicubic", align_corners=True).clamp(0, 1) * max_disp
    xs = torch.arange(W, device=device, dtype=torch.float32).view(1, 1, W).expand(1, H, W)
    ys = torch.arange(H, device=device, dtype=torch.float32).view(1, H, 1).expand(1, H, W)
    # right(x) = left(x + d): sample the left image at x + disparity
    grid = torch.stack((2 * (xs + disp[:, 0]) / (W - 1) - 1, 2 * ys / (H - 1) - 1), -1)
    right = torch.nn.functional.grid_sample(left, grid, mode="bilinear", padding_mode="border", align_corners=True)
    right = (right + 2.0 * torch.randn(right.shape, generator=g, device=device)).clamp(0, 255)
    ph, pw = (-H) % pad_to, (-W) % pad_to
    pad = (0, pw, ph, 0)
    left = torch.nn.functional.pad(left, pad, mode="replicate")
    right = torch.nn.functional.pad(right, pad, mode="replicate")
    return left.to(dtype), right.to(dtype), disp

"""Shared helpers for the tests: seeded inputs and error metrics."""
import torch

from oracle import mat_oracle as O


def make_case(B, H, W, h, Ch, r, dtype=torch.float32, seed=0, offsets="mixed", clamp=True, per_head=True):
    """Seeded q, k, v and max_offset for a small operator call.

    offsets: "mixed" (fractional, some integer, some far out of range),
             "stereo" (x = col - U(0, W/3), y = row exactly), "interior".
    """
    g = torch.Generator().manual_seed(seed)
    N, C = H * W, h * Ch
    q = torch.randn(B, N, C, generator=g)
    k = torch.randn(B, N, C, generator=g)
    v = torch.randn(B, N, C, generator=g)
    coords = O.init_coords(B, H, W).view(B, N, 1, 2)
    hh = h if per_head else 1
    if offsets == "stereo":
        rpos = torch.zeros(B, N, hh, 2)
        rpos[..., 0] = -torch.rand(B, N, hh, generator=g) * (W / 3.0)
    elif offsets == "interior":
        rpos = torch.randn(B, N, hh, 2, generator=g) * 0.7
    else:
        rpos = torch.randn(B, N, hh, 2, generator=g) * (0.4 * max(H, W))
        # a share of exactly-integer offsets (zero fractional part) and of far-away ones
        sel = torch.rand(B, N, hh, 1, generator=g)
        rpos = torch.where(sel < 0.15, rpos.round(), rpos)
        rpos = torch.where(sel > 0.9, rpos * 8, rpos)
    mo = (coords + rpos).expand(B, N, h, 2).contiguous()
    mo = mo.to(dtype)
    if clamp:
        mo = O.clamp_max_offset(mo, H, W, [r, r])
    return mo, q.to(dtype), k.to(dtype), v.to(dtype)


def rel_err(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| / max |b|  -- the norm-wise relative error the tolerances refer to."""
    a, b = a.double(), b.double()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


# Every comparison made through check_err is kept, and the session's summary (tests/conftest.py) prints the
# worst measured error per label beside its bound, so that a run shows how far each bound is from binding.
MEASURED = []


def check_err(got: torch.Tensor, want: torch.Tensor, tol: float, label: str) -> float:
    """Asserts rel_err(got, want) <= tol and records the measured value under `label`."""
    e = rel_err(got, want)
    MEASURED.append((label, e, tol))
    assert e <= tol, f"{label}: {e:.3e} > {tol:.1e}"
    return e


# Bounds of the comparisons (same metric everywhere): 1e-5 in fp32 and 2e-3 in fp16 as the operator's parity
# target states them, 2e-2 in bf16 (8 significand bits instead of 11).
TOL = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 2e-2}
# Gradients at full size (hundreds of contributions per element, errors average out) and against the reference's
# own gradients (the golden vectors) take the same bounds.
GRAD_TOL = TOL
GRAD_TOL_GOLDEN = TOL


def check_grads(got, mo, q, k, v, H, W, r, scale, d_out, d_attn, label):
    """Gradients of a small case against the exact gradient (the oracle's autograd in fp64 on the same rounded
    inputs).  fp32: within 1e-5.  16-bit types: the definition's own gradient in that type (autograd through
    half-precision gathers, products and scatter-adds) lies up to 9e-3 (fp16) from the exact one on maps this
    small (tests/test_oracle_math.py measures it), and the parity target is stated against the definition: a
    gradient within `tol` of the definition's lies within `tol + |definition - exact|` of the exact one, which is
    the bound per tensor here, with the second term measured on this very case.  (The kernel accumulates in
    fp32; comparing it with the definition's fp16 sums directly would test the reference's noise, not the kernel.)"""
    dt = q.dtype
    dbl = lambda t: None if t is None else t.double()
    exact = O.backward(dbl(mo), dbl(q), dbl(k), dbl(v), H, W, [r, r], scale, dbl(d_out), dbl(d_attn))
    own = exact if dt == torch.float32 else O.backward(mo, q, k, v, H, W, [r, r], scale, d_out, d_attn)
    name = str(dt).split(".")[1]
    for a, b, c, tensor in zip(got, exact, own, ("dq", "dk", "dv", "dmo")):
        assert torch.isfinite(a).all(), tensor
        check_err(a.cpu(), b, TOL[dt] + rel_err(c, b), f"{label} {tensor} {name}")

"""matchattention_amd.mat_torch (the `mat_impl='pytorch'` choice of the package) against the oracle: the two are
independent statements of one definition -- tap-by-tap gathers here, one [B,N,h,M,Ch] gather there."""
import pytest
import torch

from matchattention_amd.mat_torch import match_attention_torch
from oracle import mat_oracle as O
from tests.util import make_case, rel_err


@pytest.mark.parametrize("dt,tol", [(torch.float32, 1e-6), (torch.float16, 1e-3), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("shape", [(2, 9, 11, 2, 8, 1, "mixed", True), (1, 12, 10, 4, 16, 2, "stereo", True),
                                   (1, 8, 9, 1, 40, 2, "mixed", False)])
def test_forward_matches_the_oracle(dt, tol, shape):
    B, H, W, h, Ch, r, offs, clamp = shape
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=3, offsets=offs, clamp=clamp)
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], Ch ** -0.5)
    out, attn = match_attention_torch(mo, q, k, v, H, W, [r, r], Ch ** -0.5)
    assert out.dtype == dt and attn.shape == want_attn.shape
    assert rel_err(attn, want_attn) <= tol and rel_err(out, want_out) <= tol


def test_gradients_match_the_oracle():
    B, H, W, h, Ch, r = 1, 8, 9, 2, 8, 1
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float64, seed=5)
    g = torch.Generator().manual_seed(1)
    d_out = torch.randn(B, H * W, h * Ch, generator=g, dtype=torch.float64)
    d_attn = torch.randn(B, H * W, h, 16, generator=g, dtype=torch.float64)
    want = O.backward(mo, q, k, v, H, W, [r, r], 0.3, d_out, d_attn)
    ins = [t.clone().requires_grad_(True) for t in (q, k, v, mo)]
    out, attn = match_attention_torch(ins[3], ins[0], ins[1], ins[2], H, W, [r, r], 0.3)
    got = torch.autograd.grad([out, attn], ins, [d_out, d_attn])
    for a, b in zip(got, want):
        assert rel_err(a, b) <= 1e-12

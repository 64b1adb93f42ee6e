"""matchattn_forward_static: the forward on the library's own static device scratch (nothing allocated around the
call) against matchattn_forward_ws with a caller-provided workspace.  Two calls in a row share the one array; the
second is smaller, so stale contents of the first lie beyond and inside what it uses."""
import pytest
import torch

from matchattention_amd import _cabi
from tests.gpu_util import DT, hip_forward

pytestmark = pytest.mark.gpu


def _inputs(B, H, W, h, Ch, r, seed, per_head):
    g = torch.Generator(device="cuda").manual_seed(seed)
    N, C = H * W, h * Ch
    q, k, v = (torch.randn(B, N, C, generator=g, device="cuda").half() for _ in range(3))
    ys, xs = torch.meshgrid(torch.arange(H, device="cuda", dtype=torch.float32),
                            torch.arange(W, device="cuda", dtype=torch.float32), indexing="ij")
    coords = torch.stack((xs, ys), -1).view(1, N, 1, 2)
    rel = torch.randn(B, N, h if per_head else 1, 2, generator=g, device="cuda") * 9.0
    mo = (coords + rel).expand(B, N, h, 2).half().contiguous()
    mo[..., 0].clamp_(r, W - 2 - r)
    mo[..., 1].clamp_(r, H - 2 - r)
    return mo, q, k, v


def _static_forward(lib, mo, q, k, v, H, W, r, scale):
    B, N, C = q.shape
    h = mo.size(2)
    out = torch.full_like(q, float("nan"))
    attn = torch.full((B, N, h, (2 * r + 2) ** 2), float("nan"), dtype=q.dtype, device=q.device)
    _cabi.check(lib.matchattn_forward_static(mo.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                             attn.data_ptr(), B, H, W, C, h, r, r, float(scale), DT[q.dtype],
                                             torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return out, attn


def test_forward_on_static_scratch_matches_forward_ws(hip_lib):
    cap = hip_lib.matchattn_static_scratch_bytes()
    assert cap == 40 << 20, hip_lib.matchattn_last_error()
    r, Ch, h = 2, 32, 8
    # both maps take the LDS-tile path by themselves (from 2^20 head-queries), i.e. both use the scratch
    for (B, H, W, seed, per_head) in ((1, 400, 400, 11, False), (1, 300, 448, 12, True)):
        assert 0 < hip_lib.matchattn_forward_workspace_bytes(B, H, W, h * Ch, h, r, r, _cabi.F16) <= cap
        mo, q, k, v = _inputs(B, H, W, h, Ch, r, seed, per_head)
        got_out, got_attn = _static_forward(hip_lib, mo, q, k, v, H, W, r, Ch ** -0.5)
        assert _cabi.last_forward_kernel().startswith("fwd_tile_f16"), _cabi.last_forward_kernel()
        want_out, want_attn = hip_forward(hip_lib, mo, q, k, v, H, W, r, Ch ** -0.5)
        assert _cabi.last_forward_kernel().startswith("fwd_tile_f16")
        assert torch.equal(got_out, want_out) and torch.equal(got_attn, want_attn), (H, W)
        assert torch.isfinite(got_out).all() and torch.isfinite(got_attn).all()


def test_static_scratch_rejects_maps_beyond_its_capacity(hip_lib):
    # 2 x 544 x 960 x 8 heads needs 72 MiB: an error with the sizes in it, and nothing is launched
    B, H, W, h, Ch, r = 2, 544, 960, 8, 32, 2
    assert hip_lib.matchattn_forward_workspace_bytes(B, H, W, h * Ch, h, r, r, _cabi.F16) > hip_lib.matchattn_static_scratch_bytes()
    # tensors of the sizes the shape states (0.5 GiB each): were the refusal ever lost, the launch would stay inside them
    N, C, M = H * W, h * Ch, (2 * r + 2) ** 2
    qkv = torch.zeros(B, N, C, dtype=torch.float16, device="cuda")
    out = torch.empty_like(qkv)
    attn = torch.empty(B, N, h, M, dtype=torch.float16, device="cuda")
    mo = torch.full((B, N, h, 2), float(r), dtype=torch.float16, device="cuda")
    rc = hip_lib.matchattn_forward_static(mo.data_ptr(), qkv.data_ptr(), qkv.data_ptr(), qkv.data_ptr(), out.data_ptr(),
                                          attn.data_ptr(), B, H, W, C, h, r, r, 1.0, _cabi.F16,
                                          torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 2
    assert b"scratch" in hip_lib.matchattn_last_error()


def test_small_maps_need_no_scratch_and_still_run(hip_lib):
    # below the tile path's threshold the direct kernel runs: same entry point, no scratch touched
    B, H, W, h, Ch, r = 1, 24, 40, 4, 32, 1
    mo, q, k, v = _inputs(B, H, W, h, Ch, r, 5, True)
    got = _static_forward(hip_lib, mo, q, k, v, H, W, r, Ch ** -0.5)
    want = hip_forward(hip_lib, mo, q, k, v, H, W, r, Ch ** -0.5)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])

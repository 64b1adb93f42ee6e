"""The PyTorch-facing operator: same call shape as the reference's MF_FusedForwardOps,
differentiable, and reachable through the `match_attention.fused_forward` import."""
import pytest
import torch

from oracle import mat_oracle as O
from tests.util import make_case, rel_err

pytestmark = pytest.mark.gpu


def test_module_forward_and_autograd(hip_lib):
    from matchattention_amd import MF_FusedForwardOps
    B, H, W, h, Ch, r = 2, 10, 12, 4, 32, 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float32, seed=3)
    scale = Ch ** -0.5
    ref_in = [t.clone().requires_grad_(True) for t in (mo, q, k, v)]
    out_r, attn_r = O.forward(*ref_in, H, W, [r, r], scale)
    loss_r = (out_r * out_r).sum() + (attn_r * torch.arange(36.0)).sum()
    loss_r.backward()
    dev_in = [t.cuda().requires_grad_(True) for t in (mo, q, k, v)]
    op = MF_FusedForwardOps()
    out, attn = op(*dev_in, H, W, [r, r], 36, attn_type="l1_norm", scale=scale)
    loss = (out * out).sum() + (attn * torch.arange(36.0, device="cuda")).sum()
    loss.backward()
    assert rel_err(out.detach().cpu(), out_r.detach()) <= 1e-5
    assert rel_err(attn.detach().cpu(), attn_r.detach()) <= 1e-5
    for a, b in zip(dev_in, ref_in):
        assert rel_err(a.grad.cpu(), b.grad) <= 1e-5
    # inference path (no grad): in-place opaque op, same numbers
    with torch.no_grad():
        out2, attn2 = op(*[t.detach() for t in dev_in], H, W, [r, r], 36, "l1_norm", scale)
    assert torch.equal(out2, out.detach()) and torch.equal(attn2, attn.detach())


def test_reference_import_name_and_native_signature(hip_lib):
    import match_attention
    B, H, W, h, Ch, r = 1, 9, 9, 2, 16, 1
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float16, seed=4)
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], 0.25)
    mo, q, k, v = (t.cuda() for t in (mo, q, k, v))
    output = torch.zeros_like(v)
    attn_out = q.new_zeros([B, H * W, h, 16])
    match_attention.fused_forward(mo, q, k, v, output, attn_out, H, W, [r, r], 16, "l1_norm", 0.25)
    assert rel_err(output.cpu(), want_out) <= 2e-3 and rel_err(attn_out.cpu(), want_attn) <= 2e-3


def test_reference_dispatcher_fallback_route(hip_lib):
    # the reference's `except ImportError` branch: torch.ops.match_attention.fused_forward with the schema of
    # models/src/match_former_cuda.cpp:46-49 (registered when the package is imported)
    import matchattention_amd  # noqa: F401
    B, H, W, h, Ch, r = 1, 9, 10, 2, 16, 1
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float16, seed=8)
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], 0.25)
    mo, q, k, v = (t.cuda() for t in (mo, q, k, v))
    output = torch.zeros_like(v)
    attn_out = q.new_zeros([B, H * W, h, 16])
    assert torch.ops.match_attention.fused_forward(mo, q, k, v, output, attn_out, H, W, [r, r], 16, "l1_norm", 0.25) is None
    assert rel_err(output.cpu(), want_out) <= 2e-3 and rel_err(attn_out.cpu(), want_attn) <= 2e-3


def test_opaque_op_survives_torch_compile_tracing(hip_lib):
    from matchattention_amd import MF_FusedForwardOps
    B, H, W, h, Ch, r = 1, 8, 8, 2, 8, 1
    mo, q, k, v = (t.cuda() for t in make_case(B, H, W, h, Ch, r, torch.float32, seed=6))
    op = MF_FusedForwardOps()
    assert torch.library.opcheck(torch.ops.matchattention_amd.match_attention,
                                 (mo, q, k, v, H, W, [r, r], 16, "l1_norm", 0.5),
                                 test_utils=("test_schema", "test_faketensor"))


def test_fused_module_step_is_an_opaque_op_too(hip_lib):
    # schema and fake-tensor checks of the fused form (both result layouts), as torch.compile needs them
    B, H, W, h, Ch, r = 1, 8, 9, 2, 16, 1
    g = torch.Generator().manual_seed(2)
    q, k, v, gate = (torch.randn(B, H * W, h * Ch, generator=g).half().cuda() for _ in range(4))
    rel = torch.randn(B, H * W, 1, 2, generator=g).half().cuda()
    for concat in (True, False):
        assert torch.library.opcheck(torch.ops.matchattention_amd.fused_module_step,
                                     (rel, q, k, v, gate if concat else None, H, W, [r, r], h, 0.25, True, concat),
                                     test_utils=("test_schema", "test_faketensor"))


@pytest.mark.parametrize("dt,shared,gated,concat", [(torch.float32, True, True, True), (torch.float32, False, False, False),
                                                    (torch.float16, True, True, True), (torch.float16, False, True, False)])
def test_fused_module_step_trains_like_the_separate_steps(hip_lib, dt, shared, gated, concat):
    # gradients of the one-call module step (grid add, clamp, operator, gate, concatenation) against autograd through
    # the same steps written out in torch ops around the oracle, in fp64 on the same rounded inputs; some positions lie
    # outside the clamp's range, so its mask matters
    from matchattention_amd import fused_module_forward
    from tests.util import TOL, check_err
    B, H, W, h, Ch, r = 2, 12, 14, 4, 16, 2
    N, C, M = H * W, h * Ch, 36
    g = torch.Generator().manual_seed(21)
    q, k, v = (torch.randn(B, N, C, generator=g).to(dt) for _ in range(3))
    rel = (torch.randn(B, N, 1 if shared else h, 2, generator=g) * 4.0).to(dt)
    gate = torch.rand(B, N, C, generator=g).to(dt) if gated else None
    d_res = torch.randn(B, N, C + (h * M if concat else 0), generator=g).to(dt)
    d_attn = None if concat else torch.randn(B, N, h, M, generator=g).to(dt)
    scale = Ch ** -0.5

    # reference: the separate steps in fp64
    ins64 = [t.double().requires_grad_(True) for t in (rel, q, k, v)] + ([gate.double().requires_grad_(True)] if gated else [])
    grid = O.init_coords(B, H, W, dtype=torch.float64).view(B, N, 1, 2)
    raw = ins64[0] + grid
    raw = (raw + (raw.detach().to(dt).double() - raw.detach())).expand(B, N, h, 2)   # the sum is stored in the tensor dtype
    lo = float(r)
    hx, hy = (float(torch.tensor(s - 1 - r - 1e-3, dtype=dt)) for s in (W, H))
    mo = torch.cat((raw[..., 0:1].clamp(lo, hx), raw[..., 1:2].clamp(lo, hy)), -1)
    out, attn = O.forward(mo, ins64[1], ins64[2], ins64[3], H, W, [r, r], scale)
    if gated:
        out = ins64[4] * out
    if concat:
        want = torch.autograd.grad([torch.cat((out, attn.reshape(B, N, -1)), -1)], ins64, [d_res.double()])
    else:
        want = torch.autograd.grad([out, attn], ins64, [d_res.double(), d_attn.double()])

    dev = [t.cuda().requires_grad_(True) for t in (rel, q, k, v)] + ([gate.cuda().requires_grad_(True)] if gated else [])
    res = fused_module_forward(dev[0], dev[1], dev[2], dev[3], H, W, [r, r], h, scale, gate=dev[4] if gated else None,
                               relative=True, concat=concat)
    if concat:
        got = torch.autograd.grad([res], dev, [d_res.cuda()])
    else:
        got = torch.autograd.grad(list(res), dev, [d_res.cuda(), d_attn.cuda()])
    clamped = float(((raw.detach()[..., 0] < lo) | (raw.detach()[..., 0] > hx)).float().mean())
    assert clamped > 0.05                                   # the mask is exercised
    tol = TOL[dt]
    for a, b, name in zip(got, want, ("d_position", "dq", "dk", "dv", "d_gate")):
        assert a.shape == b.shape and torch.isfinite(a).all(), name
        check_err(a.cpu(), b, tol, f"fused step bwd {name} {str(dt).split('.')[1]}")

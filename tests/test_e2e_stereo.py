"""End to end: MatchStereo-T harness (random-init weights from a seed) on a synthetic 1280x720
stereo pair, operator = HIP library vs operator = PyTorch definition (the oracle, run on the GPU).

Two measurements:
  * teacher-forced: the PyTorch operator drives the network and, at each of its 52 calls, the
    HIP operator is evaluated on the very same inputs -- parity at the real model shapes
    (Ch = 40/32/16/8, r = 2/2/1/1, self and cross) to the operator tolerances;
  * free-running (a diagnostic, not a parity criterion): both operators drive the network on their
    own.  The 0.05 px mean-disparity bound quoted for this configuration is UNPINNED here: it
    presumes trained weights, and no checkpoint can be loaded.  A random-init network is chaotic
    (floor() of the sampling centres, arg-max of the initial correlation, 26 layers that divide
    the field by field_scale = 0.1; fields of several hundred px where fp16 spacing is 0.5 px):
    a half-ulp perturbation of the PyTorch operator's own outputs moves the final disparity by
    0.4-1 px.  The test prints the HIP-vs-PyTorch difference beside that measured self-noise of
    the reference (several draws) and only checks that the former is of the latter's size; what
    gates parity at the model's shapes is the teacher-forced test."""
import pytest
import torch

from oracle import mat_oracle as O

pytestmark = pytest.mark.gpu


def _run(op, left, right, dtype):
    from matchattention_amd.stereo_harness import MatchStereoHarness
    model = MatchStereoHarness(op, "tiny", seed=0).cuda().to(dtype).eval()
    with torch.inference_mode():
        full, _ = model(left, right)
    torch.cuda.synchronize()
    assert torch.isfinite(full).all()
    return full.float()[..., 0]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.float16, 2e-3)])
def test_operator_parity_at_every_call_of_the_model(hip_lib, dtype, tol):
    from matchattention_amd import MF_FusedForwardOps
    from matchattention_amd.workloads import make_stereo_pair
    hip_op = MF_FusedForwardOps()
    worst = []

    def both(mo, q, k, v, H, W, win_r, M, scale):
        want = O.forward(mo, q, k, v, H, W, win_r, scale)
        got = hip_op(mo, q, k, v, H, W, win_r, M, "l1_norm", scale)
        for g, w in zip(got, want):
            worst.append(float((g.float() - w.float()).abs().max() / w.float().abs().max()))
        return want

    left, right, _ = make_stereo_pair(720, 1280, dtype=dtype)
    assert left.shape == (1, 3, 736, 1280)        # padded to a multiple of 32 like the reference does
    _run(both, left, right, dtype)
    assert len(worst) == 2 * 52
    print(f"teacher-forced {dtype}: worst relative error over 52 calls (out, attn): {max(worst):.3e}")
    assert max(worst) <= tol


def test_free_running_difference_is_of_the_size_of_the_references_own_noise(hip_lib):
    from matchattention_amd import MF_FusedForwardOps
    from matchattention_amd.workloads import make_stereo_pair
    hip_op = MF_FusedForwardOps()

    def hip(mo, q, k, v, H, W, win_r, M, scale):
        return hip_op(mo, q, k, v, H, W, win_r, M, "l1_norm", scale)

    def ref(mo, q, k, v, H, W, win_r, M, scale):
        return O.forward(mo, q, k, v, H, W, win_r, scale)

    def jittered(mo, q, k, v, H, W, win_r, M, scale):
        out, attn = O.forward(mo, q, k, v, H, W, win_r, scale)
        half_ulp = 0.5 * torch.finfo(q.dtype).eps
        return out * (1 + half_ulp * torch.randn_like(out)), attn * (1 + half_ulp * torch.randn_like(attn))

    torch.manual_seed(0)
    for dtype in (torch.float32, torch.float16):
        left, right, _ = make_stereo_pair(720, 1280, dtype=dtype)
        d_ref = _run(ref, left, right, dtype)
        d_hip = _run(hip, left, right, dtype)
        # the random-weight network amplifies a half-ulp change of the operator's outputs to a disparity change
        # of the order of a pixel, and the library convolutions differ from run to run: the floor is one draw
        # of a wide distribution, so it is taken as the largest of three draws and compared with a margin
        floor = max(float((_run(jittered, left, right, dtype) - d_ref).abs().mean()) for _ in range(3))
        diff = float((d_hip - d_ref).abs().mean())
        print(f"free-running {dtype}: mean|hip - pytorch| = {diff:.4f} px, noise floor (half-ulp jitter, max of 3) = {floor:.4f} px, "
              f"mean |disparity| = {float(d_ref.abs().mean()):.1f} px")
        assert diff <= 3.0 * floor + 0.05


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_fusing_the_module_steps_changes_no_bit_at_any_call_of_the_model(hip_lib, dtype):
    # 52 operator calls, self- and cross-attention, four shapes: with the grid add, clamp, gate and concatenation
    # done inside the native call, what reaches the output projection must be identical to the separate launches
    # on the very same inputs (the two are compared call by call: the library convolutions around them do not
    # reproduce their own bits from one model instance to the next)
    from matchattention_amd import MF_FusedForwardOps, fused_module_forward
    from matchattention_amd.stereo_harness import MatchStereoHarness
    from matchattention_amd.workloads import make_stereo_pair
    from tests.test_hip_parity import _module_steps
    hip_op = MF_FusedForwardOps()
    calls = []

    def hip(mo, q, k, v, H, W, win_r, M, scale):
        return hip_op(mo, q, k, v, H, W, win_r, M, "l1_norm", scale)

    def checked(rel, q, k, v, H, W, win_r, h, scale, gate=None, relative=True, concat=False):
        got = fused_module_forward(rel, q, k, v, H, W, win_r, h, scale, gate=gate, relative=relative, concat=concat)
        M = (2 * win_r[0] + 2) ** 2
        _, out, attn, cat = _module_steps(rel, q, k, v, gate, H, W, win_r[0], h,
                                          lambda mo, q, k, v: hip(mo, q, k, v, H, W, win_r, M, scale))
        if concat:
            assert torch.equal(got, cat)
        else:
            assert torch.equal(got[0], out) and torch.equal(got[1], attn)
        calls.append((q.size(2) // h, win_r[0], rel.size(2), concat))
        return got

    left, right, _ = make_stereo_pair(720, 1280, dtype=dtype)
    model = MatchStereoHarness(hip, "tiny", seed=0, fused=checked).cuda().to(dtype).eval()
    with torch.inference_mode():
        full, _ = model(left, right)
    torch.cuda.synchronize()
    assert torch.isfinite(full).all()
    assert len(calls) == 52 and {c[0] for c in calls} == {40, 32, 16, 8}
    assert sum(1 for c in calls if c[3]) == 26 and all(c[2] == 1 for c in calls if c[3])     # cross: one shared position

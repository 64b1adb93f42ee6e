"""The HIP operator at the benchmark's own shapes, against the oracle.

Every benchmark shape is compared over the whole map: the forward against the oracle evaluated in bands of query
rows (the operator is independent per query, so banding only bounds the oracle's gather temporaries), the
backward of the shapes that have one (fp16 384x384, and the 2 x 384 x 384 optical-flow shape with shared and with
per-head offsets) against the oracle's autograd in fp32 on the same fp16-rounded inputs.

Tolerances (max|a-b| / max|b|): 1e-5 in fp32, 2e-3 in fp16 for outputs, attention weights and gradients alike
(tests.util.GRAD_TOL explains what the fp16 gradients are compared with)."""
import pytest
import torch

from oracle import mat_oracle as O
from tests.gpu_util import hip_backward, hip_forward
from tests.util import GRAD_TOL, TOL, check_err

pytestmark = pytest.mark.gpu



def _inputs(name, field=False):
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    wl = WORKLOADS[name]
    return wl, make_inputs(wl, smooth=field)


def test_cfg1_forward_whole_map(hip_lib):
    wl, inp = _inputs("cfg1_cross")
    assert inp["q"].dtype == torch.float32
    out, attn = hip_forward(hip_lib, inp["max_offset"], inp["q"], inp["k"], inp["v"], inp["H"], inp["W"], wl.r, wl.scale)
    want_out, want_attn = O.forward_chunked(inp["max_offset"].cpu(), inp["q"].cpu(), inp["k"].cpu(), inp["v"].cpu(),
                                            inp["H"], inp["W"], [wl.r, wl.r], wl.scale, rows_per_chunk=8)
    check_err(attn.cpu(), want_attn, TOL[torch.float32], "cfg1 fwd attn f32")
    check_err(out.cpu(), want_out, TOL[torch.float32], "cfg1 fwd out f32")


def test_cfg2_forward_and_backward_whole_map(hip_lib):
    wl, inp = _inputs("cfg2_cross")
    assert inp["q"].dtype == torch.float16
    H, W = inp["H"], inp["W"]
    args = (inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale)
    out, attn = hip_forward(hip_lib, *args)
    cpu = [inp[n].cpu() for n in ("max_offset", "q", "k", "v")]
    want_out, want_attn = O.forward_chunked(*cpu, H, W, [wl.r, wl.r], wl.scale, rows_per_chunk=8)
    check_err(attn.cpu(), want_attn, TOL[torch.float16], "cfg2 fwd attn f16")
    check_err(out.cpu(), want_out, TOL[torch.float16], "cfg2 fwd out f16")

    got = hip_backward(hip_lib, *args, inp["d_out"], inp["d_attn"])
    # (autograd in fp32 on the fp16-rounded inputs: exact to 1e-6 of the gradient, a thousandth of the tolerance,
    # at half the time of fp64 over the whole map)
    want = O.backward(*(t.float() for t in cpu), H, W, [wl.r, wl.r], wl.scale, inp["d_out"].cpu().float(),
                      None if inp["d_attn"] is None else inp["d_attn"].cpu().float(), rows_per_chunk=32)
    for a, b, name in zip(got, want, ("dq", "dk", "dv", "dmo")):
        assert torch.isfinite(a).all(), name
        check_err(a.cpu(), b, GRAD_TOL[torch.float16], f"cfg2 bwd {name} f16")


@pytest.mark.parametrize("name", ["cfg4_cross", "cfg4_self"])
def test_cfg4_backward_whole_map(hip_lib, name):
    # 2 x 384 x 384, 8 heads, 6x6 taps, 2-D offsets; cross: one offset per pixel, dO and dA given; self: one offset
    # per head, dO only.  Every gradient over the whole map against the oracle's autograd (in fp32 on the
    # fp16-rounded inputs, in bands of 16 query rows)
    wl, inp = _inputs(name)
    H, W = inp["H"], inp["W"]
    assert (inp["d_attn"] is None) == (name == "cfg4_self")
    got = hip_backward(hip_lib, inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale, inp["d_out"], inp["d_attn"])
    got = [g.cpu() for g in got]
    cpu = [None if inp[n] is None else inp[n].cpu().float() for n in ("max_offset", "q", "k", "v", "d_out", "d_attn")]
    del inp
    torch.cuda.empty_cache()
    want = O.backward(*cpu[:4], H, W, [wl.r, wl.r], wl.scale, cpu[4], cpu[5], rows_per_chunk=16)
    for a, b, tensor in zip(got, want, ("dq", "dk", "dv", "dmo")):
        assert torch.isfinite(a).all(), tensor
        check_err(a, b, GRAD_TOL[torch.float16], f"{name} bwd {tensor} f16")


@pytest.mark.parametrize("name,field,dt", [
    ("cfg3_cross", False, None), ("cfg3_self", False, None), ("cfg4_cross", False, None), ("cfg4_self", False, None),
    # spatially coherent offsets (a stereo scene's field: what a model's cross-attention produces), and bfloat16
    ("cfg3_cross", "scene", None), ("cfg3_cross", False, torch.bfloat16)],
    ids=["cfg3_cross", "cfg3_self", "cfg4_cross", "cfg4_self", "cfg3_cross_scene_field", "cfg3_cross_bf16"])
def test_large_maps_forward_whole_map(hip_lib, name, field, dt):
    wl, inp = _inputs(name, field)
    if dt is not None:
        for n in ("max_offset", "q", "k", "v"):
            inp[n] = inp[n].to(dt)
    H, W = inp["H"], inp["W"]
    out, attn = hip_forward(hip_lib, inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale)
    # A second run puts the head-queries into other lanes (the order inside a bucket is first come, first served) and
    # must give the same bits: with millions of head-queries a single channel rounded differently in one lane position
    # shows here and nowhere at the sizes of the small cases.
    out2, attn2 = hip_forward(hip_lib, inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale)
    assert torch.equal(out, out2) and torch.equal(attn, attn2)
    del out2, attn2
    out, attn = out.cpu(), attn.cpu()
    dt = inp["q"].dtype
    cpu = [inp[n].cpu() for n in ("max_offset", "q", "k", "v")]
    del inp
    torch.cuda.empty_cache()
    want_out, want_attn = O.forward_chunked(*cpu, H, W, [wl.r, wl.r], wl.scale, rows_per_chunk=8)
    check_err(attn, want_attn, TOL[dt], f"{name} fwd attn {dt}")
    check_err(out, want_out, TOL[dt], f"{name} fwd out {dt}")


def test_map_with_more_tiles_than_a_thread_keeps(hip_lib):
    """A map of 96 x 88 = 8 448 tiles of 16 x 8 pixels: the work-list kernel's threads then take nine buckets each and
    park their populations in scratch memory between the two walks (up to four stay in registers, which is what the
    benchmark shapes exercise), two images so that the tile walk crosses an image boundary inside a thread's run, a
    last strip narrower than the others (88 = 10 x 8 + 8 is even; 1 400 pixels = 87.5 tiles gives the ragged edge).
    Forward against the oracle on bands of query rows at the top, across the image boundary and at the bottom, the
    whole map against the direct-gather kernel, and the tile kernel must have served (nearly) every query."""
    from matchattention_amd import _cabi
    torch.manual_seed(11)
    B, H, W, h, Ch, r = 2, 384, 1400, 4, 16, 2
    N, C = H * W, h * Ch
    dev = "cuda"
    q, k, v = (torch.randn(B, N, C, device=dev, dtype=torch.float16) for _ in range(3))
    coords = O.init_coords(B, H, W).view(B, N, 1, 2).to(dev)
    rel = torch.zeros(B, N, h, 2, device=dev)
    rel[..., 0] = -torch.rand(B, N, 1, device=dev) * 96 + torch.randn(B, N, h, device=dev) * 0.7     # per-head positions
    rel[..., 1] = torch.randn(B, N, h, device=dev) * 2.0
    mo = O.clamp_max_offset((coords + rel).half(), H, W, [r, r]).contiguous()
    scale = Ch ** -0.5
    nbins = B * ((H + 7) // 8) * ((W + 15) // 16)
    assert nbins > 4 * 1024
    deferred = []
    _cabi.set_option("forward_lds", 1)
    try:
        out, attn = hip_forward(hip_lib, mo, q, k, v, H, W, r, scale, deferred=deferred)
        assert _cabi.last_forward_kernel().startswith("fwd_tile_")
    finally:
        _cabi.set_option("forward_lds", -1)
    assert 0 <= deferred[0] < 0.001 * B * N * h, deferred
    _cabi.set_option("forward_lds", 0)
    try:
        out_d, attn_d = hip_forward(hip_lib, mo, q, k, v, H, W, r, scale)
    finally:
        _cabi.set_option("forward_lds", -1)
    check_err(out, out_d, TOL[torch.float16], "many tiles: tile vs direct out f16")
    check_err(attn, attn_d, TOL[torch.float16], "many tiles: tile vs direct attn f16")
    for y0 in (0, H - 8, 2 * H - 16):                       # rows of the stacked images: top, image boundary, bottom
        b, y = divmod(y0, H)
        rows = min(16, H - y)
        sl = slice(y * W, (y + rows) * W)
        want_out, want_attn = _oracle_rows(mo[b:b + 1, sl].cpu(), q[b:b + 1, sl].cpu(), k[b:b + 1].cpu(), v[b:b + 1].cpu(),
                                           H, W, r, scale)
        check_err(out[b:b + 1, sl].cpu(), want_out, TOL[torch.float16], "many tiles fwd out f16")
        check_err(attn[b:b + 1, sl].cpu(), want_attn, TOL[torch.float16], "many tiles fwd attn f16")


def _oracle_rows(mo, q, k, v, H, W, r, scale):
    """The oracle's forward for a band of queries (mo [B,n,h,2], q [B,n,C]) against the whole K and V [B,N,C]:
    the steps of oracle.mat_oracle.forward_chunked on one band."""
    B, n, C = q.shape
    h = mo.size(2)
    k4, v4 = k.view(B, k.size(1), h, -1), v.view(B, v.size(1), h, -1)
    with torch.no_grad():
        idx = O.tap_indices(torch.floor(mo).to(torch.int32), [r, r], H, W)
        lg = O.window_logits(q.reshape(B, n, h, -1), k4, idx) * scale
        a = O.bilinear_softmax(lg, O.corner_weights(mo), [r, r])
        return O.aggregate(v4, a, idx), a

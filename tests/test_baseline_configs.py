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



def _inputs(name):
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    wl = WORKLOADS[name]
    return wl, make_inputs(wl)


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


@pytest.mark.parametrize("name", ["cfg3_cross", "cfg3_self", "cfg4_cross", "cfg4_self"])
def test_large_maps_forward_whole_map(hip_lib, name):
    wl, inp = _inputs(name)
    H, W = inp["H"], inp["W"]
    out, attn = hip_forward(hip_lib, inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale)
    out, attn = out.cpu(), attn.cpu()
    dt = inp["q"].dtype
    cpu = [inp[n].cpu() for n in ("max_offset", "q", "k", "v")]
    del inp
    torch.cuda.empty_cache()
    want_out, want_attn = O.forward_chunked(*cpu, H, W, [wl.r, wl.r], wl.scale, rows_per_chunk=8)
    check_err(attn, want_attn, TOL[dt], f"{name} fwd attn f16")
    check_err(out, want_out, TOL[dt], f"{name} fwd out f16")

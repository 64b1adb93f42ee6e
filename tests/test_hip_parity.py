"""Parity of the HIP operator (through the C ABI) with the oracle and the golden vectors.

Tolerances (norm-wise relative error max|a-b| / max|b|): 1e-5 in fp32, 2e-3 in fp16,
2e-2 in bf16 (bf16 keeps 8 significand bits; the stated fp16 bound scaled by 2^3)."""
import glob
import os

import pytest
import torch

from oracle import mat_oracle as O
from tests.gpu_util import hip_backward, hip_forward
from tests.test_oracle_golden import GOLDEN, load_golden
from tests.util import GRAD_TOL, GRAD_TOL_GOLDEN, TOL, check_err, check_grads, make_case, rel_err

pytestmark = pytest.mark.gpu


def _dev(*ts):
    return [None if t is None else t.cuda() for t in ts]


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_forward_matches_reference_golden(hip_lib, path):
    g = load_golden(path)
    mo, q, k, v = _dev(g["max_offset"], g["q"], g["k"], g["v"])
    out, attn = hip_forward(hip_lib, mo, q, k, v, g["H"], g["W"], g["r"], g["Ch"] ** -0.5)
    tol = TOL[g["dtype"]]
    assert rel_err(attn.cpu(), g["attn"]) <= tol
    assert rel_err(out.cpu(), g["out"]) <= tol


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_backward_matches_reference_golden(hip_lib, path):
    g = load_golden(path)
    mo, q, k, v, d_out, d_attn = _dev(g["max_offset"], g["q"], g["k"], g["v"], g["d_out"], g["d_attn"])
    grads = hip_backward(hip_lib, mo, q, k, v, g["H"], g["W"], g["r"], g["Ch"] ** -0.5, d_out, d_attn)
    # (the reference's gradients are themselves autograd in the tensor dtype)
    dtn = str(g["dtype"]).split(".")[1]
    for got, name in zip(grads, ("dq", "dk", "dv", "dmo")):
        check_err(got.cpu(), g[name], GRAD_TOL_GOLDEN[g["dtype"]], f"golden bwd {name} {dtn}")


CASES = [
    # B, H, W, h, Ch, r, dtype, offsets, clamp
    (1, 9, 11, 2, 32, 1, torch.float32, "mixed", True),
    (2, 8, 13, 4, 8, 2, torch.float32, "mixed", False),
    (1, 12, 10, 1, 40, 2, torch.float32, "stereo", True),
    (1, 9, 9, 2, 12, 1, torch.float32, "mixed", True),      # no tiled instantiation for Ch=12: generic kernel
    (1, 9, 9, 2, 6, 2, torch.float32, "mixed", True),       # generic kernel
    (1, 10, 10, 2, 16, 3, torch.float32, "mixed", True),    # r = 3: generic kernel
    (1, 16, 24, 4, 32, 1, torch.float16, "stereo", True),
    (2, 12, 17, 8, 32, 2, torch.float16, "mixed", True),
    (1, 11, 12, 4, 40, 2, torch.float16, "mixed", False),
    (1, 11, 12, 2, 8, 1, torch.float16, "mixed", True),
    (1, 11, 12, 2, 16, 1, torch.float16, "interior", True),
    (1, 10, 12, 2, 64, 2, torch.float16, "mixed", True),
    (1, 10, 12, 1, 128, 1, torch.float16, "mixed", True),
    (1, 10, 12, 2, 80, 2, torch.float16, "stereo", True),
    (1, 10, 12, 3, 12, 1, torch.float16, "mixed", True),    # generic kernel
    (1, 12, 12, 4, 32, 2, torch.bfloat16, "mixed", True),
    (1, 12, 12, 2, 16, 1, torch.bfloat16, "stereo", True),
    # the coarse levels of the reference's `small` and `base` variants in its default precision, and head sizes of its
    # `large` configuration: more than 16 vectors per head (two per lane in the forward and the per-key pass, 32 lanes per
    # head-query in the per-query pass)
    (1, 9, 11, 2, 80, 2, torch.float32, "mixed", True),
    (2, 8, 9, 1, 128, 2, torch.float32, "mixed", False),
    (1, 10, 9, 2, 96, 1, torch.float32, "stereo", True),
    (1, 9, 10, 2, 128, 1, torch.float32, "mixed", True),
    (1, 9, 11, 2, 96, 2, torch.float16, "mixed", True),
    (1, 8, 12, 1, 192, 2, torch.float16, "mixed", False),
    (1, 9, 9, 2, 192, 1, torch.bfloat16, "stereo", True),
    (1, 8, 9, 1, 192, 2, torch.float32, "mixed", True),
    (1, 9, 8, 2, 192, 1, torch.float32, "mixed", False),
]


@pytest.mark.parametrize("case", CASES, ids=[f"{c[6]}".split(".")[1] + f"_B{c[0]}_{c[1]}x{c[2]}_h{c[3]}_ch{c[4]}_r{c[5]}_{c[7]}" for c in CASES])
def test_forward_and_backward_match_oracle(hip_lib, case):
    B, H, W, h, Ch, r, dt, offs, clamp = case
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=B * 1000 + H * 10 + Ch, offsets=offs, clamp=clamp)
    scale = Ch ** -0.5
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], scale)
    dmo_, dq_, dk_, dv_ = _dev(mo, q, k, v)
    out, attn = hip_forward(hip_lib, dmo_, dq_, dk_, dv_, H, W, r, scale)
    tol = TOL[dt]
    assert torch.isfinite(out).all() and torch.isfinite(attn).all()
    assert rel_err(attn.cpu(), want_attn) <= tol
    assert rel_err(out.cpu(), want_out) <= tol
    # gradients: compare against the oracle's autograd evaluated in fp64 on the same (dtype-rounded) inputs,
    # i.e. against the exact gradient of the function the kernel evaluates
    g = torch.Generator().manual_seed(7)
    M = (2 * r + 2) ** 2
    d_out = torch.randn(B, H * W, h * Ch, generator=g).to(dt)
    d_attn = torch.randn(B, H * W, h, M, generator=g).to(dt)
    got = hip_backward(hip_lib, dmo_, dq_, dk_, dv_, H, W, r, scale, d_out.cuda(), d_attn.cuda())
    check_grads(got, mo, q, k, v, H, W, r, scale, d_out, d_attn, "seeded cases bwd")


@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("dt,offs,clamp,per_head", [(torch.float32, "mixed", False, True), (torch.float16, "stereo", True, False),
                                                     (torch.float32, "mixed", True, False)])
def test_both_backward_modes_agree_with_autograd(hip_lib, mode, dt, offs, clamp, per_head):
    # mode 0: dK/dV scattered with fp32 atomics; modes 1, 2: gathered per key through the inverse index
    # (deterministic), the per-query pass on LDS tiles (1, fp16 only) or on the direct kernel (2)
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r = 2, 13, 17, 4, 32, 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=77, offsets=offs, clamp=clamp, per_head=per_head)
    g = torch.Generator().manual_seed(3)
    d_out = torch.randn(B, H * W, h * Ch, generator=g).to(dt)
    d_attn = torch.randn(B, H * W, h, 36, generator=g).to(dt)
    try:
        _cabi.set_option("backward_mode", mode)
        got = hip_backward(hip_lib, *_dev(mo, q, k, v), H, W, r, 0.2, d_out.cuda(), d_attn.cuda())
        if mode >= 1:   # deterministic: a second run is bit-identical
            again = hip_backward(hip_lib, *_dev(mo, q, k, v), H, W, r, 0.2, d_out.cuda(), d_attn.cuda())
            assert all(torch.equal(a, b) for a, b in zip(got, again))
    finally:
        _cabi.set_option("backward_mode", -1)
    check_grads(got, mo, q, k, v, H, W, r, 0.2, d_out, d_attn, f"backward_mode {mode} bwd")


@pytest.mark.parametrize("offs,per_head,clamp,Ch,r,shape,with_dattn", [
    ("interior", True, True, 32, 2, (2, 23, 41, 4), True), ("stereo", False, True, 32, 2, (1, 37, 70, 8), True),
    ("mixed", True, False, 32, 1, (2, 23, 41, 4), True), ("mixed", False, False, 64, 2, (1, 19, 50, 2), False),
    ("mixed", True, True, 16, 2, (1, 40, 33, 8), True), ("stereo", True, True, 64, 1, (3, 9, 17, 2), False),
    ("mixed", True, True, 32, 2, (2, 6, 7, 2), True), ("interior", False, True, 16, 1, (1, 8, 130, 4), True),
    # three images whose last strip of tiles is 2 wide, one offset per pixel (the blocked layout of the pair array)
    ("mixed", False, True, 32, 2, (3, 20, 150, 2), True)])
@pytest.mark.parametrize("dt", [torch.float16, torch.float32, torch.bfloat16], ids=["f16", "f32", "bf16"])
def test_lds_tile_backward_matches_autograd(hip_lib, dt, offs, per_head, clamp, Ch, r, shape, with_dattn):
    # backward_mode=1: pass A on LDS tiles (bucketed queries; unclamped offsets exercise the flagged finishing run)
    from matchattention_amd import _cabi
    B, H, W, h = shape
    M = (2 * r + 2) ** 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=55, offsets=offs, per_head=per_head, clamp=clamp)
    g = torch.Generator().manual_seed(9)
    d_out = torch.randn(B, H * W, h * Ch, generator=g).to(dt)
    d_attn = torch.randn(B, H * W, h, M, generator=g).to(dt) if with_dattn else None
    scale = Ch ** -0.5
    dev = _dev(mo, q, k, v)
    try:
        _cabi.set_option("backward_mode", 1)
        got = hip_backward(hip_lib, *dev, H, W, r, scale, d_out.cuda(), d_attn.cuda() if with_dattn else None)
        name = _cabi.last_backward_kernel()
        again = hip_backward(hip_lib, *dev, H, W, r, scale, d_out.cuda(), d_attn.cuda() if with_dattn else None)
        _cabi.set_option("backward_mode", 2)
        direct = hip_backward(hip_lib, *dev, H, W, r, scale, d_out.cuda(), d_attn.cuda() if with_dattn else None)
    finally:
        _cabi.set_option("backward_mode", -1)
    assert name == "bwd_tile_" + {torch.float16: "f16", torch.float32: "f32", torch.bfloat16: "bf16"}[dt], name
    check_grads(got, mo, q, k, v, H, W, r, scale, d_out, d_attn, "lds-tile bwd")
    for a, c, d, nm in zip(got, again, direct, ("dq", "dk", "dv", "dmo")):
        assert torch.equal(a, c), nm                          # bucket order does not change a result
        assert rel_err(a.cpu(), d.cpu().double()) <= TOL[dt], nm     # the two pass-A kernels agree


@pytest.mark.parametrize("per_head", [True, False], ids=["per_head", "shared"])
@pytest.mark.parametrize("shape", [(1, 127, 128), (1, 130, 130), (3, 30, 40)], ids=lambda s: "x".join(map(str, s)))
def test_inverse_index_of_small_and_larger_maps(hip_lib, shape, per_head):
    # The per-key pass follows an inverse index (which queries sample each pixel).  Maps of up to 16384 pixels get it
    # from one workgroup per image and head, larger ones from the chain of count, scan, scatter and ordering kernels:
    # a map on either side of that size and a batch of small ones, with unclamped offsets of which a good share lies
    # outside the map, so that the bins along the border hold hundreds of entries.  Gradients against the oracle's,
    # and a second call bit for bit (the order inside a bin must not depend on the order of the atomics).
    B, H, W = shape
    h, Ch, r = 2, 16, 1
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float32, seed=313, offsets="mixed", clamp=False, per_head=per_head)
    g = torch.Generator().manual_seed(17)
    d_out = torch.randn(B, H * W, h * Ch, generator=g)
    d_attn = torch.randn(B, H * W, h, 16, generator=g)
    dev = _dev(mo, q, k, v)
    got = hip_backward(hip_lib, *dev, H, W, r, 0.25, d_out.cuda(), d_attn.cuda())
    again = hip_backward(hip_lib, *dev, H, W, r, 0.25, d_out.cuda(), d_attn.cuda())
    assert all(torch.equal(a, b) for a, b in zip(got, again))
    check_grads(got, mo, q, k, v, H, W, r, 0.25, d_out, d_attn, "inverse index bwd")


def test_backward_without_attention_gradient(hip_lib):
    B, H, W, h, Ch, r = 1, 9, 10, 2, 32, 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float32, seed=5)
    d_out = torch.randn(B, H * W, h * Ch, generator=torch.Generator().manual_seed(1))
    got = hip_backward(hip_lib, *_dev(mo, q, k, v), H, W, r, 0.2, d_out.cuda(), None)
    check_grads(got, mo, q, k, v, H, W, r, 0.2, d_out, None, "no-dattn bwd")


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("r", [1, 2])
def test_every_forward_variant_agrees(hip_lib, variant, r):
    from matchattention_amd import _cabi
    B, H, W, h, Ch = 1, 14, 19, 4, 32
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float16, seed=21 + r, offsets="stereo")
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], Ch ** -0.5)
    try:
        _cabi.set_option("forward_variant", variant)
        out, attn = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, Ch ** -0.5)
        name = _cabi.last_forward_kernel()
    finally:
        _cabi.set_option("forward_variant", -1)
    assert ("generic" in name) == (variant == 0), name
    assert rel_err(attn.cpu(), want_attn) <= 2e-3 and rel_err(out.cpu(), want_out) <= 2e-3


def test_row_skip_does_not_change_results(hip_lib):
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r = 1, 16, 32, 4, 32, 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float16, seed=33, offsets="stereo")
    args = _dev(mo, q, k, v)
    try:
        _cabi.set_option("stereo_row_skip", 0)
        out0, attn0 = hip_forward(hip_lib, *args, H, W, r, Ch ** -0.5)
    finally:
        _cabi.set_option("stereo_row_skip", 1)
    out1, attn1 = hip_forward(hip_lib, *args, H, W, r, Ch ** -0.5)
    # the window maximum may sit in the skipped row, so the two paths may differ by a final rounding
    assert rel_err(out0, out1) <= 1e-3 and rel_err(attn0, attn1) <= 1e-3
    a = attn1.view(B, H * W, h, 2 * r + 2, 2 * r + 2)
    assert (a[..., -1, :] == 0).all()          # integer y: the last window row has weight exactly 0


@pytest.mark.parametrize("offs,per_head,clamp,Ch,r,shape", [
    ("interior", True, True, 32, 2, (2, 23, 41, 4)), ("interior", False, True, 16, 1, (2, 23, 41, 4)),
    ("stereo", False, True, 32, 2, (1, 37, 70, 8)), ("mixed", True, True, 32, 2, (2, 23, 41, 4)),
    ("mixed", True, False, 32, 1, (2, 23, 41, 4)), ("mixed", False, False, 64, 2, (1, 19, 50, 2)),
    ("stereo", True, True, 64, 1, (3, 9, 17, 2)), ("mixed", True, False, 16, 2, (1, 40, 33, 8)),
    ("mixed", True, True, 32, 2, (2, 6, 7, 2)), ("interior", False, True, 16, 1, (1, 8, 130, 4)),
    # one tile row 188 tiles wide; one tile column 313 tiles tall; three images whose last strip of tiles is 2 wide
    ("stereo", False, True, 16, 2, (1, 6, 3000, 4)), ("mixed", True, True, 32, 2, (1, 2500, 7, 2)),
    ("mixed", False, True, 32, 2, (3, 20, 150, 2)),
    # heads of 64 channels, an odd number of them, a position per head and a shared one (16-bit types: two half-heads of 32)
    ("mixed", True, True, 64, 2, (2, 21, 37, 3)), ("stereo", False, True, 64, 2, (1, 30, 45, 1))])
@pytest.mark.parametrize("dt", [torch.float16, torch.float32, torch.bfloat16], ids=["f16", "f32", "bf16"])
def test_lds_tile_forward_matches_oracle(hip_lib, dt, offs, per_head, clamp, Ch, r, shape):
    # forward_lds=1: queries bucketed by K/V tile, every tap read from LDS; without the input clamp some
    # windows lie far outside the image and go through the deferred list
    from matchattention_amd import _cabi
    B, H, W, h = shape
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=77, offsets=offs, per_head=per_head, clamp=clamp)
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], Ch ** -0.5)
    try:
        _cabi.set_option("forward_lds", 1)
        out, attn = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, Ch ** -0.5)
        name = _cabi.last_forward_kernel()
        out2, attn2 = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, Ch ** -0.5)
    finally:
        _cabi.set_option("forward_lds", -1)
    assert name.startswith("fwd_tile_" + {torch.float16: "f16", torch.float32: "f32", torch.bfloat16: "bf16"}[dt]), name
    assert torch.isfinite(out).all() and torch.isfinite(attn).all()
    assert rel_err(attn.cpu(), want_attn) <= TOL[dt] and rel_err(out.cpu(), want_out) <= TOL[dt]
    assert torch.equal(out, out2) and torch.equal(attn, attn2)       # the bucket order does not change a result


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_full_size_tile_path_in_fp32_and_bf16(hip_lib, dt):
    # the same at the benchmark's largest map in the other storage types: the LDS-tile kernel against the direct
    # one (per-head positions), nothing deferred, attention rows sum to one
    import dataclasses
    from matchattention_amd import _cabi
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    wl = WORKLOADS["cfg3_self"]
    inp = make_inputs(wl)
    H, W = inp["H"], inp["W"]
    mo, q, k, v = (inp[n].to(dt) for n in ("max_offset", "q", "k", "v"))
    del inp
    res, left = {}, []
    try:
        for mode in (0, -1):
            _cabi.set_option("forward_lds", mode)
            res[mode] = hip_forward(hip_lib, mo, q, k, v, H, W, wl.r, wl.scale, deferred=left) + (_cabi.last_forward_kernel(),)
    finally:
        _cabi.set_option("forward_lds", -1)
    tag = "f32" if dt == torch.float32 else "bf16"
    assert res[-1][2].startswith("fwd_tile_" + tag) and res[0][2].startswith("fwd_tiled_" + tag), (res[0][2], res[-1][2])
    assert left == [-1, 0], left
    for a, b in zip(res[0][:2], res[-1][:2]):
        assert torch.isfinite(b).all()
        assert float((a.float() - b.float()).abs().max() / a.float().abs().max()) <= TOL[dt]
    assert float((res[-1][1].float().sum(-1) - 1).abs().max()) <= {torch.float32: 1e-5, torch.bfloat16: 4e-2}[dt]


@pytest.mark.parametrize("name,field", [("cfg3_cross", False), ("cfg4_self", False), ("cfg3_cross", "scene"), ("cfg3_cross", True)],
                         ids=["cfg3_cross", "cfg4_self", "cfg3_cross_scene_field", "cfg3_cross_smooth_field"])
def test_full_size_tile_and_direct_paths_agree(hip_lib, name, field):
    # at the benchmark's full sizes the oracle is too slow: the two HIP paths (LDS tiles / direct gather) must
    # agree with each other, attention rows must sum to one and a constant V must come back unchanged -- on the
    # i.i.d. fields of the benchmark and on spatially coherent ones (a stereo scene's, and the blurred field)
    from matchattention_amd import _cabi
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    wl = WORKLOADS[name]
    inp = make_inputs(wl, smooth=field)
    H, W = inp["H"], inp["W"]
    res = {}
    left = []
    try:
        for mode in (0, 1):
            _cabi.set_option("forward_lds", mode)
            res[mode] = hip_forward(hip_lib, inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale, deferred=left)
            res[mode] = res[mode] + (_cabi.last_forward_kernel(),)
        _cabi.set_option("forward_lds", 1)
        vconst = torch.full_like(inp["v"], 0.75)
        out_c, _ = hip_forward(hip_lib, inp["max_offset"], inp["q"], inp["k"], vconst, H, W, wl.r, wl.scale)
    finally:
        _cabi.set_option("forward_lds", -1)
    assert res[1][2].startswith("fwd_tile_f16") and res[0][2].startswith("fwd_tiled_f16"), (res[0][2], res[1][2])
    # the tile kernel itself serves these fields (shared and per-head positions): next to nothing is left to the
    # direct kernel, which would give the same results at a fraction of the speed
    assert left[0] == -1 and 0 <= left[1] <= inp["q"].shape[0] * inp["q"].shape[1] * wl.h // 1000, left
    for a, b in zip(res[0][:2], res[1][:2]):
        assert torch.isfinite(b).all()
        assert float((a.float() - b.float()).abs().max() / a.float().abs().max()) <= 2e-3
    assert float((res[1][1].float().sum(-1) - 1).abs().max()) <= 4e-3
    assert float((out_c.float() - 0.75).abs().max()) <= 2e-3


def test_full_size_backward_paths_agree(hip_lib):
    # cfg4 (2 x 384 x 384, C=256, 8 heads, r=2, 2-D offsets): pass A on LDS tiles against pass A on the direct
    # kernel, bit equality of a second run, and linearity in dO
    from matchattention_amd import _cabi
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    wl = WORKLOADS["cfg4_cross"]
    inp = make_inputs(wl)
    H, W = inp["H"], inp["W"]
    args = (inp["max_offset"], inp["q"], inp["k"], inp["v"], H, W, wl.r, wl.scale)
    try:
        _cabi.set_option("backward_mode", 1)
        tile = hip_backward(hip_lib, *args, inp["d_out"], inp["d_attn"])
        name = _cabi.last_backward_kernel()
        again = hip_backward(hip_lib, *args, inp["d_out"], inp["d_attn"])
        twice = hip_backward(hip_lib, *args, inp["d_out"] * 2, inp["d_attn"] * 2)
        _cabi.set_option("backward_mode", 2)
        direct = hip_backward(hip_lib, *args, inp["d_out"], inp["d_attn"])
    finally:
        _cabi.set_option("backward_mode", -1)
    assert name == "bwd_tile_f16", name
    for a, b, c, d, nm in zip(tile, again, direct, twice, ("dq", "dk", "dv", "dmo")):
        assert torch.isfinite(a).all(), nm
        assert torch.equal(a, b), nm
        ref = c.float().abs().max()
        assert float((a.float() - c.float()).abs().max() / ref) <= 2e-3, nm
        assert float((d.float() - 2 * a.float()).abs().max() / (2 * ref)) <= 2e-3, nm      # doubling dO, dA doubles every gradient


def test_kernel_timer_reports_the_dominant_kernel(hip_lib):
    # off by default; when on, the time between the library's two events is positive and below the wall time of
    # the call, on the tile path (several kernels per call) and on the direct one
    import time
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r = 1, 64, 96, 4, 32, 2
    dev = _dev(*make_case(B, H, W, h, Ch, r, torch.float16, seed=5, offsets="stereo", per_head=False))
    assert hip_lib.matchattn_last_forward_kernel_ms() < 0
    try:
        _cabi.set_option("time_kernels", 1)
        for lds in (1, 0):
            _cabi.set_option("forward_lds", lds)
            hip_forward(hip_lib, *dev, H, W, r, 0.2)
            t0 = time.perf_counter()
            hip_forward(hip_lib, *dev, H, W, r, 0.2)
            wall = (time.perf_counter() - t0) * 1e3
            ms = float(hip_lib.matchattn_last_forward_kernel_ms())
            assert 0 < ms < wall, (lds, ms, wall)
    finally:
        _cabi.set_option("forward_lds", -1)
        _cabi.set_option("time_kernels", 0)
    assert hip_lib.matchattn_last_forward_kernel_ms() < 0


def test_lds_tile_forward_defers_the_exact_softmax(hip_lib):
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r = 1, 12, 12, 2, 32, 1
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float16, seed=41, offsets="interior")
    k = (k.float() * 30.0).half()
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], 1.0)
    left = []
    try:
        _cabi.set_option("forward_lds", 1)
        out, attn = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, 1.0, deferred=left)
    finally:
        _cabi.set_option("forward_lds", -1)
    assert left[0] > 0                       # some windows did go to the exact softmax of the direct kernel
    assert torch.isfinite(attn).all()
    assert rel_err(attn.cpu(), want_attn) <= 2e-3 and rel_err(out.cpu(), want_out) <= 2e-3


def test_far_apart_subwindows_take_the_exact_softmax(hip_lib):
    # One key is made enormously closer than the rest so that sub-windows not containing it
    # sit > 60 below the window maximum: the shared-exponential shortcut must not be used.
    B, H, W, h, Ch, r = 1, 8, 8, 1, 8, 1
    mo, q, k, v = make_case(B, H, W, h, Ch, r, torch.float32, seed=41, offsets="interior")
    k = k * 40.0
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], 1.0)
    out, attn = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, 1.0)
    assert torch.isfinite(attn).all()
    assert rel_err(attn.cpu(), want_attn) <= 1e-5 and rel_err(out.cpu(), want_out) <= 1e-5
    assert torch.allclose(attn.sum(-1).cpu(), torch.ones(B, H * W, h), atol=1e-5)


def test_argument_errors_are_reported(hip_lib):
    from matchattention_amd import _cabi
    t = torch.zeros(1, 64, 8, device="cuda")
    mo = torch.zeros(1, 64, 1, 2, device="cuda")
    attn = torch.zeros(1, 64, 1, 16, device="cuda")
    s = torch.cuda.current_stream().cuda_stream
    p = lambda x: x.data_ptr()
    assert hip_lib.matchattn_forward(p(mo), p(t), p(t), p(t), p(t), p(attn), 1, 8, 8, 8, 1, 1, 2, 1.0, 0, s) == 1
    assert b"square" in hip_lib.matchattn_last_error()
    assert hip_lib.matchattn_forward(p(mo), p(t), p(t), p(t), p(t), p(attn), 1, 8, 8, 8, 3, 1, 1, 1.0, 0, s) == 1
    assert hip_lib.matchattn_forward(p(mo), p(t), p(t), p(t), p(t), p(attn), 1, 8, 8, 8, 1, 1, 1, 1.0, 7, s) == 1
    assert hip_lib.matchattn_forward(None, p(t), p(t), p(t), p(t), p(attn), 1, 8, 8, 8, 1, 1, 1, 1.0, 0, s) == 1
    assert hip_lib.matchattn_forward(p(mo), p(t), p(t), p(t), p(t), p(attn), 1, 3, 8, 8, 1, 1, 1, 1.0, 0, s) == 1
    h16 = t.half()
    assert hip_lib.matchattn_backward(p(mo), p(h16), p(h16), p(h16), p(h16), None, p(h16), p(h16), p(h16), p(mo),
                                      None, 0, 1, 8, 8, 8, 1, 1, 1, 1.0, 1, s) == 2
    assert b"workspace" in hip_lib.matchattn_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("tiles", [False, True])
def test_calls_replay_from_a_hip_graph(hip_lib, tiles):
    # the C ABI allocates nothing, copies nothing between host and device and clears its scratch with kernels:
    # a forward + backward pair captured once must give the eager results on every replay
    from matchattention_amd import _cabi
    from tests.gpu_util import DT
    B, H, W, h, Ch, r = 1, 21, 34, 4, 32, 2
    M, C = 36, h * Ch
    mo, q, k, v = (t.cuda() for t in make_case(B, H, W, h, Ch, r, torch.float16, seed=123, offsets="mixed"))
    g = torch.Generator().manual_seed(4)
    d_out = torch.randn(B, H * W, C, generator=g).half().cuda()
    d_attn = torch.randn(B, H * W, h, M, generator=g).half().cuda()
    try:
        _cabi.set_option("forward_lds", 1 if tiles else 0)
        _cabi.set_option("backward_mode", 1 if tiles else 2)
        want_f = hip_forward(hip_lib, mo, q, k, v, H, W, r, 0.2)
        want_b = hip_backward(hip_lib, mo, q, k, v, H, W, r, 0.2, d_out, d_attn)
        dt = DT[torch.float16]
        nf = hip_lib.matchattn_forward_workspace_bytes(B, H, W, C, h, r, r, dt)
        nb = hip_lib.matchattn_backward_workspace_bytes(B, H, W, C, h, r, r, dt)
        wsf = torch.empty(max(nf, 16), dtype=torch.uint8, device="cuda")
        wsb = torch.empty(max(nb, 16), dtype=torch.uint8, device="cuda")
        out, attn = torch.empty_like(q), torch.empty(B, H * W, h, M, dtype=q.dtype, device="cuda")
        dq, dk, dv, dmo = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q), torch.empty_like(mo)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            def calls():
                s = torch.cuda.current_stream().cuda_stream
                _cabi.check(hip_lib.matchattn_forward_ws(mo.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                         attn.data_ptr(), wsf.data_ptr() if nf else None, nf, B, H, W, C, h, r, r,
                                                         0.2, dt, s))
                _cabi.check(hip_lib.matchattn_backward(mo.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), d_out.data_ptr(),
                                                       d_attn.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                                       dmo.data_ptr(), wsb.data_ptr(), nb, B, H, W, C, h, r, r, 0.2, dt, s))
            calls()                                   # warm-up outside the capture
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                calls()
        for rep in range(3):
            for t in (out, attn, dq, dk, dv, dmo):
                t.fill_(float("nan"))
            wsf.random_(0, 255)                       # stale scratch must not matter
            wsb.random_(0, 255)
            (q * 2).sum().item()                      # eager work and a synchronisation between the replays
            graph.replay()
            torch.cuda.synchronize()
            for got, want, name in zip((out, attn, dq, dk, dv, dmo), want_f + want_b, ("out", "attn", "dq", "dk", "dv", "dmo")):
                assert torch.equal(got, want), (name, rep)
    finally:
        _cabi.set_option("forward_lds", -1)
        _cabi.set_option("backward_mode", -1)


def _module_steps(rel, q, k, v, gate, H, W, r, h, attend):
    """The attention module's own sequence around the operator (reference models/attention_blocks.py:149-151 /
    162-163 for the coordinate add, :45-59 for the clamp, :96-98 for gate and concatenation), in torch ops."""
    B, N, C = q.shape
    dt = q.dtype
    ys, xs = torch.meshgrid(torch.arange(H, device=q.device, dtype=dt), torch.arange(W, device=q.device, dtype=dt), indexing="ij")
    grid = torch.stack((xs, ys), -1).reshape(1, N, 1, 2)
    mo = (rel.expand(B, N, h, 2) + grid).contiguous()
    lo = torch.tensor(float(r), dtype=dt, device=q.device)
    hx = torch.tensor(W - 1 - r - 1e-3, dtype=dt, device=q.device)
    hy = torch.tensor(H - 1 - r - 1e-3, dtype=dt, device=q.device)
    mo = torch.cat((torch.clamp(mo[..., 0:1], min=lo, max=hx), torch.clamp(mo[..., 1:2], min=lo, max=hy)), -1).contiguous()
    out, attn = attend(mo, q, k, v)
    if gate is not None:
        out = gate * out
    return mo, out, attn, torch.cat((out, attn.reshape(B, N, -1)), -1)


@pytest.mark.parametrize("dt,Ch,h,r,shape,shared,gated,opt", [
    (torch.float16, 32, 4, 2, (2, 23, 41), True, True, ("forward_lds", 1)),      # LDS tiles, cross-attention form
    (torch.float16, 32, 4, 2, (2, 23, 41), False, False, ("forward_lds", 1)),    # LDS tiles, self-attention form
    (torch.float16, 16, 8, 1, (1, 30, 37), False, True, ("forward_lds", 0)),     # direct gather
    (torch.float16, 40, 4, 2, (2, 12, 20), True, True, ("forward_lds", 0)),      # padded lane groups
    (torch.float32, 16, 4, 1, (2, 15, 22), True, True, ("forward_lds", -1)),
    (torch.bfloat16, 32, 2, 2, (1, 8, 300), True, True, ("forward_lds", -1)),    # x beyond bf16's exact integers
    (torch.float16, 32, 4, 2, (1, 17, 19), False, True, ("forward_variant", 0)),  # generic kernel
    (torch.float16, 64, 4, 2, (2, 23, 41), True, True, ("forward_lds", 1)),      # LDS tiles, heads of 64 channels as two half-heads
    (torch.bfloat16, 64, 2, 2, (1, 21, 40), False, True, ("forward_lds", 1)),
    (torch.float32, 80, 2, 2, (1, 12, 20), True, True, ("forward_lds", -1)),     # two vectors per lane
])
def test_fused_module_forward_is_bit_identical_to_the_separate_steps(hip_lib, dt, Ch, h, r, shape, shared, gated, opt):
    from matchattention_amd import _cabi, fused_module_forward
    B, H, W = shape
    N, C, M = H * W, h * Ch, (2 * r + 2) ** 2
    g = torch.Generator().manual_seed(5)
    q, k, v, gate = (torch.randn(B, N, C, generator=g).to(dt).cuda() for _ in range(4))
    rel = torch.randn(B, N, 1 if shared else h, 2, generator=g) * 0.3 * max(H, W)     # many land outside: the clamp acts
    rel = torch.where(torch.rand(B, N, rel.size(2), 1, generator=g) < 0.2, rel.round(), rel).to(dt).cuda()
    scale = Ch ** -0.5
    try:
        _cabi.set_option(*opt)
        mo, out, attn, cat = _module_steps(rel, q, k, v, gate if gated else None, H, W, r, h,
                                           lambda mo, q, k, v: hip_forward(hip_lib, mo, q, k, v, H, W, r, scale))
        unfused_kernel = _cabi.last_forward_kernel()
        got_cat = fused_module_forward(rel, q, k, v, H, W, [r, r], h, scale, gate=gate if gated else None, concat=True)
        assert _cabi.last_forward_kernel() == unfused_kernel
        got_out, got_attn = fused_module_forward(rel, q, k, v, H, W, [r, r], h, scale, gate=gate if gated else None)
        # sampling positions given (no coordinate add), outputs still placed and gated
        got_cat0 = fused_module_forward(mo, q, k, v, H, W, [r, r], h, scale, gate=gate if gated else None,
                                        relative=False, concat=True)
        torch.cuda.synchronize()
    finally:
        _cabi.set_option(opt[0], -1)
    assert torch.isfinite(cat.float()).all()
    assert torch.equal(got_cat, cat) and torch.equal(got_cat0, cat)
    assert torch.equal(got_out, out) and torch.equal(got_attn, attn)
    # and the whole sequence against the CPU oracle
    want_mo = O.clamp_max_offset((rel.cpu().expand(B, N, h, 2) + O.init_coords(B, H, W).view(B, N, 1, 2).to(dt)).contiguous(),
                                 H, W, [r, r])
    assert torch.equal(want_mo, mo.cpu())
    want_out, want_attn = O.forward(want_mo, q.cpu(), k.cpu(), v.cpu(), H, W, [r, r], scale)
    if gated:
        want_out = gate.cpu() * want_out
    tol = TOL[dt]
    assert rel_err(got_out.cpu(), want_out) <= tol and rel_err(got_attn.cpu(), want_attn) <= tol


def test_fused_concat_rows_that_are_not_whole_16_byte_pieces(hip_lib):
    # one head at r = 2: the concatenated row is C + 36 halves, 8 bytes short of a multiple of 16, so the vector kernels'
    # 16-byte stores cannot be used and the fused call takes the generic kernel -- same results to the tolerance, not
    # to the bit, as the separate steps (which write contiguous tensors through the vector kernel)
    from matchattention_amd import _cabi, fused_module_forward
    dt, Ch, h, r, (B, H, W) = torch.float16, 32, 1, 2, (2, 21, 30)
    N, C = H * W, h * Ch
    g = torch.Generator().manual_seed(8)
    q, k, v, gate = (torch.randn(B, N, C, generator=g).to(dt).cuda() for _ in range(4))
    rel = (torch.randn(B, N, 1, 2, generator=g) * 6.0).to(dt).cuda()
    scale = Ch ** -0.5
    mo, out, attn, cat = _module_steps(rel, q, k, v, gate, H, W, r, h,
                                       lambda mo, q, k, v: hip_forward(hip_lib, mo, q, k, v, H, W, r, scale))
    assert _cabi.last_forward_kernel().startswith("fwd_tiled_f16")
    got_cat = fused_module_forward(rel, q, k, v, H, W, [r, r], h, scale, gate=gate, concat=True)
    assert _cabi.last_forward_kernel().startswith("fwd_generic_f16"), _cabi.last_forward_kernel()
    got_out, got_attn = fused_module_forward(rel, q, k, v, H, W, [r, r], h, scale, gate=gate)     # contiguous outputs
    assert _cabi.last_forward_kernel().startswith("fwd_tiled_f16")
    assert torch.equal(got_out, out) and torch.equal(got_attn, attn)
    assert torch.isfinite(got_cat).all()
    want_out, want_attn = O.forward(mo.cpu(), q.cpu(), k.cpu(), v.cpu(), H, W, [r, r], scale)
    want_out = gate.cpu() * want_out
    assert rel_err(got_cat[..., :C].cpu(), want_out) <= TOL[dt]
    assert rel_err(got_cat[..., C:].reshape(B, N, h, -1).cpu(), want_attn) <= TOL[dt]


def test_fused_forward_accepts_any_row_stride(hip_lib):
    # rows that are not a multiple of 16 bytes leave the vector kernels; results stay the same
    from matchattention_amd import _cabi
    from tests.gpu_util import DT
    B, H, W, h, Ch, r = 1, 14, 18, 4, 16, 1
    N, C, M = H * W, h * Ch, 16
    mo, q, k, v = _dev(*make_case(B, H, W, h, Ch, r, torch.float16, seed=3))
    out, attn = hip_forward(hip_lib, mo, q, k, v, H, W, r, 0.25)
    so, sa = C + 3, h * M + 5
    obuf = torch.full((B, N, so), 7.0, dtype=q.dtype, device=q.device)
    abuf = torch.full((B, N, sa), 7.0, dtype=q.dtype, device=q.device)
    _cabi.check(hip_lib.matchattn_forward_fused(mo.data_ptr(), 0, q.data_ptr(), k.data_ptr(), v.data_ptr(), None,
                                                obuf.data_ptr(), so, abuf.data_ptr(), sa, None, 0,
                                                B, H, W, C, h, r, r, 0.25, DT[q.dtype], torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert _cabi.last_forward_kernel().startswith("fwd_generic")
    assert torch.equal(obuf[..., :C], out) and torch.equal(abuf[..., :h * M], attn.reshape(B, N, -1))
    assert (obuf[..., C:] == 7).all() and (abuf[..., h * M:] == 7).all()      # nothing written between the rows
    # strides shorter than a row are refused
    rc = hip_lib.matchattn_forward_fused(mo.data_ptr(), 0, q.data_ptr(), k.data_ptr(), v.data_ptr(), None, obuf.data_ptr(), C - 1,
                                         abuf.data_ptr(), sa, None, 0, B, H, W, C, h, r, r, 0.25, DT[q.dtype], None)
    assert rc != 0 and "stride" in hip_lib.matchattn_last_error().decode()


def _sweep_cases(n=48, seed=2024):
    import random
    rnd = random.Random(seed)
    cases = []
    while len(cases) < n:
        dt = rnd.choice([torch.float32, torch.float16, torch.float16, torch.bfloat16])
        r = rnd.choice([1, 1, 2, 2, 3])
        Ch = rnd.choice([8, 16, 32, 40, 64] if dt != torch.float32 else [4, 8, 16, 32, 40]) if rnd.random() < 0.85 else rnd.choice([12, 20, 24])
        h = rnd.choice([1, 2, 3, 4, 5, 6, 8])
        B = rnd.choice([1, 1, 2, 3])
        H, W = rnd.randint(2 * r + 2, 30), rnd.randint(2 * r + 2, 45)
        if B * H * W * h * Ch > 400_000:
            continue
        cases.append((B, H, W, h, Ch, r, dt, rnd.choice(["mixed", "stereo", "interior"]), rnd.random() < 0.6, rnd.random() < 0.6,
                      rnd.choice([-1, 1]), rnd.choice([-1, 0, 1, 2]), len(cases)))
    return cases


@pytest.mark.parametrize("case", _sweep_cases(), ids=lambda c: f"{c[12]}_{str(c[6]).split('.')[1]}_B{c[0]}_{c[1]}x{c[2]}_h{c[3]}_ch{c[4]}_r{c[5]}_{c[7]}_lds{c[10]}_bm{c[11]}")
def test_random_shapes_match_oracle(hip_lib, case):
    # a seeded sweep over shapes (odd head counts, head sizes without a vector kernel, maps barely larger than the
    # window, every dtype) and over the kernel choices the options allow; forward and backward against the oracle
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r, dt, offs, clamp, per_head, lds, bmode, idx = case
    M = (2 * r + 2) ** 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=500 + idx, offsets=offs, clamp=clamp, per_head=per_head)
    scale = Ch ** -0.5
    g = torch.Generator().manual_seed(idx)
    d_out = torch.randn(B, H * W, h * Ch, generator=g).to(dt)
    d_attn = torch.randn(B, H * W, h, M, generator=g).to(dt) if idx % 3 else None
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], scale)
    dev = _dev(mo, q, k, v)
    try:
        _cabi.set_option("forward_lds", lds)
        _cabi.set_option("backward_mode", bmode)
        out, attn = hip_forward(hip_lib, *dev, H, W, r, scale)
        got = hip_backward(hip_lib, *dev, H, W, r, scale, d_out.cuda(), None if d_attn is None else d_attn.cuda())
    finally:
        _cabi.set_option("forward_lds", -1)
        _cabi.set_option("backward_mode", -1)
    tol = TOL[dt]
    assert torch.isfinite(out).all() and torch.isfinite(attn).all()
    assert rel_err(attn.cpu(), want_attn) <= tol and rel_err(out.cpu(), want_out) <= tol
    check_grads(got, mo, q, k, v, H, W, r, scale, d_out, d_attn, "random shapes bwd")


def _big_head_cases(n=16, seed=4711):
    import random
    rnd = random.Random(seed)
    cases = []
    while len(cases) < n:
        dt = rnd.choice([torch.float32, torch.float32, torch.float16, torch.bfloat16])
        Ch = rnd.choice([80, 96, 128, 192])
        r = rnd.choice([1, 2])
        h = rnd.choice([1, 2, 3, 4])
        B = rnd.choice([1, 2])
        H, W = rnd.randint(2 * r + 2, 14), rnd.randint(2 * r + 2, 18)
        if B * H * W * h * Ch > 150_000:
            continue
        cases.append((B, H, W, h, Ch, r, dt, rnd.choice(["mixed", "stereo", "interior"]), rnd.random() < 0.6, rnd.random() < 0.6,
                      rnd.choice([-1, 0, 2]), len(cases)))
    return cases


@pytest.mark.parametrize("case", _big_head_cases(), ids=lambda c: f"{c[11]}_{str(c[6]).split('.')[1]}_B{c[0]}_{c[1]}x{c[2]}_h{c[3]}_ch{c[4]}_r{c[5]}_{c[7]}_bm{c[10]}")
def test_heads_of_more_than_sixteen_vectors_match_oracle(hip_lib, case):
    # heads of 80 to 192 channels (the coarse levels of the reference's larger variants): two vectors per lane in the
    # forward and the per-key pass, 32 lanes per head-query in the per-query pass; seeded shapes with odd head counts
    # and maps barely larger than the window, in every type and in the gathering and the scattering backward
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r, dt, offs, clamp, per_head, bmode, idx = case
    M = (2 * r + 2) ** 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=900 + idx, offsets=offs, clamp=clamp, per_head=per_head)
    scale = Ch ** -0.5
    g = torch.Generator().manual_seed(idx)
    d_out = torch.randn(B, H * W, h * Ch, generator=g).to(dt)
    d_attn = torch.randn(B, H * W, h, M, generator=g).to(dt) if idx % 3 else None
    want_out, want_attn = O.forward(mo, q, k, v, H, W, [r, r], scale)
    dev = _dev(mo, q, k, v)
    try:
        _cabi.set_option("backward_mode", bmode)
        out, attn = hip_forward(hip_lib, *dev, H, W, r, scale)
        assert "generic" not in _cabi.last_forward_kernel(), _cabi.last_forward_kernel()
        got = hip_backward(hip_lib, *dev, H, W, r, scale, d_out.cuda(), None if d_attn is None else d_attn.cuda())
        assert "generic" not in _cabi.last_backward_kernel(), _cabi.last_backward_kernel()
    finally:
        _cabi.set_option("backward_mode", -1)
    tol = TOL[dt]
    assert torch.isfinite(out).all() and torch.isfinite(attn).all()
    assert rel_err(attn.cpu(), want_attn) <= tol and rel_err(out.cpu(), want_out) <= tol
    check_grads(got, mo, q, k, v, H, W, r, scale, d_out, d_attn, "big heads bwd")


@pytest.mark.parametrize("tiles", [False, True])
def test_fused_call_replays_from_a_hip_graph(hip_lib, tiles):
    # the fused entry point touches nothing on the host (on the LDS-tile path it adds one small kernel that writes the
    # sampling positions into the workspace; otherwise the one kernel that runs adds the pixel grid and clamps
    # itself and there is no scratch at all): captured once, every replay over stale scratch gives the eager result
    from matchattention_amd import _cabi, fused_module_forward
    from tests.gpu_util import DT
    B, H, W, h, Ch, r = 2, 19, 27, 4, 32, 2
    N, C, M = H * W, h * Ch, 36
    g = torch.Generator().manual_seed(8)
    q, k, v, gate = (torch.randn(B, N, C, generator=g).half().cuda() for _ in range(4))
    rel = (torch.randn(B, N, 1, 2, generator=g) * 9).half().cuda()
    try:
        _cabi.set_option("forward_lds", 1 if tiles else 0)
        want = fused_module_forward(rel, q, k, v, H, W, [r, r], h, 0.2, gate=gate, concat=True)
        dt = DT[torch.float16]
        n = hip_lib.matchattn_forward_fused_workspace_bytes(B, H, W, C, h, r, r, dt)
        ws = torch.empty(n, dtype=torch.uint8, device="cuda")
        buf = torch.empty(B, N, C + h * M, dtype=q.dtype, device="cuda")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            def call():
                _cabi.check(hip_lib.matchattn_forward_fused(
                    rel.data_ptr(), 1, q.data_ptr(), k.data_ptr(), v.data_ptr(), gate.data_ptr(), buf.data_ptr(), C + h * M,
                    buf.data_ptr() + C * 2, C + h * M, ws.data_ptr(), n, B, H, W, C, h, r, r, 0.2, dt,
                    torch.cuda.current_stream().cuda_stream))
            call()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph, stream=side):
                call()
        for rep in range(3):
            buf.fill_(float("nan"))
            ws.random_(0, 255)
            (q * 2).sum().item()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(buf, want), rep
    finally:
        _cabi.set_option("forward_lds", -1)


@pytest.mark.parametrize("dt,lds,bmode", [(torch.float16, 1, 1), (torch.float16, 0, 2), (torch.float32, -1, -1), (torch.bfloat16, -1, 0)])
def test_non_finite_offsets_stay_local(hip_lib, dt, lds, bmode):
    # NaN / inf / huge sampling positions (a diverged field) must neither fault nor disturb other queries: every
    # coordinate is bounded before it enters index arithmetic.  (Regression test: +inf used to convert to INT_MAX, and
    # `centre + tap` then overflowed past the compiler's folded clamp into a negative index in the generic kernel.)
    from matchattention_amd import _cabi
    B, H, W, h, Ch, r = 1, 18, 25, 4, 32, 2
    M = (2 * r + 2) ** 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=31, offsets="interior")
    bad = mo.clone()
    poison = [float("nan"), float("inf"), -float("inf"), 6.0e4, -6.0e4, 3.0e38 if dt != torch.float16 else 6.5e4]
    rows = torch.arange(7, 7 + len(poison)) * 11                      # a few scattered queries
    for n, val in zip(rows.tolist(), poison):
        bad[0, n, :, 0] = val
        bad[0, n + 1, 1, 1] = val
    touched = torch.zeros(H * W, dtype=torch.bool)
    touched[rows] = True
    touched[rows + 1] = True
    g = torch.Generator().manual_seed(1)
    d_out = torch.randn(B, H * W, h * Ch, generator=g).to(dt).cuda()
    d_attn = torch.randn(B, H * W, h, M, generator=g).to(dt).cuda()
    try:
        _cabi.set_option("forward_lds", lds)
        _cabi.set_option("backward_mode", bmode)
        good_f = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, 0.2)
        bad_f = hip_forward(hip_lib, *_dev(bad, q, k, v), H, W, r, 0.2)
        good_b = hip_backward(hip_lib, *_dev(mo, q, k, v), H, W, r, 0.2, d_out, d_attn)
        bad_b = hip_backward(hip_lib, *_dev(bad, q, k, v), H, W, r, 0.2, d_out, d_attn)
    finally:
        _cabi.set_option("forward_lds", -1)
        _cabi.set_option("backward_mode", -1)
    keep = ~touched.cuda()
    for a, b in zip(good_f, bad_f):
        assert torch.equal(a[0, keep], b[0, keep])
    assert torch.equal(good_b[0][0, keep], bad_b[0][0, keep])            # dq and d max_offset are per query
    assert torch.equal(good_b[3][0, keep], bad_b[3][0, keep])
    # huge finite positions are well defined (every tap is a border pixel): finite outputs.  NaN and +-inf have no
    # fractional part (inf - inf), so their own rows are NaN, as in the definition.
    finite_rows = torch.cat((rows[3:], rows[3:] + 1)).cuda()
    assert torch.isfinite(bad_f[0][0, finite_rows]).all() and torch.isfinite(bad_f[1][0, finite_rows]).all()


@pytest.mark.parametrize("Ch", [32, 64])
@pytest.mark.parametrize("dt,big", [(torch.float16, 6.0e4), (torch.bfloat16, 3.0e38)], ids=["f16", "bf16"])
def test_non_finite_values_stay_local_on_the_matrix_unit(hip_lib, dt, big, Ch):
    # The 16-bit LDS-tile kernel adds the |q - k| of a lane pair with a matrix instruction whose zero entries multiply the
    # values of the other head-queries of the wavefront: 0 * inf = NaN.  A non-finite q or k value (or a difference
    # that overflows: 6e4 - (-6e4) in fp16, 3e38 - (-3e38) in bf16) must only change the queries that own it or whose window reaches it.
    # (Heads of 64 channels run on the same kernel as two half-heads of 32, whose sums meet before the softmax and whose
    # outputs are checked together: the poisoned channels lie in either half, and V is poisoned as well -- the
    # aggregation multiplies the V values of a whole row of the tile by the zeros of the queries that do not reach them.)
    from matchattention_amd import _cabi
    B, H, W, h, r = 1, 40, 50, 4, 2
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=77, offsets="interior", per_head=False)
    qb, kb, vb = q.clone(), k.clone(), v.clone()
    q_poison = {5 * W + 7: float("inf"), 17 * W + 30: float("nan"), 30 * W + 12: big}
    k_poison = {9 * W + 40: -float("inf"), 22 * W + 21: float("nan"), 33 * W + 5: -big}
    for n, val in q_poison.items():
        qb[0, n, 3] = val
        qb[0, n, Ch + 9] = val
    for n, val in k_poison.items():
        kb[0, n, 2 * Ch + 1] = val
        vb[0, n, 3 * Ch - 3] = val                       # (head 2, its last channels)
    qb[0, 5 * W + 7, Ch - 5] = float("nan")              # (head 0, its last channels)
    # the query of the large entry reaches keys that hold its negative in the same channel: the difference overflows
    kb[0, 30 * W + 12, 3] = -big
    k_bad = set(k_poison) | {30 * W + 12}
    ix = torch.floor(mo[0, :, 0, 0].float()).long()
    iy = torch.floor(mo[0, :, 0, 1].float()).long()
    touched = torch.zeros(H * W, dtype=torch.bool)
    touched[list(q_poison)] = True
    taps = torch.arange(-r, r + 2)
    xs = (ix[:, None] + taps[None]).clamp(0, W - 1)          # [N, 2r+2]
    ys = (iy[:, None] + taps[None]).clamp(0, H - 1)
    for n in k_bad:
        py, px = divmod(n, W)
        touched |= (xs == px).any(1) & (ys == py).any(1)
    assert 0 < int(touched.sum()) < H * W // 4
    try:
        _cabi.set_option("forward_lds", 1)
        good = hip_forward(hip_lib, *_dev(mo, q, k, v), H, W, r, 0.2)
        assert _cabi.last_forward_kernel().startswith("fwd_tile_f16" if dt == torch.float16 else "fwd_tile_bf16")
        bad = hip_forward(hip_lib, *_dev(mo, qb, kb, vb), H, W, r, 0.2)
        _cabi.set_option("forward_lds", 0)
        direct = hip_forward(hip_lib, *_dev(mo, qb, kb, vb), H, W, r, 0.2)
    finally:
        _cabi.set_option("forward_lds", -1)
    keep = ~touched.cuda()
    for a, b in zip(good, bad):
        assert torch.isfinite(b[0, keep]).all()
        # Head-queries that shared a matrix instruction with a poisoned one are recomputed by the generic kernel: the
        # same values to the operator's tolerance, not necessarily to the bit; all others are untouched.
        assert rel_err(b[0, keep].float().cpu(), a[0, keep].float().cpu()) <= TOL[dt]
        same = (a[0, keep] == b[0, keep]).flatten(1).all(1).float().mean().item()
        assert same >= 0.95, same
    # the queries that own a poisoned value get what the kernels without a matrix unit give them -- in every run: which
    # queries share a wavefront changes from call to call, and what an owner gets must not (one of them has an integer
    # y and its NaN in the window row such a lane drops)
    own = touched.cuda()
    for _ in range(6):
        for a, b in zip(bad, direct):
            assert torch.equal(torch.isfinite(a[0, own]), torch.isfinite(b[0, own]))
        try:
            _cabi.set_option("forward_lds", 1)
            bad = hip_forward(hip_lib, *_dev(mo, qb, kb, vb), H, W, r, 0.2)
        finally:
            _cabi.set_option("forward_lds", -1)


def test_bf16_backward_keeps_small_gradients(hip_lib):
    # upstream gradients of 1e-6 (a mean-reduced loss, no loss scaling): the logit gradient between the two passes of
    # the gather backward must keep bfloat16's exponent range -- as halves these values lose bits or vanish.
    B, H, W, h, Ch, r = 1, 20, 24, 2, 32, 2
    M = (2 * r + 2) ** 2
    dt = torch.bfloat16
    mo, q, k, v = make_case(B, H, W, h, Ch, r, dt, seed=5, offsets="interior")
    g = torch.Generator().manual_seed(3)
    d_out = (torch.randn(B, H * W, h * Ch, generator=g) * 1e-6).to(dt)
    d_attn = (torch.randn(B, H * W, h, M, generator=g) * 1e-6).to(dt)
    scale = Ch ** -0.5
    got = hip_backward(hip_lib, *_dev(mo, q, k, v), H, W, r, scale, d_out.cuda(), d_attn.cuda())
    check_grads(got, mo, q, k, v, H, W, r, scale, d_out, d_attn, "bwd small gradients")


def test_misaligned_tensors_take_the_generic_kernels(hip_lib):
    # views that start one element into an allocation are not 16-byte aligned: no vector kernel may touch them;
    # the results must agree with the aligned call
    from matchattention_amd import _cabi
    from tests.gpu_util import DT
    B, H, W, h, Ch, r = 1, 11, 13, 2, 32, 1
    N, C, M = H * W, h * Ch, 16
    mo, q, k, v = _dev(*make_case(B, H, W, h, Ch, r, torch.float16, seed=12))
    g = torch.Generator().manual_seed(2)
    d_out = torch.randn(B, N, C, generator=g).half().cuda()
    d_attn = torch.randn(B, N, h, M, generator=g).half().cuda()
    want_f = hip_forward(hip_lib, mo, q, k, v, H, W, r, 0.3)
    want_b = hip_backward(hip_lib, mo, q, k, v, H, W, r, 0.3, d_out, d_attn)

    def shifted(t):                                   # same values, storage offset of one element (2 bytes)
        buf = torch.empty(t.numel() + 8, dtype=t.dtype, device=t.device)
        view = buf[1:1 + t.numel()].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 != 0 and view.is_contiguous()
        return view

    q2, k2, v2, mo2, g2, da2 = (shifted(t) for t in (q, k, v, mo, d_out, d_attn))
    out, attn, dq, dk, dv = (shifted(torch.zeros_like(t)) for t in (q, want_f[1], q, q, q))
    dmo = shifted(torch.zeros_like(mo))
    s = torch.cuda.current_stream().cuda_stream
    dt = DT[torch.float16]
    _cabi.check(hip_lib.matchattn_forward(mo2.data_ptr(), q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), out.data_ptr(),
                                          attn.data_ptr(), B, H, W, C, h, r, r, 0.3, dt, s))
    assert _cabi.last_forward_kernel().startswith("fwd_generic")
    nb = hip_lib.matchattn_backward_workspace_bytes(B, H, W, C, h, r, r, dt)
    ws = torch.empty(max(nb, 16), dtype=torch.uint8, device="cuda")
    _cabi.check(hip_lib.matchattn_backward(mo2.data_ptr(), q2.data_ptr(), k2.data_ptr(), v2.data_ptr(), g2.data_ptr(), da2.data_ptr(),
                                           dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dmo.data_ptr(), ws.data_ptr(), nb,
                                           B, H, W, C, h, r, r, 0.3, dt, s))
    torch.cuda.synchronize()
    assert _cabi.last_backward_kernel().startswith("bwd_generic")
    for got, want in zip((out, attn, dq, dk, dv, dmo), want_f + want_b):
        assert rel_err(got.float().cpu(), want.float().cpu()) <= 2e-3

"""Inference script for stereo pairs on the MI355X operator: `python -m matchattention_amd.run_img`.

Flags, outputs and the timing protocol follow the reference's script (run_img.py:35-201): images from
--img0_dir / --img1_dir (png, jpg, bmp, paired in sorted order), padding to multiples of 32 or
--inference_size, `<name>_stereo.pfm` (+ `_noc.png`, `_r.pfm` with --save_right) under --output_path, and with
--test_inference_time five warm-up forwards, then five timed ones between two events on the stream,
reported per frame.  The network is the harness of matchattention_amd.stereo_harness: random-init from
--seed unless --checkpoint_path names a state dict saved from that harness (the reference's checkpoints use
other parameter names and do not load).  --mat_impl chooses the operator: 'hip' (the library; without it the
script fails, nothing is substituted) or 'pytorch' (matchattention_amd.mat_torch, the definition in plain torch ops,
as the reference's own 'pytorch' choice).  --low_res_init runs the pair at half size first and starts the
full-size run from that result (run_img.py:17-32); the model is compiled with torch.compile unless --no_compile
is given (run_img.py:55-58; the operator is an opaque custom op with a fake implementation, so it traces);
--save_rpos writes the self-attention's relative positions (run_img.py:161-165).
"""
import argparse
import os
from glob import glob

import numpy as np
import torch
import torch.nn.functional as F

from .file_io import InputPadder, write_pfm
from .stereo_harness import MatchLayer, MatchStereoHarness

# as the reference's script does (run_img.py:15): let the convolution library pick its kernels by measurement
# (on this ROCm image the frame time is the same either way: 22.2 ms at 1280x720, 32.5 ms at 1536x1536)
torch.backends.cudnn.benchmark = True

DTYPES = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(description="Stereo inference with the MatchAttention operator on MI355X")
    p.add_argument("--checkpoint_path", default=None, type=str, help="state dict of the harness (optional)")
    p.add_argument("--mode", choices=["stereo"], default="stereo")
    p.add_argument("--img0_dir", required=True, type=str, help="reference (left) view")
    p.add_argument("--img1_dir", required=True, type=str, help="target (right) view")
    p.add_argument("--output_path", default="outputs", type=str)
    p.add_argument("--device_id", default=0, type=int)
    p.add_argument("--scale", default=1.0, type=float, help="resize factor applied to the images first")
    p.add_argument("--inference_size", default=None, type=int, nargs=2, help="H W, divisible by 32")
    p.add_argument("--mat_impl", choices=["pytorch", "hip"], default="hip", help="MatchAttention implementation")
    p.add_argument("--precision", choices=list(DTYPES), default="fp32")
    p.add_argument("--variant", choices=["tiny", "small", "base"], default="tiny")
    p.add_argument("--no_fuse", action="store_true", help="run the elementwise steps around the operator as separate launches")
    p.add_argument("--test_inference_time", action="store_true")
    p.add_argument("--no_compile", action="store_true", help="run the model eagerly instead of through torch.compile")
    p.add_argument("--compile_backend", default="inductor", type=str, help="backend handed to torch.compile")
    p.add_argument("--save_right", action="store_true", help="also save the right view's disparity")
    p.add_argument("--save_rpos", action="store_true", help="also save the self-attention's relative positions")
    p.add_argument("--low_res_init", action="store_true",
                   help="run at half size first and start from that result; for images of 2K and beyond")
    p.add_argument("--seed", default=0, type=int, help="seed of the random-init weights")
    return p


def load_image(path: str) -> torch.Tensor:
    from PIL import Image
    return torch.from_numpy(np.array(Image.open(path).convert("RGB")).astype(np.float32)).permute(2, 0, 1)[None]


def list_pairs(dir0: str, dir1: str):
    def names(d):
        return sorted(sum((glob(os.path.join(d, e)) for e in ("*.png", "*.jpg", "*.bmp")), []))
    left, right = names(dir0), names(dir1)
    if len(left) != len(right):
        raise SystemExit(f"{len(left)} images in {dir0} but {len(right)} in {dir1}")
    return list(zip(left, right))


def consistency_mask(field: torch.Tensor, A: float = 8.0) -> torch.Tensor:
    """[2B,H,W,2] -> [2B,H,W] bool: the other view's field, sampled where this one points, cancels it to
    within A px (utils/utils.py:50-59)."""
    return MatchLayer.consistency(field, A)[..., 0] > 0


def run_frame(model, left, right, low_res_init: bool, factor: float = 2.0):
    """One pair through the model; with `low_res_init` the pair first runs at 1/factor size and its result, brought to
    1/32 of the full size, replaces the initial correlation of the full-size run (run_img.py:17-32).
    Returns (field [2,H,W,2], self_rpos [2,H/4,W/4,2])."""
    if not low_res_init:
        full, _, rpos = model(left, right, None, True)
        return full, rpos
    small = [F.interpolate(x, scale_factor=1 / factor, mode="bilinear", align_corners=True) for x in (left, right)]
    padder = InputPadder(small[0].shape, 32)
    small = padder.pad(*small)
    coarse, _, _ = model(small[0], small[1], None, True)
    coarse = padder.unpad(coarse.permute(0, 3, 1, 2).contiguous()).contiguous()
    init = F.interpolate(coarse, scale_factor=factor / 32, mode="bilinear", align_corners=True) * (factor / 32)
    full, _, rpos = model(left, right, init.permute(0, 2, 3, 1).contiguous(), True)
    return full, rpos


def make_model(args, device, dtype):
    """The harness with the operator --mat_impl names; compiled unless --no_compile."""
    if args.mat_impl == "hip":
        if not torch.cuda.is_available():
            raise SystemExit("no GPU: mat_impl='hip' needs one")
        from . import MF_FusedForwardOps, fused_module_forward
        op = MF_FusedForwardOps()

        def attend(mo, q, k, v, H, W, win_r, M, scale):
            return op(mo, q, k, v, H, W, win_r, M, "l1_norm", scale)
        fused = None if args.no_fuse else fused_module_forward
    else:
        from .mat_torch import attend_torch as attend
        fused = None
    model = MatchStereoHarness(attend, args.variant, seed=args.seed, fused=fused)
    if args.checkpoint_path:
        model.load_state_dict(torch.load(args.checkpoint_path, map_location="cpu", weights_only=True))
    model = model.to(device).to(dtype).eval()
    if not args.no_compile and device.type == "cuda":
        print("compiling the model, this may take several minutes")
        model = torch.compile(model, dynamic=False, backend=args.compile_backend)
    return model


def run(args) -> list:
    if args.inference_size is not None and any(s % 32 for s in args.inference_size):
        raise SystemExit("--inference_size must be divisible by 32")
    device = torch.device(f"cuda:{args.device_id}") if torch.cuda.is_available() and args.device_id >= 0 else torch.device("cpu")
    dtype = DTYPES[args.precision]
    model = make_model(args, device, dtype)
    timed = args.test_inference_time and device.type == "cuda"
    os.makedirs(args.output_path, exist_ok=True)
    pairs = list_pairs(args.img0_dir, args.img1_dir)
    print("%d test samples found" % len(pairs))
    written = []
    for name0, name1 in pairs:
        left, right = (load_image(n).to(device) for n in (name0, name1))
        if args.scale != 1.0:
            left, right = (F.interpolate(x, scale_factor=args.scale, mode="bilinear", align_corners=False) for x in (left, right))
        left, right = left.to(dtype), right.to(dtype)
        if args.inference_size is None:
            padder = InputPadder(left.shape, 32)
            left, right = padder.pad(left, right)
        else:
            ori = left.shape[-2:]
            left, right = (F.interpolate(x, size=tuple(args.inference_size), mode="bilinear", align_corners=True) for x in (left, right))
        print("Resolution: ", tuple(left.shape))
        with torch.inference_mode():
            if timed:
                for _ in range(5):
                    model(left, right, None, True)
                start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                start.record()
                for _ in range(5):
                    full, rpos = run_frame(model, left, right, args.low_res_init)
                end.record()
                end.synchronize()
                print(f"Inference Time (GPU) on {name0}: {start.elapsed_time(end) / 5:.6f} ms")
            else:
                full, rpos = run_frame(model, left, right, args.low_res_init)
            field = full.permute(0, 3, 1, 2).float().contiguous()                    # [2,2,H,W]
            rpos = F.interpolate(rpos.permute(0, 3, 1, 2).float().contiguous(), scale_factor=4, mode="bilinear",
                                 align_corners=True) * 4
            if args.inference_size is None:
                field, rpos = padder.unpad(field), padder.unpad(rpos)
            else:
                field, rpos = (F.interpolate(t, size=tuple(ori), mode="bilinear", align_corners=True) for t in (field, rpos))
                for t in (field, rpos):
                    t[:, 0] *= ori[1] / float(args.inference_size[1])
                    t[:, 1] *= ori[0] / float(args.inference_size[0])
            noc = consistency_mask(field.permute(0, 2, 3, 1).contiguous())
        stem = os.path.join(args.output_path, os.path.basename(name0)[:-4] + f"_{args.mode}")
        from PIL import Image
        Image.fromarray(np.where(noc[0].cpu().numpy(), 255, 128).astype(np.uint8)).save(stem + "_noc.png")
        disp_l = (-field[0, 0]).clamp(min=0).cpu().numpy()                           # left view: negative x-flow
        disp_r = field[1, 0].clamp(min=0).cpu().numpy()
        write_pfm(stem + ".pfm", disp_l)
        written.append(stem + ".pfm")
        if args.save_right:
            write_pfm(stem + "_r.pfm", disp_r)
            written.append(stem + "_r.pfm")
        if args.save_rpos:
            for axis, tag in ((0, "x"), (1, "y")):
                write_pfm(stem + f"_self_rpos_{tag}.pfm", rpos[0, axis].cpu().numpy())
                written.append(stem + f"_self_rpos_{tag}.pfm")
    print("Inference done.")
    return written


def main(argv=None):
    run(build_parser().parse_args(argv))


if __name__ == "__main__":
    main()

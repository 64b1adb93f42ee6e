#!/usr/bin/env python3
"""Benchmark of the MI355X MatchAttention operator (mat_impl='hip').

One "step" is one forward pass of the operator over one synthetic batch of the
high-resolution stereo shape (fp16, B=1, 544x960 query map = 1/4 of 2176x3840,
C=256 in 8 heads, 5x5 window i.e. r=2, cross-attention, x-offset ~ U(-240, 0), y = 0),
inputs resident in HBM.  Prints ONE JSON line:

  metric/value   MatchAttention queries/s (one query = one pixel with all its heads)
  roofline       algorithmic bytes of the forward / the mean duration of its dominant kernel (HIP
                 events either side of that launch, on the launch stream), against 8 TB/s HBM peak;
                 whole_call_*: the same over the whole call (bucketing kernels included)
  cpu_baseline   the CPU restatement of the reference's PyTorch path (oracle/), timed on the host
                 cores: the fp32 104x208 shape the baseline plan names (the bench's own workload,
                 on a bounded sample of its rows, is extra.cpu_baseline_bench_workload)
  extra          the other operator workloads (forward and backward), for the record

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E bandwidth
# HBM bytes per forward launch of the headline workload from rocprofv3 FETCH_SIZE + WRITE_SIZE
# (see profiles/): filled in from the committed counter summary, None when not measured.
# keyed by (workload, first part of the kernel name that ran)
MEASURED_TRAFFIC_BYTES = {
    ("cfg3_cross", "fwd_tile_f16"): 1803636736,    # LDS-tile kernel: 2.0 x 572323 KiB fetched + 616718 KiB written
    ("cfg3_cross", "fwd_tiled_f16"): 1470390272,   # direct-gather kernel: 2.0 x 424204 KiB fetched + 587520 KiB written
    ("cfg3_cross", "fwd_tile_f32"): 3778794496,    # fp32 LDS-tile kernel: 2.0 x 1233603 KiB fetched + 1223023 KiB written
}


# HBM bytes per backward call, per kernel, from the same two counters (profiles/bwd_gather_cfg4_cfg2.md)
MEASURED_BWD_TRAFFIC_BYTES = {
    ("cfg4_cross", "bwd_tile_f16"): {
        "bwd_h16_tile_kernel": (2 * 737252 + 606083) * 1024,      # pass A: 2.0 x FETCH_SIZE + WRITE_SIZE (KiB)
        "bwd_key_kernel": (2 * 545658 + 294912) * 1024,           # pass B
    },
}


# Kernel names (as rocprofv3 prints them) of the dominant forward kernels, by the library's own name for the path
_TRAFFIC_KERNELS = {"fwd_tile_f16": "fwd_h16_tile_kernel", "fwd_tile_bf16": "fwd_h16_tile_kernel", "fwd_tile_f32": "fwd_tile_kernel",
                    "fwd_tiled_": "fwd_h16_kernel"}


def _measure_traffic(argv_tail, kernel_hint, timeout_s=150):
    """HBM-side bytes per launch of the dominant forward kernel, measured now: two child runs of this script under
    `rocprofv3 --pmc` (FETCH_SIZE, then WRITE_SIZE: KiB per dispatch), each reading scaled by what the same counter
    reads for a device copy of known size in the same run (`--calibrate-copy`: 64 MiB per dispatch).  Returns a dict,
    or None when anything fails (no rocprofv3, counters refused, time-out): the caller then reports the recorded figure.
    Runs before this process touches the GPU."""
    import csv, glob, shutil, signal, subprocess, tempfile
    rocprof = shutil.which("rocprofv3") or "/opt/rocm/bin/rocprofv3"
    if not os.path.exists(rocprof):
        return None
    here = os.path.abspath(__file__)
    got = {}
    tmp = tempfile.mkdtemp(prefix="ma_traffic_", dir="/tmp")
    try:
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            out = os.path.join(tmp, counter)
            cmd = [rocprof, "--pmc", counter, "--kernel-trace", "-d", out, "--output-format", "csv", "--",
                   sys.executable, here, "--no-cpu", "--no-extra", "--no-traffic", "--steps", "5", "--warmup", "2",
                   "--calibrate-copy"] + argv_tail
            env = dict(os.environ, TMPDIR="/tmp")
            proc = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                                    start_new_session=True)
            try:
                if proc.wait(timeout=timeout_s) != 0:
                    return None
            except subprocess.TimeoutExpired:
                os.killpg(proc.pid, signal.SIGKILL)
                proc.wait()
                return None
            files = glob.glob(os.path.join(out, "**", "*counter_collection.csv"), recursive=True)
            if not files:
                return None
            vals = {"kernel": [], "copy": []}
            for row in csv.DictReader(open(files[0])):
                if row.get("Counter_Name") != counter:
                    continue
                name = row.get("Kernel_Name", "")
                if kernel_hint in name:
                    vals["kernel"].append(float(row["Counter_Value"]))
                elif "copyBuffer" in name:
                    vals["copy"].append(float(row["Counter_Value"]))
            if not vals["kernel"] or not vals["copy"]:
                return None
            got[counter] = (sum(vals["kernel"]) / len(vals["kernel"]), sum(vals["copy"]) / len(vals["copy"]), len(vals["kernel"]))
    except Exception:
        return None
    finally:
        shutil.rmtree(tmp, ignore_errors=True)
    copy_kib = 65536.0                                  # one copy dispatch: 64 MiB read, 64 MiB written
    f_fetch, f_write = copy_kib / got["FETCH_SIZE"][1], copy_kib / got["WRITE_SIZE"][1]
    if not (0.5 < f_fetch < 8 and 0.5 < f_write < 8):
        return None
    nbytes = (got["FETCH_SIZE"][0] * f_fetch + got["WRITE_SIZE"][0] * f_write) * 1024.0
    return {"bytes": int(round(nbytes)), "fetch_kib": got["FETCH_SIZE"][0], "write_kib": got["WRITE_SIZE"][0],
            "fetch_factor": f_fetch, "write_factor": f_write, "dispatches": got["FETCH_SIZE"][2]}


def _events_ms(fn, steps, warmup):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    per = [a.elapsed_time(b) for a, b in evs]
    return wall, sum(per) / len(per), min(per)


def _cold_ms(fn, reps=10):
    """Mean event time of `fn` when a 1 GiB fill (four times the 256 MB memory-side cache) runs before
    every call, so that no input is left in L2 or the memory-side cache by the previous call."""
    import torch
    junk = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    for _ in range(2):          # (the first call of a process loads the kernels' code: not what is measured here)
        fn()
    torch.cuda.synchronize()
    per = []
    for i in range(reps):
        junk.fill_(i & 0xff)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        per.append(a.elapsed_time(b))
    del junk
    return sum(per) / len(per)


def _forward_call(lib, wl, inp):
    import torch
    from matchattention_amd import _cabi
    from matchattention_amd.match_former_ops import _DTYPES
    B, N, C = inp["q"].shape
    out = torch.empty_like(inp["q"])
    attn = torch.empty(B, N, wl.h, wl.M, dtype=wl.dtype, device=inp["q"].device)
    stream = torch.cuda.current_stream().cuda_stream
    ptr = [inp[k].data_ptr() for k in ("max_offset", "q", "k", "v")] + [out.data_ptr(), attn.data_ptr()]
    dt = _DTYPES[wl.dtype]
    # scratch the library may use to order the queries by sampling target (allocated once, outside the timed region)
    nbytes = lib.matchattn_forward_workspace_bytes(B, inp["H"], inp["W"], C, wl.h, wl.r, wl.r, dt)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=inp["q"].device)

    def call():
        _cabi.check(lib.matchattn_forward_ws(*ptr, ws.data_ptr() if nbytes else None, nbytes, B, inp["H"], inp["W"], C,
                                             wl.h, wl.r, wl.r, wl.scale, dt, stream))
    return call, (out, attn, ws)


def _backward_call(lib, wl, inp):
    import torch
    from matchattention_amd import _cabi
    from matchattention_amd.match_former_ops import _DTYPES
    B, N, C = inp["q"].shape
    dt = _DTYPES[wl.dtype]
    dq, dk, dv = (torch.empty_like(inp["q"]) for _ in range(3))
    dmo = torch.empty_like(inp["max_offset"])
    nbytes = lib.matchattn_backward_workspace_bytes(B, inp["H"], inp["W"], C, wl.h, wl.r, wl.r, dt)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=inp["q"].device)
    stream = torch.cuda.current_stream().cuda_stream
    d_attn = inp["d_attn"]

    def call():
        _cabi.check(lib.matchattn_backward(
            inp["max_offset"].data_ptr(), inp["q"].data_ptr(), inp["k"].data_ptr(), inp["v"].data_ptr(),
            inp["d_out"].data_ptr(), None if d_attn is None else d_attn.data_ptr(),
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dmo.data_ptr(), ws.data_ptr() if nbytes else None, nbytes,
            B, inp["H"], inp["W"], C, wl.h, wl.r, wl.r, wl.scale, dt, stream))
    return call, (dq, dk, dv, dmo, ws)


def _cpu_threads():
    """Threads the CPU legs use: torch's own default, which follows OMP_NUM_THREADS where the machine sets it to this
    job's share of the host (and is the host's core count otherwise)."""
    import torch
    return torch.get_num_threads()


def _cpu_baseline_cfg1():
    """The CPU configuration the baseline plan names: the oracle (a port of the reference's PyTorch path) on the whole
    cfg1 map in fp32 (1 x 104 x 208, C=128 in 4 heads, r=1, x ~ U(-40, 0), y = 0), 2 warm-ups, median of 5 runs."""
    import torch
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    from oracle import mat_oracle as O
    wl = WORKLOADS["cfg1_cross"]
    inp = make_inputs(wl, device="cpu")
    times = []
    for i in range(7):
        t0 = time.perf_counter()
        O.forward(inp["max_offset"], inp["q"], inp["k"], inp["v"], inp["H"], inp["W"], [wl.r, wl.r], wl.scale)
        times.append(time.perf_counter() - t0)
    t = sorted(times[2:])[2]
    return {"value": wl.B * wl.N / t, "unit": "queries/s", "cores": _cpu_threads(), "kind": "port",
            "host_cpus": os.cpu_count(), "ms": round(t * 1e3, 2),
            "sample": f"cfg1_cross, the whole {wl.H}x{wl.W} map, float32, C={wl.C} in {wl.h} heads, r={wl.r}: "
                      f"oracle/mat_oracle.py forward, 2 warm-ups then the median of 5 runs ({sum(times):.1f} s of CPU work in all)"}


def _cpu_baseline(wl, seconds_target=12.0):
    """The oracle on the host cores on the first rows of the bench's own workload, sized to roughly
    `seconds_target` seconds."""
    import torch
    from matchattention_amd.workloads import make_inputs
    from oracle import mat_oracle as O
    cores = _cpu_threads()

    def run(rows):
        inp = make_inputs(wl, device="cpu", rows=rows)
        t0 = time.perf_counter()
        O.forward_chunked(inp["max_offset"], inp["q"], inp["k"], inp["v"], inp["H"], inp["W"], [wl.r, wl.r],
                          wl.scale, rows_per_chunk=4)
        return time.perf_counter() - t0

    run(8)                                   # warm-up (thread pool, allocator)
    probe_rows = 16
    t = run(probe_rows)
    rows = int(max(probe_rows, min(wl.H, probe_rows * seconds_target / max(t, 1e-3))))
    rows -= rows % 4
    t = run(rows)
    q = wl.B * rows * wl.W
    return {"value": q / t, "unit": "queries/s", "cores": cores, "kind": "port", "host_cpus": os.cpu_count(),
            "sample": f"first {rows} of {wl.H} query rows of the same workload as its own {rows}x{wl.W} map, "
                      f"{str(wl.dtype).split('.')[-1]}, oracle/mat_oracle.py forward_chunked, {t:.1f} s"}


def _e2e_ms_per_frame(only_size=None):
    """MatchStereo-T harness (random-init weights), fp16, mat_impl='hip': ms/frame with the
    reference's protocol -- 5 warm-up forwards, then 5 timed ones between events
    (reference run_img.py:101-112) -- at 1280x720 (padded to 1280x736) and 1536x1536."""
    import torch
    from matchattention_amd import MF_FusedForwardOps, fused_module_forward
    from matchattention_amd.stereo_harness import MatchStereoHarness
    from matchattention_amd.workloads import make_stereo_pair
    op = MF_FusedForwardOps()

    def attend(mo, q, k, v, H, W, win_r, M, scale):
        return op(mo, q, k, v, H, W, win_r, M, "l1_norm", scale)

    out = {}
    # "fused": the coordinate add, clamp, gate and concatenation either side of the operator run inside it
    variants = (("", None), ("_fused", fused_module_forward)) if only_size is None else (("_fused", fused_module_forward),)
    sizes = ((720, 1280), (1536, 1536)) if only_size is None else (only_size,)
    for tag, fused in variants:
        model = MatchStereoHarness(attend, "tiny", seed=0, fused=fused).cuda().half().eval()
        for (H, W) in sizes:
            left, right, _ = make_stereo_pair(H, W, dtype=torch.float16)
            with torch.inference_mode():
                for _ in range(5):
                    model(left, right)
                torch.cuda.synchronize()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for _ in range(5):
                    model(left, right)
                b.record()
                torch.cuda.synchronize()
            out[f"{W}x{H}_ms_per_frame{tag}"] = round(a.elapsed_time(b) / 5, 3)
    if only_size is None:
        # the one published latency of the reference (README.md:52,56: MatchStereo-T at 1536x1536, fp16, torch.compile,
        # one RTX 5090, trained weights) beside this harness's figure: other hardware and random weights, same protocol
        out["1536x1536_ms_per_frame_published_rtx5090"] = 38.0
    return out


def _e2e_pytorch_baseline():
    """The baseline legs of the end-to-end plan: the same harness with the operator in plain PyTorch ops
    (`mat_impl='pytorch'`, matchattention_amd.mat_torch) at 1280x720 -- on the GPU in fp16 with the 5 + 5 protocol, and
    on the host cores in fp32, one frame."""
    import torch
    from matchattention_amd.mat_torch import attend_torch
    from matchattention_amd.stereo_harness import MatchStereoHarness
    from matchattention_amd.workloads import make_stereo_pair
    out = {}
    model = MatchStereoHarness(attend_torch, "tiny", seed=0).cuda().half().eval()
    left, right, _ = make_stereo_pair(720, 1280, dtype=torch.float16)
    with torch.inference_mode():
        for _ in range(5):
            model(left, right)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(5):
            model(left, right)
        b.record()
        torch.cuda.synchronize()
    out["1280x720_ms_per_frame_pytorch_operator_gpu_fp16"] = round(a.elapsed_time(b) / 5, 3)
    del model
    torch.cuda.empty_cache()
    model = MatchStereoHarness(attend_torch, "tiny", seed=0).eval()
    left, right, _ = make_stereo_pair(720, 1280, device="cpu", dtype=torch.float32)
    with torch.inference_mode():
        t0 = time.perf_counter()
        model(left, right)
        out["1280x720_ms_per_frame_pytorch_operator_cpu_fp32"] = round((time.perf_counter() - t0) * 1e3, 1)
    out["cpu_threads"] = _cpu_threads()
    return out


def _module_step_ms(wl, inp, steps=20):
    """The cross-attention module's sequence around the operator at this workload's size -- pixel grid add,
    clamp, operator, gate, concatenation (reference models/attention_blocks.py:162-163, 45-59, 96-98) -- as
    separate launches and as the one fused native call."""
    import torch
    from matchattention_amd import MF_FusedForwardOps, fused_module_forward
    from matchattention_amd.stereo_harness import pixel_grid
    op = MF_FusedForwardOps()
    B, H, W, h, r = wl.B, inp["H"], inp["W"], wl.h, wl.r
    N, M = H * W, (2 * r + 2) ** 2
    q, k, v = inp["q"], inp["k"], inp["v"]
    grid = pixel_grid(B, H, W, q.dtype, q.device).reshape(B, N, 1, 2)
    shared = bool((inp["max_offset"][:, :, :1] == inp["max_offset"]).all())
    rel = ((inp["max_offset"][:, :, :1] if shared else inp["max_offset"]) - grid).contiguous()
    gate = torch.sigmoid(inp["d_out"].float()).to(q.dtype)
    hi_x = float(torch.tensor(W - 1 - r - 1e-3, dtype=q.dtype)); hi_y = float(torch.tensor(H - 1 - r - 1e-3, dtype=q.dtype))

    def separate():
        mo = (rel + grid).expand(B, N, h, 2)
        mo = torch.cat((torch.clamp(mo[..., 0:1], min=float(r), max=hi_x), torch.clamp(mo[..., 1:2], min=float(r), max=hi_y)), -1).contiguous()
        out, attn = op(mo, q, k, v, H, W, [r, r], M, "l1_norm", wl.scale)
        return torch.cat((gate * out, attn.reshape(B, N, -1)), -1)

    def fused():
        return fused_module_forward(rel, q, k, v, H, W, [r, r], h, wl.scale, gate=gate, concat=True)

    res = {}
    with torch.inference_mode():
        same = torch.equal(separate(), fused())
        for name, fn in (("separate_ms", separate), ("fused_ms", fused)):
            for _ in range(3):
                fn()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            a.record()
            for _ in range(steps):
                fn()
            b.record()
            torch.cuda.synchronize()
            res[name] = round(a.elapsed_time(b) / steps, 4)
    res["bit_identical"] = same
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="cfg3_cross")
    ap.add_argument("--direct", action="store_true",
                    help="time the direct-gather forward kernel instead of the LDS-tile path (forward_lds=0)")
    ap.add_argument("--backward", action="store_true",
                    help="time the backward of --workload instead (prints its own line; for profiling)")
    ap.add_argument("--dtype", choices=["f16", "f32", "bf16"], default=None,
                    help="run the workload in this storage type instead of its own (extras and CPU leg keep theirs)")
    ap.add_argument("--e2e", nargs="?", const="all", default=None, metavar="HxW",
                    help="run only the end-to-end MatchStereo-T harness leg and print its ms/frame (prints its own "
                         "line; for profiling); with HxW, e.g. 720x1280, only that size with the fused module step")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--no-traffic", action="store_true",
                    help="do not measure roofline.traffic in this run (two child runs under rocprofv3 --pmc, about a "
                         "minute); the figure recorded in profiles/ is reported instead")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known HBM traffic, "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this operator benchmark runs on exactly one GPU (--gpus 1); "
              "sharding across GPUs is a design note, not part of this build", file=sys.stderr)
        sys.exit(2)

    # roofline.traffic of the headline line is measured by this run itself, before this process touches the GPU
    traffic_now = None
    if not (args.no_traffic or args.backward or args.e2e):
        from matchattention_amd.workloads import WORKLOADS as _W0, MODEL_SHAPES as _W1, MODEL_SHAPES_BASE_F32 as _W2
        _W = {**_W0, **_W1, **_W2}
        dt_name = args.dtype or {"float16": "f16", "float32": "f32", "bfloat16": "bf16"}[str(_W[args.workload].dtype).split(".")[-1]]
        hint = "fwd_h16_kernel" if (args.direct and dt_name == "f16") else ("fwd_tiled_kernel" if args.direct else _TRAFFIC_KERNELS["fwd_tile_" + dt_name])
        tail = ["--workload", args.workload] + (["--dtype", args.dtype] if args.dtype else []) + (["--direct"] if args.direct else [])
        traffic_now = _measure_traffic(tail, hint)

    import torch
    from matchattention_amd import _cabi
    from matchattention_amd.workloads import WORKLOADS, make_inputs
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = _cabi.load()
    torch.cuda.set_device(0)

    if args.e2e:
        size = None if args.e2e == "all" else tuple(int(t) for t in args.e2e.lower().split("x"))
        print(json.dumps({"e2e_matchstereo_tiny": _e2e_ms_per_frame(size)}))
        return

    if args.calibrate_copy:
        src = torch.ones(1 << 26, dtype=torch.float32, device="cuda")    # 256 MiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # (--workload also takes the names of workloads.MODEL_SHAPES, the model's own operator shapes, on their smooth fields)
    from matchattention_amd.workloads import MODEL_SHAPES, MODEL_SHAPES_BASE_F32
    _models = {**MODEL_SHAPES, **MODEL_SHAPES_BASE_F32}
    wl = WORKLOADS[args.workload] if args.workload in WORKLOADS else _models[args.workload]
    inp = make_inputs(wl, smooth=args.workload in _models)
    if args.dtype:      # the same workload (same offset field and values, rounded) in another storage type
        import dataclasses
        dt = {"f16": torch.float16, "f32": torch.float32, "bf16": torch.bfloat16}[args.dtype]
        for key in ("max_offset", "q", "k", "v", "d_out", "d_attn"):
            if inp[key] is not None:
                inp[key] = inp[key].to(dt)
        wl = dataclasses.replace(wl, dtype=dt)
    if args.backward:
        call, keep = _backward_call(lib, wl, inp)
        wall_ms, ev_ms, ev_min = _events_ms(call, args.steps, args.warmup)
        nbytes = wl.backward_bytes(inp["d_attn"] is not None)
        print(json.dumps({"metric": "matchattention_backward_queries_per_sec", "value": wl.B * wl.N / (wall_ms * 1e-3),
                          "unit": "queries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": wall_ms,
                          "higher_is_better": True, "dtype": str(wl.dtype).split(".")[-1], "data": "synthetic",
                          "config": {"workload": wl.name, "kernel": _cabi.last_backward_kernel()},
                          "algorithmic_GBps": nbytes / (ev_ms * 1e-3) / 1e9, "call_ms_mean": ev_ms, "call_ms_min": ev_min,
                          "algorithmic_bytes_per_call": nbytes,
                          "traffic": MEASURED_BWD_TRAFFIC_BYTES.get((args.workload, _cabi.last_backward_kernel()))}))
        return
    if args.direct:
        _cabi.set_option("forward_lds", 0)
    call, keep = _forward_call(lib, wl, inp)
    # The side measurements come first, the timed region last.  The first 25-30 ms of GPU work after start-up run at a
    # lower clock (a kernel trace shows every kernel of a call, whatever it touches, 10-25 % slower over the first ~35
    # calls and settling afterwards): with these ~45 calls in front, the W warm-up and K timed steps below see the GPU
    # as a long-running caller does.
    cold_ms = _cold_ms(call)
    # the dominant kernel alone (the library's own events either side of its launch), outside the timed region
    _cabi.set_option("time_kernels", 1)
    dom = []
    for _ in range(35):
        call()
        dom.append(float(lib.matchattn_last_forward_kernel_ms()))
    _cabi.set_option("time_kernels", 0)
    dom_ms = sum(dom[15:]) / len(dom[15:]) if min(dom) > 0 else None
    wall_ms, ev_ms, ev_min = _events_ms(call, args.steps, args.warmup)
    kernel = _cabi.last_forward_kernel()
    queries = wl.B * wl.N
    alg_bytes = wl.forward_bytes()
    # the roofline figure is the dominant kernel's: algorithmic bytes of the launch over its own mean duration
    # (the library's events either side of that one launch); the whole call -- bucketing kernels before it, the flag
    # scan after it -- is what `value` and `whole_call_*` report
    whole_call = alg_bytes / (ev_ms * 1e-3) / 1e9
    achieved = whole_call if dom_ms is None else alg_bytes / (dom_ms * 1e-3) / 1e9
    traffic = next((v for (w, k), v in MEASURED_TRAFFIC_BYTES.items()
                    if w == args.workload and kernel.startswith(k + "_")), None)
    traffic_source = "recorded: profiles/ (rocprofv3 --pmc FETCH_SIZE x 2.0 + WRITE_SIZE of an earlier run)" if traffic else None
    if traffic_now is not None:
        traffic = traffic_now["bytes"]
        traffic_source = ("measured in this run: rocprofv3 --pmc, FETCH_SIZE %.0f KiB x %.3f + WRITE_SIZE %.0f KiB x %.3f per launch "
                          "(factors from a 64 MiB device copy in the same runs; mean of %d launches)"
                          % (traffic_now["fetch_kib"], traffic_now["fetch_factor"], traffic_now["write_kib"],
                             traffic_now["write_factor"], traffic_now["dispatches"]))

    extra = {}
    if not args.no_extra:
        del keep
        for name, w2 in WORKLOADS.items():
            i2 = make_inputs(w2)
            rec = {}
            c2, k2 = _forward_call(lib, w2, i2)
            _, ms, _ = _events_ms(c2, max(5, args.steps // 5), 3)
            rec["fwd_ms"] = round(ms, 4)
            rec["fwd_queries_per_s"] = w2.B * w2.N / (ms * 1e-3)
            rec["fwd_GBps"] = round(w2.forward_bytes() / (ms * 1e-3) / 1e9, 1)
            rec["fwd_kernel"] = _cabi.last_forward_kernel()
            del k2
            if w2.backward:
                c3, k3 = _backward_call(lib, w2, i2)
                _, ms, _ = _events_ms(c3, max(5, args.steps // 5), 3)
                rec["bwd_ms"] = round(ms, 4)
                rec["bwd_GBps"] = round(w2.backward_bytes(i2["d_attn"] is not None) / (ms * 1e-3) / 1e9, 1)
                rec["bwd_kernel"] = _cabi.last_backward_kernel()
                tr = MEASURED_BWD_TRAFFIC_BYTES.get((name, rec["bwd_kernel"]))
                if tr:      # HBM-side bytes per kernel of the call (counters, profiles/bwd_gather_cfg4_cfg2.md)
                    rec["bwd_traffic"] = dict(tr, algorithmic_bytes=w2.backward_bytes(i2["d_attn"] is not None))
                del k3
            if name in ("cfg3_cross", "cfg2_cross"):
                rec["module_step"] = _module_step_ms(w2, i2)
            if rec["fwd_kernel"].startswith("fwd_tile_"):
                # the same forward through the direct-gather kernel (no bucketing, taps fetched from L2)
                _cabi.set_option("forward_lds", 0)
                try:
                    c4, k4 = _forward_call(lib, w2, i2)
                    _, ms, _ = _events_ms(c4, max(5, args.steps // 5), 3)
                    rec["fwd_direct_ms"] = round(ms, 4)
                    rec["fwd_direct_kernel"] = _cabi.last_forward_kernel()
                    del k4
                finally:
                    _cabi.set_option("forward_lds", -1)
            extra[name] = rec
            del i2
            torch.cuda.empty_cache()

    if not args.no_extra:
        # the same headline workload with other offset fields: the i.i.d. one blurred to sigma = 8 px at the same amplitude
        # (correlated, but the offsets still change by several pixels per pixel), and a field as a stereo scene gives it
        # (slanted surfaces and discontinuities: the offsets of neighbours differ by a fraction of a pixel)
        for field_tag, kind in (("_smooth_field", True), ("_scene_field", "scene")):
            if kind == "scene" and not wl.offsets.startswith("stereo"):
                continue
            i3 = make_inputs(wl, smooth=kind)
            rec = {}
            for tag, lds in (("fwd_ms", -1), ("fwd_direct_ms", 0)):
                _cabi.set_option("forward_lds", lds)
                try:
                    c5, k5 = _forward_call(lib, wl, i3)
                    _, ms, _ = _events_ms(c5, max(5, args.steps // 5), 3)
                    rec[tag] = round(ms, 4)
                    del k5
                finally:
                    _cabi.set_option("forward_lds", -1)
            extra[args.workload + field_tag] = rec
            del i3
        # the largest maps in the other storage types (fp32 is the reference script's default precision)
        import dataclasses
        for name in ("cfg3_cross", "cfg3_self"):
            for dt, tag in ((torch.float32, "f32"), (torch.bfloat16, "bf16")):
                w4 = dataclasses.replace(WORKLOADS[name], dtype=dt)
                i4 = make_inputs(WORKLOADS[name])
                for key in ("max_offset", "q", "k", "v"):
                    i4[key] = i4[key].to(dt)
                rec = {}
                for col, lds in (("fwd_ms", -1), ("fwd_direct_ms", 0)):
                    _cabi.set_option("forward_lds", lds)
                    try:
                        c6, k6 = _forward_call(lib, w4, i4)
                        _, ms, _ = _events_ms(c6, max(5, args.steps // 5), 3)
                        rec[col] = round(ms, 4)
                        if lds == -1:
                            rec["fwd_GBps"] = round(w4.forward_bytes() / (ms * 1e-3) / 1e9, 1)
                            rec["fwd_kernel"] = _cabi.last_forward_kernel()
                        del k6
                    finally:
                        _cabi.set_option("forward_lds", -1)
                extra[f"{name}_{tag}"] = rec
                del i4
                torch.cuda.empty_cache()
        for dt, tag in ((torch.float32, "f32"), (torch.bfloat16, "bf16")):
            w5 = dataclasses.replace(WORKLOADS["cfg4_cross"], dtype=dt)
            i5 = make_inputs(WORKLOADS["cfg4_cross"])
            for key in ("max_offset", "q", "k", "v", "d_out", "d_attn"):
                i5[key] = i5[key].to(dt)
            rec = {}
            for col, mode in (("bwd_ms", -1), ("bwd_direct_pass_a_ms", 2)):
                _cabi.set_option("backward_mode", mode)
                try:
                    c7, k7 = _backward_call(lib, w5, i5)
                    _, ms, _ = _events_ms(c7, max(5, args.steps // 5), 3)
                    rec[col] = round(ms, 4)
                    if mode == -1:
                        rec["bwd_GBps"] = round(w5.backward_bytes(True) / (ms * 1e-3) / 1e9, 1)
                        rec["bwd_kernel"] = _cabi.last_backward_kernel()
                    del k7
                finally:
                    _cabi.set_option("backward_mode", -1)
            extra[f"cfg4_cross_{tag}"] = rec
            del i5
            torch.cuda.empty_cache()
        # the operator at the shapes a MatchStereo-T frame calls it with (1536 x 1536 input: maps of 48^2 .. 384^2, B = 2),
        # forward and backward, on smooth fields: mostly one launch of a few microseconds, bound by launch latency
        # (and at the `base` variant's in fp32, the script's default precision: heads of up to 128 fp32 channels)
        from matchattention_amd.workloads import MODEL_SHAPES, MODEL_SHAPES_BASE_F32
        shapes = {}
        for name, w6 in list(MODEL_SHAPES.items()) + list(MODEL_SHAPES_BASE_F32.items()):
            i6 = make_inputs(w6, smooth=True)
            rec = {}
            c8, k8 = _forward_call(lib, w6, i6)
            _, ms, _ = _events_ms(c8, 30, 10)
            rec["fwd_ms"] = round(ms, 4)
            rec["fwd_GBps"] = round(w6.forward_bytes() / (ms * 1e-3) / 1e9, 1)
            rec["fwd_frac"] = round(w6.forward_bytes() / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            rec["fwd_kernel"] = _cabi.last_forward_kernel()
            c9, k9 = _backward_call(lib, w6, i6)
            _, ms, _ = _events_ms(c9, 30, 10)
            rec["bwd_ms"] = round(ms, 4)
            rec["bwd_GBps"] = round(w6.backward_bytes(i6["d_attn"] is not None) / (ms * 1e-3) / 1e9, 1)
            rec["bwd_frac"] = round(w6.backward_bytes(i6["d_attn"] is not None) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
            rec["bwd_kernel"] = _cabi.last_backward_kernel()
            shapes[name] = rec
            del k8, k9, i6
        extra["model_shapes_matchstereo_tiny_1536"] = {k_: v_ for k_, v_ in shapes.items() if k_ in MODEL_SHAPES}
        extra["model_shapes_matchstereo_base_fp32_1536"] = {k_: v_ for k_, v_ in shapes.items() if k_ in MODEL_SHAPES_BASE_F32}
        torch.cuda.empty_cache()
        # a plain device-to-device copy on this box, read + write bytes per second (what the HBM path delivers
        # to the simplest possible kernel)
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()       # 1 GiB
        dst = torch.empty_like(src)
        _, ms, _ = _events_ms(lambda: dst.copy_(src), 10, 3)
        extra["device_copy_GBps"] = round(2 * src.numel() * 4 / (ms * 1e-3) / 1e9, 1)
        del src, dst
        torch.cuda.empty_cache()
        extra["e2e_matchstereo_tiny"] = _e2e_ms_per_frame()
        if not args.no_cpu:
            extra["e2e_matchstereo_tiny"].update(_e2e_pytorch_baseline())

    cpu = None
    if not args.no_cpu:
        cpu = _cpu_baseline_cfg1()
        extra["cpu_baseline_bench_workload"] = _cpu_baseline(wl)

    line = {
        "metric": "matchattention_queries_per_sec",
        "value": queries / (wall_ms * 1e-3),
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if wl.dtype == torch.float16 else ("bf16" if wl.dtype == torch.bfloat16 else "f32"),
        "data": "synthetic",
        "config": {
            "workload": f"{wl.name}: MatchAttention forward, {str(wl.dtype).split('.')[-1]}, B={wl.B}, "
                        f"{wl.H}x{wl.W} query map, C={wl.C} in {wl.h} heads, r={wl.r} (M={wl.M}), offsets {wl.offsets} "
                        f"i.i.d. per pixel ({'per head' if wl.per_head else 'shared by heads'}), replicate-clamped taps",
            "kernel": kernel,
            "queries_per_step": queries,
            "head_queries_per_sec": queries * wl.h / (wall_ms * 1e-3),
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": traffic,
            "traffic_source": traffic_source,
            "algorithmic_bytes_per_launch": alg_bytes,
            "dominant_kernel": kernel,
            "dominant_kernel_ms": dom_ms,
            "whole_call_ms_mean": ev_ms,
            "whole_call_ms_min": ev_min,
            "whole_call_ms_cold_caches": cold_ms,
            "whole_call_GBps": whole_call,
            "whole_call_frac": whole_call / HBM_PEAK_GBS,
        },
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

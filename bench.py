"""Benchmark of the PTv3 forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

A step is one full PointTransformerV3 forward (default architecture, fp16, eval) over a batch
of 4 synthetic room scenes of ~100k voxelised points each, inputs resident in HBM. Prints one
JSON line: throughput in points/s, the roofline of the dominant kernel (patch attention,
MFMA-bound) measured with HIP events around every launch inside the timed region, and the
CPU oracle timed on this machine's host cores on one of the four scenes.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16/bf16


class LaunchTimer:
    """HIP events around selected kernel launches, on the stream they are launched on."""

    def __init__(self):
        self.records = {}

    def launch(self, name, work, fn):
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        out = fn()
        e.record()
        self.records.setdefault(name, []).append((s, e, work))
        return out

    def summary(self, name, work_fn):
        recs = self.records.get(name, [])
        ms = sum(s.elapsed_time(e) for s, e, _ in recs)
        work = sum(work_fn(w) for _, _, w in recs)
        return len(recs), ms, work


def attention_flops(work):
    """4 * sum(len^2) * C for one launch (QK^T and PV, 2 flops per multiply-add)."""
    cu, channels = work
    lens = torch.diff(cu.long()).double()
    return float(4.0 * (lens * lens).sum().item() * channels)


def build_inputs(n_scenes, pts_per_scene, seed0):
    from pointtransformerv3_amd import synthetic
    scenes = [synthetic.room_scene(pts_per_scene, seed0 + i, 0.02) for i in range(n_scenes)]
    d = synthetic.collate(scenes)
    feat = synthetic.room_features(d["coord"], seed0)
    return d, feat


def cpu_baseline(model, d, feat):
    """The CPU oracle (fp32, torch CPU operators) on the first scene of the batch."""
    from oracle.forward import ptv3_forward
    n0 = int(d["offset"][0])
    sd = {k: v.float().cpu() for k, v in model.state_dict().items()}
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    t0 = time.perf_counter()
    ptv3_forward(sd, d["grid_coord"][:n0], feat[:n0], d["offset"][:1])
    dt = time.perf_counter() - t0
    return {"value": n0 / dt, "unit": "points/s", "cores": cores, "kind": "port",
            "sample": f"one forward of the CPU oracle over scene 0 of the batch ({n0} points), {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--scenes", type=int, default=4)
    ap.add_argument("--points", type=int, default=106_000, help="points drawn per scene before voxel dedup")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (scenes would shard across "
              "GPUs with no exchange in inference); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    from pointtransformerv3_amd import PointTransformerV3, ops

    dev = "cuda:0"
    torch.manual_seed(0)
    model = PointTransformerV3().eval().half()
    d, feat = build_inputs(args.scenes, args.points, 4000)
    n_points = len(feat)
    cpu = None if args.no_cpu else cpu_baseline(model, d, feat)
    model = model.to(dev)
    data = dict(feat=torch.from_numpy(feat).to(dev).half(), grid_coord=torch.from_numpy(d["grid_coord"]).to(dev),
                coord=torch.from_numpy(d["coord"]).to(dev), offset=torch.from_numpy(d["offset"]).to(dev))

    def step():
        with torch.inference_mode():
            return model(dict(data))

    for _ in range(args.warmup):
        step()
    timer = LaunchTimer()
    ops.set_launch_timer(timer)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        out = step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ops.set_launch_timer(None)
    assert torch.isfinite(out.feat.float()).all()

    ms_per_step = wall / args.steps * 1e3
    launches, attn_ms, attn_flops = timer.summary("patch_attn", attention_flops)
    achieved = attn_flops / (attn_ms * 1e-3) / 1e12 if attn_ms > 0 else 0.0
    result = {
        "metric": "PTv3 fwd points/sec (4x100k-pt scenes)",
        "value": n_points / (ms_per_step * 1e-3),
        "unit": "points/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": f"full PTv3 encoder-decoder forward, default architecture, {args.scenes} room "
                               f"scenes, {n_points} voxelised points, grid 0.02 m, 6-dim input, random-init weights"},
        "roofline": {"bound": "mfma", "kernel": "patch_attn_half_kernel<f16>", "achieved": achieved,
                     "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                     "traffic": None, "launches": launches,
                     "avg_launch_us": attn_ms * 1e3 / max(launches, 1),
                     "flops_per_launch": attn_flops / max(launches, 1),
                     "attn_ms_per_step": attn_ms / args.steps},
        "cpu_baseline": cpu,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()

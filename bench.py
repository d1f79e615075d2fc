"""Benchmark of the PTv3 forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

A step is one full PointTransformerV3 forward (default architecture, fp16, eval) over a batch
of 4 synthetic room scenes of ~100k voxelised points each, inputs resident in HBM. Prints one
JSON line: throughput in points/s, the roofline of the dominant kernel (patch attention,
MFMA-bound nominally, VALU-bound in fact: both fractions are given) and of the sparse convolutions,
measured with HIP events around every launch inside the timed region, the CPU oracle timed on
this machine's host cores (one of the four scenes, and baseline config 1 in full), and short
runs of the other baseline configurations (5, 2, 3) after the timed region.
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
HBM_PEAK_GBS = 8000.0


class LaunchTimer:
    """HIP events around selected kernel launches, on the stream they are launched on."""

    def __init__(self, names=None):
        self.records = {}
        self.names = names   # None: every launch the operators announce; else only these (an event pair costs a
                             # few microseconds of idle queue on either side of the launch it brackets)

    def launch(self, name, work, fn):
        if self.names is not None and name not in self.names:
            return fn()
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


def conv_flops(work):
    """2 * active pairs * Cin * Cout for one convolution launch (pair or tile form)."""
    n_pairs, n, cin, cout, taps, form = work
    return 2.0 * n_pairs * cin * cout


def conv_min_bytes(work):
    """Rows in and out once, the weights once, one index per pair."""
    n_pairs, n, cin, cout, taps, form = work
    return 2.0 * n * (cin + cout) + 2.0 * taps * cin * cout + 4.0 * n_pairs


def encode_bytes(work):
    """12 B of coordinates + 8 B of scene id read, k codes of 8 B written, per point."""
    n, k = work
    return n * (12.0 + 8.0 + 8.0 * k)


def argsort_bytes(work):
    """An 8-bit-digit LSD radix sort that reads and writes (key, index) once per pass, then writes order and
    inverse: per point and order 24 B per pass + 16 B, passes = ceil(significant bits / 8)."""
    n, k, bits = work
    return float(k) * n * (((bits + 7) // 8) * 24.0 + 16.0)


def kmap_bytes(work):
    """16 B of [batch, x, y, z] read and one 4-byte entry per kernel offset written, per voxel and build (the byte
    model of a stored neighbour map; the pair lists that are written instead are smaller). The count and fill
    passes of one build are two timed regions: the bytes are booked on the first."""
    n, ks, part = work
    return 0.0 if part == "fill" else n * (16.0 + 4.0 * ks ** 3)


def hbm_entry(timer, name, bytes_fn, steps, kernels):
    launches, ms, byts = timer.summary(name, bytes_fn)
    gbs = byts / (ms * 1e-3) / 1e9 if ms > 0 else 0.0
    return {"kernels": kernels, "bound": "hbm", "launches": launches, "ms_per_step": ms / steps, "achieved": gbs,
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
            "bytes_per_step": byts / steps}


def index_kernels_alone(d):
    """encode, argsort and the pair-list build called alone, 20 times back to back (so that the queue never runs
    dry and the time is the kernels', not the host's): at the benchmark batch, and at 16 times its points (64
    scenes), where these kernels are long enough for bandwidth rather than launch and ramp-up to set the time."""
    from pointtransformerv3_amd import ops
    dev = "cuda:0"
    g = torch.from_numpy(d["grid_coord"]).to(dev)
    b = torch.from_numpy(d["batch"]).to(dev)
    orders = ["z", "z-trans", "hilbert", "hilbert-trans"]
    out = {"encode": {}, "sort": {}, "kmap": {}}

    def entry(us, byts):
        gbs = byts / us / 1e3
        return {"us": us, "achieved": gbs, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}

    for tag, reps in (("alone", 1), ("alone_16x", 16)):
        gg = g.repeat(reps, 1)
        bb = (b[None, :] + 4 * torch.arange(reps, device=dev)[:, None]).reshape(-1)
        n = len(bb)
        depth = 9
        bits = 3 * depth + int(4 * reps - 1).bit_length()
        iters = 20 if reps == 1 else 5
        us = _time_us(lambda: ops.encode_orders(gg, bb, depth, orders), iters=iters)
        out["encode"][tag] = dict(entry(us, encode_bytes((n, 4))), points=n)
        code = ops.encode_orders(gg, bb, depth, orders)
        us = _time_us(lambda: ops.argsort_rows(code, bits), iters=iters)
        out["sort"][tag] = dict(entry(us, argsort_bytes((n, 4, bits))), points=n, key_bits=bits)
        del code
        idx = torch.cat([bb[:, None].int(), gg.int()], 1).contiguous()
        for ks in (3, 5):
            us = _time_us(lambda: ops.conv_plan_direct(idx, ks), iters=iters)
            out["kmap"][f"{tag}_{ks}x{ks}x{ks}"] = dict(entry(us, kmap_bytes((n, ks, "count"))), voxels=n)
        del idx, gg, bb
    return out


# per 64 keys x 32 queries a wave has to issue 32 v_exp_f32 (8 cycles each on this part) and 16 packed conversions
# (4 each) whatever else it does: 320 VALU cycles per 2048 scores and SIMD
VALU_CYCLES_PER_SCORE = 320.0 / 2048.0
NOMINAL_CLOCK_HZ = 2.4e9
N_SIMDS = 1024


def recorded_traffic(n_points):
    """HBM bytes per attention launch from the committed rocprofv3 --pmc summary of this same
    workload (FETCH_SIZE and WRITE_SIZE runs, each scaled by a 1 GiB copy in the same process);
    None when the summary is for another workload."""
    path = os.path.join(ROOT, "profiles", "attention_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    return rec.get("traffic_bytes_per_launch") if rec.get("workload_points") == n_points else None


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
            "sample": f"one forward of the CPU oracle over scene 0 of the batch ({n0} points), {dt:.1f} s",
            "config1": cpu_baseline_config1(cores)}


def cpu_baseline_config1(cores):
    """Baseline configuration 1 on the host cores: z-order + Hilbert serialization (adaptive depth and depth 16) of
    16,384 points uniform in a 5 m cube, then one attention block (patch 1024, C = 64, 4 heads) in fp32 through
    the CPU oracle. Median of 3."""
    from oracle import functional as OF
    from oracle import indexing as OI
    from oracle import serialization as OS
    from pointtransformerv3_amd import synthetic
    sc = synthetic.cube_scene(16_384, 1000, 0.02)
    grid = sc["grid_coord"]
    n = len(grid)
    batch = np.zeros(n, np.int64)
    gen = torch.Generator().manual_seed(1001)
    feat = torch.randn(n, 64, generator=gen)
    wq, bq = torch.randn(192, 64, generator=gen) / 8, torch.zeros(192)
    wp, bp = torch.randn(64, 64, generator=gen) / 8, torch.zeros(64)
    pad, unpad, cu = OI.padding_tables(np.array([n], np.int64), 1024)
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        OS.serialize(grid, batch, ["z", "hilbert"])
        _, _, order, inverse = OS.serialize(grid, batch, ["z", "hilbert"], depth=16)
        qkv = torch.nn.functional.linear(feat, wq, bq)
        core = OF.serialized_attention_core(qkv, order[1], inverse[1], pad, unpad, cu, 4)
        torch.nn.functional.linear(core, wp, bp)
        times.append(time.perf_counter() - t0)
    med = sorted(times)[1]
    return {"value": n / med, "unit": "points/s", "cores": cores, "kind": "port",
            "sample": f"baseline config 1 in full (16,384 points: z + Hilbert serialization at depth 8 and 16, one "
                      f"attention block, fp32), median of 3: {med * 1e3:.0f} ms"}


def _time_us(fn, iters=20, warmup=3):
    """Average device time of fn() in microseconds (HIP events on the current stream)."""
    for _ in range(warmup):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 1e3 / iters


def attention_config2(reps, dtype=torch.float16):
    """Baseline config 2 alone: Hilbert order of one room scene, patch 1024, C=512, 32 heads."""
    from pointtransformerv3_amd import ops, synthetic
    dev = "cuda:0"
    sc = synthetic.room_scene(106_000, 2000, 0.02)
    n2 = len(sc["grid_coord"])
    g2 = torch.from_numpy(sc["grid_coord"]).to(dev)
    b2 = torch.zeros(n2, dtype=torch.int64, device=dev)
    order2, inv2 = ops.argsort_rows(ops.encode_orders(g2, b2, 9, ["hilbert"]), 28)
    pad2, unpad2, cu2 = ops.pad_index(torch.tensor([n2], device=dev), [n2], 1024)
    src2, dst2 = ops.attn_slots(order2[0], inv2[0], pad2, unpad2)
    gen = torch.Generator(device="cpu").manual_seed(2)
    qkv = (torch.randn(n2, 3 * 512, generator=gen) / 4).to(dtype).to(dev)
    us = _time_us(lambda: ops.patch_attention(qkv, 32, src2, dst2, cu2, 1024, 0.25), iters=reps, warmup=1)
    lens = torch.diff(cu2.long()).double()
    fl = float(4.0 * (lens * lens).sum().item() * 512)
    name = {torch.float16: "f16", torch.bfloat16: "bf16"}[dtype]
    return {"kernel": f"patch_attn_half_kernel<{name}>", "points": n2, "sequences": int(len(cu2) - 1), "heads": 32,
            "us": us, "flops": fl, "tflops": fl / us / 1e6, "frac_mfma_peak": fl / us / 1e6 / MFMA_PEAK_TFLOPS}


ENC_CHANNELS = (32, 64, 128, 256, 512)


class _FormProbe:
    """Stands in for the launch timer for one call: remembers the form of the convolution that was launched."""
    form = "dense"

    def launch(self, kind, work, call):
        if kind == "subm_conv":
            self.form = work[-1]
        call()


def conv_case(which, reps):
    """The xCPE convolution alone, through the module's own dispatch (pair, tile, sparse tile or dense form), fp16:
    `config3` = baseline config 3 (200,000 room voxels at 2 cm, 64 -> 64); `level0` .. `level4` = the voxel set
    of that encoder level of the benchmark batch (4 rooms pooled with stride 2 per level) at that level's width.
    Returns the time per call against both rooflines (printed as one JSON line by --conv: the command to put under
    rocprofv3)."""
    from pointtransformerv3_amd import ops, synthetic
    from pointtransformerv3_amd.sparse import SparseConvTensor, SubMConv3d
    dev = "cuda:0"
    if which == "config3":
        vox = synthetic.room_voxels(200_000, 3000)["grid_coord"]
        idx = torch.from_numpy(np.concatenate([np.zeros((len(vox), 1), np.int32), vox], 1)).to(dev)
        channels, label = 64, "baseline config 3: 200,000 room voxels at 2 cm"
    else:
        level = int(which[len("level"):])
        d, _ = build_inputs(4, 106_000, 4000)
        full = torch.from_numpy(np.concatenate([d["batch"][:, None].astype(np.int32), d["grid_coord"]], 1)).to(dev)
        full[:, 1:] >>= level
        idx = torch.unique(full, dim=0).contiguous() if level else full.contiguous()
        channels = ENC_CHANNELS[level]
        label = f"encoder level {level} of the benchmark batch ({2 << level} cm voxels)"
    n = len(idx)
    gen = torch.Generator(device="cpu").manual_seed(3)
    conv = SubMConv3d(channels, channels, 3, bias=True, indice_key="bench").to(dev).half()
    x = SparseConvTensor(torch.randn(n, channels, generator=gen).half().to(dev), idx, [1, 1, 1], 4)
    with torch.inference_mode():
        plan = x.conv_plan(3, "bench")
        per_voxel = plan.n_pairs / n
        probe = _FormProbe()          # which form the module's dispatch picks: what the operator layer reports
        ops.set_launch_timer(probe)
        conv(x)
        ops.set_launch_timer(None)
        form = probe.form
        us = _time_us(lambda: conv(x), iters=reps, warmup=2)
    flops = 2.0 * plan.n_pairs * channels * channels
    min_bytes = 2.0 * n * channels * 2 + 27.0 * channels * channels * 2 + 4.0 * plan.n_pairs
    return {"workload": label, "voxels": n, "channels": channels, "pairs": plan.n_pairs,
            "pairs_per_voxel": per_voxel, "form": form, "us": us, "flops": flops, "tflops": flops / us / 1e6,
            "frac_mfma_peak": flops / us / 1e6 / MFMA_PEAK_TFLOPS, "min_bytes": min_bytes,
            "gbs": min_bytes / us / 1e3, "frac_hbm_peak": min_bytes / us / 1e3 / HBM_PEAK_GBS}


DENSE_CASES = {   # name: (rows, channels) at the levels of the benchmark batch
    "tail64": (308_615, 64), "tail32": (403_093, 32), "head64": (308_615, 64), "mlp128": (146_195, 128),
    "mlp256": (37_681, 256), "linear_ln256": (37_681, 256),
    "tail128": (146_195, 128), "tail256": (37_681, 256), "head128": (146_195, 128),
}


def dense_case(which, reps):
    """One fused dense kernel of a transformer block alone at the rows and width of a level of the benchmark batch,
    fp16: `tail*` = proj + residual + LayerNorm + MLP + residual (block_tail_kernel; from 128 channels on the tail mode
    of mlp_wide_kernel), `head*` = cpe Linear + LayerNorm + residual + LayerNorm + qkv Linear (block_head_kernel, the
    head mode of mlp_wide_kernel), `mlp*` = fc1 + GELU + fc2 + residual (mlp_wide_kernel on packed weights),
    `linear_ln256` = proj Linear + residual + LayerNorm. The command to put under rocprofv3 --pmc."""
    from pointtransformerv3_amd import ops
    from pointtransformerv3_amd.modules import MLP
    dev = "cuda:0"
    n, c = DENSE_CASES[which]
    torch.manual_seed(3)
    lin = lambda i, o: torch.nn.Linear(i, o).half().to(dev)
    ln = lambda: torch.nn.LayerNorm(c).half().to(dev)
    x, res = torch.randn(n, c, device=dev).half(), torch.randn(n, c, device=dev).half()
    gelus, flops, byts = 0, 0.0, 0.0
    if which.startswith("tail"):
        proj, ln2, fc1, fc2 = lin(c, c), ln(), lin(c, 4 * c), lin(4 * c, c)
        if c >= 128:      # the TAIL mode of mlp_wide_kernel
            from pointtransformerv3_amd.modules import LayerNorm
            mlp, ln2 = MLP(c, 4 * c).half().to(dev), LayerNorm(c).half().to(dev)
            fn = lambda: ops.block_tail_wide(x, res, proj, ln2, mlp)
        else:
            fn = lambda: ops.block_tail_fused(x, res, proj, ln2, fc1, fc2)
        gelus, flops, byts = 4 * n * c, 2.0 * n * c * c * 9, 3.0 * n * c * 2
    elif which.startswith("head"):
        cpe, lnc, ln1, qkv = lin(c, c), ln(), ln(), lin(c, 3 * c)
        fn = (lambda: ops.block_head_wide(x, res, cpe, lnc, ln1, qkv)) if c >= 128 else (
            lambda: ops.block_head_fused(x, res, cpe, lnc, ln1, qkv))
        flops, byts = 2.0 * n * c * c * 4, 6.0 * n * c * 2
    elif which.startswith("mlp"):
        mlp = MLP(c, 4 * c).half().to(dev)
        fn = lambda: ops.mlp_fused_module(x, res, mlp)
        gelus, flops, byts = 4 * n * c, 2.0 * n * c * c * 8, 3.0 * n * c * 2
    else:
        proj, ln2 = lin(c, c), ln()
        fn = lambda: ops.linear_ln(x, proj, res, ln2, 2)
        flops, byts = 2.0 * n * c * c, 4.0 * n * c * 2
    us = _time_us(fn, iters=reps, warmup=3)
    return {"workload": which, "rows": n, "channels": c, "us": us, "flops": flops, "tflops": flops / us / 1e6,
            "frac_mfma_peak": flops / us / 1e6 / MFMA_PEAK_TFLOPS, "min_bytes": byts, "gbs": byts / us / 1e3,
            "frac_hbm_peak": byts / us / 1e3 / HBM_PEAK_GBS, "gelu_evaluations": gelus}


def other_configs():
    """The baseline configurations that are not the headline, a few iterations each: config 5 (two LiDAR-like sweeps,
    full forward, fp16), config 2 (patch attention alone, bf16), config 3 (pair lists + 3x3x3 convolution alone, fp16)."""
    from pointtransformerv3_amd import PointTransformerV3, ops, synthetic
    dev = "cuda:0"
    res = {}
    # ---- config 5
    scenes = [synthetic.lidar_scene(5000 + i, 0.05) for i in range(2)]
    d = synthetic.collate(scenes)
    feat = synthetic.lidar_features(d["coord"], 5000)
    torch.manual_seed(5)
    model = PointTransformerV3(in_channels=4).eval().half().to(dev)
    data = dict(feat=torch.from_numpy(feat).to(dev).half(), grid_coord=torch.from_numpy(d["grid_coord"]).to(dev),
                offset=torch.from_numpy(d["offset"]).to(dev))
    with torch.inference_mode():
        for _ in range(3):
            out = model(dict(data))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            out = model(dict(data))
        torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / 10 * 1e3
    assert torch.isfinite(out.feat.float()).all()
    res["config5_lidar_forward_fp16"] = {"points": len(feat), "scenes": 2, "ms": ms, "points_per_s": len(feat) / ms * 1e3}
    del model, data, out
    # ---- config 2
    a = attention_config2(10, torch.bfloat16)
    res["config2_attention_bf16"] = {"points": a["points"], "ms": a["us"] / 1e3, "points_per_s": a["points"] / a["us"] * 1e6,
                                     "tflops": a["tflops"], "frac_mfma_peak": a["frac_mfma_peak"]}
    # ---- config 3
    c = conv_case("config3", 10)
    vox = synthetic.room_voxels(200_000, 3000)["grid_coord"]
    idx = torch.from_numpy(np.concatenate([np.zeros((len(vox), 1), np.int32), vox], 1)).to(dev)
    kmap_us = _time_us(lambda: ops.conv_plan_direct(idx, 3), iters=10)
    res["config3_kmap_conv_fp16"] = {"voxels": c["voxels"], "pairs": c["pairs"], "kmap_us": kmap_us, "conv_us": c["us"],
                                     "ms": (kmap_us + c["us"]) / 1e3, "voxels_per_s": c["voxels"] / (kmap_us + c["us"]) * 1e6,
                                     "conv_tflops": c["tflops"], "conv_frac_mfma_peak": c["frac_mfma_peak"],
                                     "conv_frac_hbm_peak": c["frac_hbm_peak"]}
    return res


def kernel_rooflines(path):
    """Per-kernel measurements at the sizes the baseline configs name, each against the roofline
    that bounds it (algorithmic bytes or flops / measured time). Written to `path` as JSON."""
    from pointtransformerv3_amd import ops, synthetic
    dev = "cuda:0"
    rows = []

    def add(name, workload, bound, work, us, unit_work):
        ach = work / (us * 1e-6) / (1e9 if bound == "hbm" else 1e12)
        peak = HBM_PEAK_GBS if bound == "hbm" else MFMA_PEAK_TFLOPS
        rows.append({"kernel": name, "workload": workload, "bound": bound, "us": us, "work": work,
                     "work_unit": unit_work, "achieved": ach, "peak": peak,
                     "unit": "GB/s" if bound == "hbm" else "TFLOP/s", "frac": ach / peak})

    # ---- serialization: 4 room scenes, k = 4 orders, depth 9 (adaptive) and 16 (explicit)
    d, _ = build_inputs(4, 106_000, 4000)
    n = len(d["batch"])
    g = torch.from_numpy(d["grid_coord"]).to(dev)
    b = torch.from_numpy(d["batch"]).to(dev)
    orders = ["z", "z-trans", "hilbert", "hilbert-trans"]
    for depth in (9, 16):
        us = _time_us(lambda: ops.encode_orders(g, b, depth, orders))
        add("encode", f"{n} points, 4 orders, depth {depth}", "hbm", n * 52.0, us, "B (52 B/point)")
        code = ops.encode_orders(g, b, depth, orders)
        bits = 3 * depth + 2
        passes = (bits + 7) // 8
        us = _time_us(lambda: ops.argsort_rows(code, bits))
        add("argsort+inverse", f"4 x {n} codes, {bits} significant bits, {passes} passes", "hbm",
            4.0 * n * (passes * 24 + 16), us, f"B ({passes * 24 + 16} B per point and order)")
    # ---- the same two at 16x the points (64 scenes): at 400k points these kernels run for a few
    # microseconds each, a size at which launch and ramp-up, not bandwidth, set the time
    reps = 16
    g_big = g.repeat(reps, 1)
    b_big = (b[None, :] + 4 * torch.arange(reps, device=dev)[:, None]).reshape(-1)
    nb = n * reps
    us = _time_us(lambda: ops.encode_orders(g_big, b_big, 9, orders), iters=10)
    add("encode", f"{nb} points (64 scenes), 4 orders, depth 9", "hbm", nb * 52.0, us, "B (52 B/point)")
    code_big = ops.encode_orders(g_big, b_big, 9, orders)
    bits = 27 + 6
    passes = (bits + 7) // 8
    us = _time_us(lambda: ops.argsort_rows(code_big, bits), iters=5)
    add("argsort+inverse", f"4 x {nb} codes, {bits} significant bits, {passes} passes", "hbm",
        4.0 * nb * (passes * 24 + 16), us, f"B ({passes * 24 + 16} B per point and order)")
    del code_big
    # ---- for scale: a device-to-device copy of as many bytes as the encode above moves (what a kernel that does
    # nothing but move its algorithmic bytes reaches on this part)
    half_bytes = nb * 52 // 2 // 8 * 8
    src = torch.zeros(half_bytes // 8, dtype=torch.int64, device=dev)
    dst = torch.empty_like(src)
    us = _time_us(lambda: dst.copy_(src), iters=20)
    add("device copy (reference)", f"{half_bytes / 1e6:.0f} MB read + {half_bytes / 1e6:.0f} MB written", "hbm", 2.0 * half_bytes, us, "B")
    del src, dst
    # ---- padding tables + slot tables
    off_host = [int(v) for v in d["offset"]]
    off = torch.from_numpy(d["offset"]).to(dev)
    us = _time_us(lambda: ops.pad_index(off, off_host, 1024))
    pad, unpad, cu = ops.pad_index(off, off_host, 1024)
    add("pad_index", f"{n} points, patch 1024", "hbm", 8.0 * (len(pad) + n) + 4.0 * len(cu), us, "B")
    # ---- config 2: patch attention alone, bf16, one 100k-point scene, C=512, H=32
    sc = synthetic.room_scene(106_000, 2000, 0.02)
    n2 = len(sc["grid_coord"])
    g2 = torch.from_numpy(sc["grid_coord"]).to(dev)
    b2 = torch.zeros(n2, dtype=torch.int64, device=dev)
    code2 = ops.encode_orders(g2, b2, 9, ["hilbert"])
    order2, inv2 = ops.argsort_rows(code2, 28)
    off2 = torch.tensor([n2], device=dev)
    pad2, unpad2, cu2 = ops.pad_index(off2, [n2], 1024)
    src2, dst2 = ops.attn_slots(order2[0], inv2[0], pad2, unpad2)
    gen = torch.Generator(device="cpu").manual_seed(2)
    for dt, nm in ((torch.bfloat16, "bf16"), (torch.float16, "f16")):
        qkv = (torch.randn(n2, 3 * 512, generator=gen) / 4).to(dt).to(dev)
        us = _time_us(lambda: ops.patch_attention(qkv, 32, src2, dst2, cu2, 1024, 0.25), iters=10)
        lens = torch.diff(cu2.long()).double()
        fl = float(4.0 * (lens * lens).sum().item() * 512)
        add(f"patch_attn<{nm}>", f"{n2} points (Hilbert order), patch 1024, C=512, 32 heads", "mfma", fl, us,
            "FLOP (4 * sum len^2 * C)")
    # ---- config 3: kmap + SubMConv3d 3x3x3 on 200k voxels, C=64, fp16
    vox = synthetic.room_voxels(200_000, 3000)["grid_coord"]
    idx = torch.from_numpy(np.concatenate([np.zeros((len(vox), 1), np.int32), vox], 1)).to(dev)
    nv = len(vox)
    us = _time_us(lambda: ops.kmap_build(idx, 3, tap_major=True))
    add("kmap 3x3x3", f"{nv} voxels", "hbm", nv * 124.0, us, "B (124 B/voxel)")
    nbr = ops.kmap_build(idx, 3, tap_major=True)
    us = _time_us(lambda: ops.conv_plan(nbr, tap_major=True), iters=10)
    plan = ops.conv_plan(nbr, tap_major=True)
    add("conv_plan", f"{nv} voxels, {plan.n_pairs} active pairs", "hbm", nv * 27 * 4.0 * 2 + plan.n_pairs * 8.0 + nv * 4.0,
        us, "B (map read twice, pair lists written)")
    us = _time_us(lambda: ops.conv_plan_direct(idx, 3), iters=10)
    add("kmap+plan direct 3x3x3", f"{nv} voxels, {plan.n_pairs} active pairs", "hbm", nv * 16.0 + plan.n_pairs * 8.0 + nv * 4.0,
        us, "B (coordinates read, pair lists written; no stored map)")
    idx_big = torch.cat([torch.cat([b_big[:, None].int(), g_big.int()], 1)]).contiguous()
    for ks in (3, 5):
        us = _time_us(lambda: ops.conv_plan_direct(idx_big, ks), iters=5)
        pb = ops.conv_plan_direct(idx_big, ks)
        add(f"kmap+plan direct {ks}x{ks}x{ks}", f"{nb} voxels (64 scenes), {pb.n_pairs} active pairs", "hbm",
            nb * 16.0 + pb.n_pairs * 8.0 + nb * 4.0, us, "B (coordinates read, pair lists written; no stored map)")
        del pb
    del idx_big
    feat = torch.randn(nv, 64, generator=gen).half().to(dev)
    w = ((torch.rand(64, 27, 64, generator=gen) * 2 - 1) / np.sqrt(27 * 64)).half().to(dev)
    bias = torch.zeros(64).half().to(dev)
    us = _time_us(lambda: ops.subm_conv_pairs(feat, plan, w, bias))
    add("subm_conv pairs<f16>", f"{nv} voxels, {plan.n_pairs} pairs ({plan.n_pairs / nv:.2f}/voxel), 64->64", "mfma",
        2.0 * plan.n_pairs * 64 * 64, us, "FLOP (2 * P_act * Cin * Cout)")
    us = _time_us(lambda: ops.subm_conv(feat, nbr, w, bias, tap_major=True))
    add("subm_conv dense<f16>", f"{nv} voxels, all 27 taps visited, 64->64", "mfma", 2.0 * plan.n_pairs * 64 * 64, us,
        "FLOP (2 * P_act * Cin * Cout)")
    packed = ops.conv_pack_weight(w, 27, torch.float16)
    plan.tiles()
    us = _time_us(lambda: ops.subm_conv_tiles(feat, plan, packed, bias))
    add("subm_conv tiles<f16>", f"{nv} voxels, {plan.n_pairs} pairs ({plan.n_pairs / nv:.2f}/voxel), 64->64", "mfma",
        2.0 * plan.n_pairs * 64 * 64, us, "FLOP (2 * P_act * Cin * Cout)")
    us = _time_us(lambda: ops.subm_conv_sparse(feat, plan, packed, bias))
    add("subm_conv sparse tiles<f16>", f"{nv} voxels, {plan.n_pairs} pairs ({plan.n_pairs / nv:.2f}/voxel), 64->64", "mfma",
        2.0 * plan.n_pairs * 64 * 64, us, "FLOP (2 * P_act * Cin * Cout); the form the model's dispatch picks here")
    # the level the forward runs the tile form on: the 4-scene batch pooled twice (8 cm voxels), 128 channels
    lvl = torch.unique(torch.cat([b[:, None].int(), (g >> 2).int()], 1), dim=0).contiguous()
    nl = len(lvl)
    plan2 = ops.conv_plan_direct(lvl, 3)
    plan2.tiles()
    feat2 = torch.randn(nl, 128, generator=gen).half().to(dev)
    w2 = ((torch.rand(128, 27, 128, generator=gen) * 2 - 1) / np.sqrt(27 * 128)).half().to(dev)
    bias2 = torch.zeros(128).half().to(dev)
    packed2 = ops.conv_pack_weight(w2, 27, torch.float16)
    for name, fn in (("subm_conv pairs<f16>", lambda: ops.subm_conv_pairs(feat2, plan2, w2, bias2)),
                     ("subm_conv tiles<f16>", lambda: ops.subm_conv_tiles(feat2, plan2, packed2, bias2))):
        us = _time_us(fn)
        add(name, f"{nl} voxels (4 scenes at 8 cm), {plan2.n_pairs} pairs ({plan2.n_pairs / nl:.2f}/voxel), 128->128", "mfma",
            2.0 * plan2.n_pairs * 128 * 128, us, "FLOP (2 * P_act * Cin * Cout)")
    del plan2, feat2, w2, packed2, lvl
    # ---- voxelisation in front of the model: the 4 rooms' raw points (before the one-point-per-voxel cut)
    raw = [synthetic.room_points(106_000, 4000 + i).astype(np.float32) for i in range(4)]
    raw_coord = torch.from_numpy(np.concatenate(raw)).to(dev)
    raw_off = torch.from_numpy(np.cumsum([len(r) for r in raw])).to(dev)
    us = _time_us(lambda: ops.voxelize(raw_coord, raw_off, 0.02), iters=10)
    kept = len(ops.voxelize(raw_coord, raw_off, 0.02)["index"])
    nr = len(raw_coord)
    add("voxelize", f"{nr} points (4 rooms) -> {kept} voxels at 2 cm", "hbm", 20.0 * nr + 20.0 * kept, us,
        "B (12 B coordinates read + 8 B inverse written per point, 20 B grid_coord + index per voxel)")
    del raw, raw_coord
    # ---- pooling on the 4-scene batch
    code = ops.encode_orders(g, b, 9, orders)
    order, inverse = ops.argsort_rows(code, 29)
    us = _time_us(lambda: ops.pool_clusters(code[0], order[0], 3), iters=10)
    cluster, idx_ptr, head, m = ops.pool_clusters(code[0], order[0], 3)
    add("pool_clusters", f"{n} points -> {m} clusters", "hbm", 24.0 * n + 16.0 * m, us, "B")
    x = torch.randn(n, 64, generator=gen).half().to(dev)
    us = _time_us(lambda: ops.segment_reduce(x, order[0], idx_ptr, "max"))
    add("segment_reduce max<f16>", f"{n} x 64 -> {m} x 64", "hbm", (n * 64 + m * 64) * 2.0 + 8.0 * n, us, "B")
    child = torch.randn(m, 64, generator=gen).half().to(dev)
    us = _time_us(lambda: ops.unpool_add(x, child, cluster))
    add("unpool_add<f16>", f"{n} x 64", "hbm", (2 * n * 64 + m * 64) * 2.0 + 8.0 * n, us, "B")
    # ---- fused MLP (fc1 + GELU + fc2 + residual) at the widths and sizes of the model's levels
    for nm, cm in ((n, 64), (148_000, 128)):
        xm = torch.randn(nm, cm, generator=gen).half().to(dev)
        w1 = (torch.randn(4 * cm, cm, generator=gen) / cm ** 0.5).half().to(dev)
        w2 = (torch.randn(cm, 4 * cm, generator=gen) / (4 * cm) ** 0.5).half().to(dev)
        bm1, bm2 = torch.zeros(4 * cm).half().to(dev), torch.zeros(cm).half().to(dev)
        us = _time_us(lambda: ops.mlp_fused(xm, xm, w1, bm1, w2, bm2))
        add("mlp_fused<f16>", f"{nm} x {cm}, hidden {4 * cm}", "mfma", 16.0 * nm * cm * cm, us, "FLOP (16 N C^2)")
    wln = torch.ones(64).half().to(dev)
    us = _time_us(lambda: ops.layer_norm(x, wln, wln, 1e-5, residual=x, mode=2))
    add("layer_norm mode 2<f16>", f"{n} x 64", "hbm", 4.0 * n * 64 * 2, us, "B (2 reads, 2 writes)")

    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    with open(path, "w") as f:
        json.dump(rows, f, indent=1)
    for r in rows:
        print(f"{r['kernel']:26s} {r['us']:9.1f} us  {r['achieved']:9.1f} {r['unit']:8s} {100 * r['frac']:5.1f}% of peak   {r['workload']}",
              file=sys.stderr)


def training_step(args):
    """Forward + backward + AdamW of the default model in training mode (batch-norm batch statistics,
    stochastic depth 0.3, order shuffling) on the benchmark's input, cross-entropy against random labels
    through a 13-class linear head. Not the headline metric: reported beside it."""
    from pointtransformerv3_amd import PointTransformerV3
    dev = "cuda:0"
    dtype = getattr(torch, args.train)
    torch.manual_seed(0)
    model = PointTransformerV3().to(dev).train()
    head = torch.nn.Linear(64, 13).to(dev)
    opt = torch.optim.AdamW(list(model.parameters()) + list(head.parameters()), lr=1e-3, fused=True)
    d, feat = build_inputs(args.scenes, args.points, 4000)
    n_points = len(feat)
    data = dict(feat=torch.from_numpy(feat).to(dev), grid_coord=torch.from_numpy(d["grid_coord"]).to(dev),
                offset=torch.from_numpy(d["offset"]).to(dev))
    target = torch.randint(0, 13, (n_points,), device=dev)

    def step():
        opt.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=dtype):
            out = model(dict(data)).feat
            loss = torch.nn.functional.cross_entropy(head(out).float(), target)
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    assert torch.isfinite(loss.detach())
    print(json.dumps({
        "metric": "PTv3 training step points/sec (4x100k-pt scenes)", "value": n_points / (ms * 1e-3), "unit": "points/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": {"bfloat16": "bf16", "float16": "f16"}[args.train],
        "data": "synthetic",
        "config": {"workload": f"forward + backward + fused AdamW, default architecture in training mode, autocast, "
                               f"{args.scenes} room scenes, {n_points} voxelised points, grid 0.02 m"},
        "peak_memory_gib": torch.cuda.max_memory_allocated() / 2 ** 30}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50,
                    help="timed forwards (the first one after the synchronisation in front of the timed region runs "
                         "its index pass with nothing beside it: 50 steps keep that at 1 %% of the figure)")
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--scenes", type=int, default=4)
    ap.add_argument("--points", type=int, default=106_000, help="points drawn per scene before voxel dedup")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-overlap", action="store_true",
                    help="time the plain schedule only: by default the model's opt-in overlap_index_prologue is on (the "
                         "inputs are resident and complete before the timed region, which is what it asks for), so the "
                         "index work of forward k + 1 runs beside the feature kernels of forward k; the plain schedule is timed "
                         "after the timed region as well and reported beside it")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the short runs of baseline configs 5, 2 and 3 after the timed region")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device copy (a kernel of known traffic) so that rocprofv3 --pmc "
                         "FETCH_SIZE / WRITE_SIZE readings of this process can be scaled to bytes")
    ap.add_argument("--attention-config2", metavar="REPS", type=int, default=0,
                    help="only run the patch attention kernel at baseline config 2 (one 100k-point scene, C=512, 32 "
                         "heads, fp16) REPS times and print its rate: the command to put under rocprofv3 --pmc")
    ap.add_argument("--conv", metavar="CASE", default=None,
                    choices=["config3", "level0", "level1", "level2", "level3", "level4"],
                    help="only run the 3x3x3 submanifold convolution of one workload (baseline config 3, or one encoder "
                         "level of the benchmark batch at its width) --reps times and print its rate: the command to "
                         "put under rocprofv3 --pmc")
    ap.add_argument("--dense", metavar="CASE", default=None, choices=sorted(DENSE_CASES),
                    help="only run one fused dense kernel of a block (block tail / head, fused MLP, Linear + LayerNorm) "
                         "at the rows and width of a level of the benchmark batch --reps times and print its rate")
    ap.add_argument("--reps", type=int, default=20, help="timed calls of --conv / --dense")
    ap.add_argument("--train", metavar="DTYPE", default=None, choices=["bfloat16", "float16"],
                    help="instead of the forward benchmark, time a training step (forward, backward, AdamW) of the "
                         "same model and input under autocast to DTYPE and print its own JSON line")
    ap.add_argument("--micro", metavar="WHICH", default=None, choices=["issue", "loads"],
                    help="only run a microbenchmark of the part (libptv3_micro.so): `issue` = issue cycles of the "
                         "instructions the attention and GELU loops are made of, `loads` = vector-load throughput by "
                         "access pattern and working set; prints the report as text")
    ap.add_argument("--summarise", metavar="DIR", default=None,
                    help="no GPU work: turn the raw files a measurement batch left in DIR (JSON lines of this script, "
                         "rocprofv3 traces and counter collections) into the text summaries under --out; sections "
                         "whose raw files are missing say which command writes them")
    ap.add_argument("--recipe", action="store_true", help="with --summarise DIR: only print the measurement batch as shell lines")
    ap.add_argument("--out", metavar="DIR", default=os.path.join(ROOT, "profiles"), help="where --summarise writes")
    ap.add_argument("--kernels", metavar="PATH", default=None,
                    help="also measure every kernel alone against its roofline and write the table to PATH")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (scenes would shard across "
              "GPUs with no exchange in inference); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.summarise:
        import bench_summaries
        if args.recipe:
            print("\n".join(bench_summaries.recipe(args.summarise)))
        else:
            bench_summaries.summarise(args.summarise, args.out)
        return

    if args.micro:
        import ctypes
        path = os.path.join(ROOT, "pointtransformerv3_amd", "libptv3_micro.so")
        if not os.path.exists(path):
            sys.exit(f"{path} not found: build it with `make -C pointtransformerv3_amd/csrc`")
        lib = ctypes.CDLL(path)
        lib.ptv3_micro_run.restype = ctypes.c_int
        lib.ptv3_micro_run.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t]
        buf = ctypes.create_string_buffer(1 << 16)
        rc = lib.ptv3_micro_run(args.micro.encode(), buf, len(buf))
        print(buf.value.decode(), end="")
        sys.exit(0 if rc == 0 else f"ptv3_micro_run({args.micro}) failed with code {rc}")

    from pointtransformerv3_amd import PointTransformerV3, ops

    if args.attention_config2 > 0:
        print(json.dumps(attention_config2(args.attention_config2)))
        return
    if args.conv:
        print(json.dumps(conv_case(args.conv, args.reps)))
        return
    if args.dense:
        print(json.dumps(dense_case(args.dense, args.reps)))
        return
    if args.train:
        training_step(args)
        return
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

    def timed_loop(events):
        """`steps` forwards back to back between two synchronisations, with HIP events around the launches named."""
        t = LaunchTimer(events)
        ops.set_launch_timer(t)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            o = step()
        torch.cuda.synchronize()
        w = time.perf_counter() - t0
        ops.set_launch_timer(None)
        return t, w, o

    model.overlap_index_prologue = not args.no_overlap
    for _ in range(args.warmup):
        step()
    # the timed region: events around the launches of the dominant kernel only
    timer, wall, out = timed_loop({"patch_attn"})
    assert torch.isfinite(out.feat.float()).all()
    plain_ms = None
    if model.overlap_index_prologue:
        # the same loop on the plain schedule (every forward's index work in front of its own feature kernels)
        model.overlap_index_prologue = False
        for _ in range(2):
            step()
        plain_ms = timed_loop({"patch_attn"})[1] / args.steps * 1e3
    # and once more (plain schedule) with events around every launch the operators announce: the convolutions and the
    # index kernels against their rooflines, measured inside the forward but outside the timed region
    model.overlap_index_prologue = False
    for _ in range(2):
        step()
    every, every_wall, _ = timed_loop(None)
    model.overlap_index_prologue = not args.no_overlap

    ms_per_step = wall / args.steps * 1e3
    launches, attn_ms, attn_flops = timer.summary("patch_attn", attention_flops)
    achieved = attn_flops / (attn_ms * 1e-3) / 1e12 if attn_ms > 0 else 0.0
    # the bound that actually applies at head_dim 16: one exponential and half a conversion per score on the VALU
    scores = attn_flops / 64.0                       # flops = 4 * sum len^2 * C, scores = sum len^2 * C / 16
    exp_floor_ms = scores * VALU_CYCLES_PER_SCORE / N_SIMDS / NOMINAL_CLOCK_HZ * 1e3
    conv_launches, conv_ms, conv_fl = every.summary("subm_conv", conv_flops)
    _, _, conv_by = every.summary("subm_conv", conv_min_bytes)
    conv_tf = conv_fl / (conv_ms * 1e-3) / 1e12 if conv_ms > 0 else 0.0
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
                               f"scenes, {n_points} voxelised points, grid 0.02 m, 6-dim input, random-init weights",
                   "schedule": ("forwards back to back; the index pass of a forward (curve codes, sort, clusters, pooled "
                                "tables, pair and tile lists, attention tables of every level: no feature touched) runs on "
                                "its own stream beside the feature kernels of the forward before "
                                "(PointTransformerV3.overlap_index_prologue, for inputs resident before the call)"
                                if plain_ms is not None else "forwards back to back, plain schedule"),
                   "plain_schedule_ms_per_step": plain_ms,
                   "ms_per_step_with_events_around_every_launch": every_wall / args.steps * 1e3},
        "roofline": {"bound": "mfma", "kernel": "patch_attn_half_kernel<f16>", "achieved": achieved,
                     "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                     "traffic": recorded_traffic(n_points), "launches": launches,
                     "avg_launch_us": attn_ms * 1e3 / max(launches, 1),
                     "flops_per_launch": attn_flops / max(launches, 1),
                     "attn_ms_per_step": attn_ms / args.steps,
                     "valu_exp_floor_ms_per_step": exp_floor_ms / args.steps,
                     "valu_exp_frac": exp_floor_ms / attn_ms if attn_ms > 0 else 0.0,
                     "conv": {"kernels": "conv_sparse, conv_tile, pair_wstat / pair_gemm + pair_segment_sum",
                              "measured": "events around every convolution launch, in a loop of the same forwards "
                                          "right after the timed region (so are encode, sort and kmap below)",
                              "bound": "mfma", "launches": conv_launches, "ms_per_step": conv_ms / args.steps,
                              "achieved": conv_tf, "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                              "frac": conv_tf / MFMA_PEAK_TFLOPS,
                              "hbm_frac": (conv_by / (conv_ms * 1e-3) / 1e9 / HBM_PEAK_GBS) if conv_ms > 0 else 0.0}},
        "cpu_baseline": cpu,
    }
    # the index kernels inside the forward against HBM bandwidth, algorithmic bytes over the time between events
    result["roofline"]["encode"] = hbm_entry(every, "encode", encode_bytes, args.steps, "encode_kernel (4 orders in one pass)")
    result["roofline"]["sort"] = hbm_entry(every, "argsort", argsort_bytes, args.steps,
                                           "radix sort passes + order / inverse of the 4 code rows")
    result["roofline"]["kmap"] = hbm_entry(every, "kmap", kmap_bytes, args.steps,
                                           "voxel hash + pair lists of the 5 levels (5x5x5 and 3x3x3 at the first)")
    if not args.no_other_configs:
        del model, data, out
        for name, alone in index_kernels_alone(d).items():
            result["roofline"][name].update(alone)
        result["other_configs"] = other_configs()
    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)          # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
    if args.kernels:
        kernel_rooflines(args.kernels)
    print(json.dumps(result))


if __name__ == "__main__":
    main()

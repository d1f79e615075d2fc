"""`python bench.py --summarise DIR`: turn the raw files a measurement batch left in DIR (bench.py's JSON lines, rocprofv3's
kernel traces and counter collections) into the short text summaries kept under profiles/.

Every summary names the commands its figures come from. A section whose raw files are missing from DIR is skipped and
says which command writes them; `python bench.py --summarise DIR --recipe` prints the whole batch, in order, as shell
lines (run them from the repository root on the GPU box, `cd /tmp && export TMPDIR=/tmp` first; each rocprofv3 --pmc
line is a run of its own and holds at most 8 SQ and 4 TCC counters).
"""
import collections
import csv
import glob
import json
import os
import re

POINTS = 403_093
# what FETCH_SIZE / WRITE_SIZE (KiB) read for a 1 GiB device-to-device copy gives these; refreshed by the attention
# traffic section when DIR holds a calibration run
FETCH_SCALE, WRITE_SCALE = 1.9999, 1.0

SQ_A = ("SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_VALU_TRANS_F32 SQ_INSTS_VALU_CVT SQ_INSTS_LDS SQ_INSTS_SALU SQ_BUSY_CYCLES "
        "SQ_ACTIVE_INST_VALU")
SQ_B = ("SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_ANY SQ_CYCLES SQ_WAVES "
        "SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE")
CONV_A = "SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_INSTS_VALU SQ_WAVE_CYCLES SQ_CYCLES SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_LDS"
DENSE_A = "SQ_INSTS_VALU SQ_INSTS_MFMA SQ_INSTS_VALU_TRANS_F32 SQ_INSTS_VALU_CVT SQ_ACTIVE_INST_VALU SQ_VALU_MFMA_BUSY_CYCLES SQ_WAVE_CYCLES SQ_CYCLES"
DENSE_B = "SQ_WAIT_INST_ANY SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT SQ_INSTS_LDS SQ_BUSY_CYCLES"
CONV_CASES = ("level0", "level1", "level2", "level3", "level4", "config3")
DENSE_CASES = ("tail64", "tail32", "head64", "mlp128", "mlp256", "linear_ln256", "tail128", "tail256", "head128")
DENSE_KERNEL = {"tail64": "block_tail_kernel", "tail32": "block_tail_kernel", "head64": "block_head_kernel",
                "mlp128": "mlp_wide_kernel", "mlp256": "mlp_wide_kernel", "linear_ln256": "linear_wide_resident_kernel",
                "tail128": "mlp_wide_kernel", "tail256": "mlp_wide_kernel", "head128": "mlp_wide_kernel"}


def recipe(d):
    """The measurement batch as shell lines writing into directory d."""
    prof = "rocprofv3 --output-format csv"
    lines = [
        f"python3 bench.py > {d}/bench.json",
        f"{prof} --kernel-trace --stats -d {d}/prof_csv -o fwd -- python3 bench.py --no-cpu --no-other-configs --steps 20 --warmup 5 > {d}/prof_bench.json",
        f"{prof} --pmc FETCH_SIZE -d {d}/pmc_fetch -o f -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --copy-calibration > {d}/pmc_fetch.json",
        f"{prof} --pmc WRITE_SIZE -d {d}/pmc_write -o w -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --copy-calibration > {d}/pmc_write.json",
        f"python3 bench.py --attention-config2 20 > {d}/attn_cfg2.json",
        f"{prof} --pmc {SQ_A} -d {d}/pmc_attn -o a -- python3 bench.py --attention-config2 3",
        f"{prof} --pmc {SQ_B} -d {d}/pmc_attn -o b -- python3 bench.py --attention-config2 3",
        f"python3 bench.py --no-cpu --no-other-configs --steps 5 --warmup 2 --kernels {d}/kernel_rooflines.json > {d}/kernels_bench.json",
        f"{prof} --kernel-trace -d {d}/kern_pmc -o t -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --kernels {d}/kr_t.json",
        f"{prof} --pmc FETCH_SIZE TCC_HIT_sum -d {d}/kern_pmc -o f -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --kernels {d}/kr_f.json",
        f"{prof} --pmc WRITE_SIZE TCC_REQ_sum TCC_MISS_sum -d {d}/kern_pmc -o w -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --kernels {d}/kr_w.json",
        f"python3 bench.py --train bfloat16 --steps 8 --warmup 3 > {d}/train_bench.json",
        f"python3 bench.py --train float16 --steps 8 --warmup 3 > {d}/train_bench_f16.json",
        f"{prof} --kernel-trace --stats -d {d}/train_prof -o tr -- python3 bench.py --train bfloat16 --steps 8 --warmup 3 > {d}/train_prof_bench.json",
    ]
    for c in CONV_CASES:
        lines += [
            f"python3 bench.py --conv {c} --reps 20 > {d}/conv_{c}.json",
            f"{prof} --kernel-trace --stats -d {d}/conv_{c} -o t -- python3 bench.py --conv {c} --reps 5",
            f"{prof} --pmc {CONV_A} -d {d}/conv_{c} -o a -- python3 bench.py --conv {c} --reps 3",
            f"{prof} --pmc FETCH_SIZE TCC_HIT_sum -d {d}/conv_{c} -o f -- python3 bench.py --conv {c} --reps 3",
            f"{prof} --pmc WRITE_SIZE TCC_MISS_sum TCC_REQ_sum -d {d}/conv_{c} -o w -- python3 bench.py --conv {c} --reps 3",
        ]
    for c in DENSE_CASES:
        lines += [
            f"python3 bench.py --dense {c} --reps 20 > {d}/dense_{c}.json",
            f"{prof} --pmc {DENSE_A} -d {d}/dense_{c} -o a -- python3 bench.py --dense {c} --reps 3",
            f"{prof} --pmc {DENSE_B} -d {d}/dense_{c} -o b -- python3 bench.py --dense {c} --reps 3",
        ]
    lines += [f"python3 bench.py --micro issue > {d}/micro_issue.txt", f"python3 bench.py --micro loads > {d}/micro_loads.txt"]
    return lines


# ---------------------------------------------------------------------------------------------------- helpers
def _last_json(path):
    return json.loads(open(path).read().strip().splitlines()[-1])


def _find(d, pattern):
    """The one file under d (any depth: rocprofv3 adds a host/pid level to some outputs) that matches pattern."""
    hits = sorted(glob.glob(os.path.join(d, "**", pattern), recursive=True))
    return hits[0] if hits else None


def _counters(path):
    agg = collections.defaultdict(list)
    for r in csv.DictReader(open(path)):
        agg[(r["Kernel_Name"], r["Counter_Name"])].append(float(r["Counter_Value"]))
    return agg


def _pick(agg, key, counter):
    return [v for (k, c), vs in agg.items() if key in k and c == counter for v in vs]


def _avg(v):
    return sum(v) / len(v) if v else float("nan")


def _short(name):
    name = re.sub(r"\(anonymous namespace\)::", "", name)
    name = re.sub(r"^void ", "", name)
    m = re.match(r"_ZN12_GLOBAL__N_1\d+([a-z_0-9]+kernel)", name)
    return m.group(1) if m else name.split("(")[0][:60]


def _template_args(name):
    """kernel<type, integer arguments> of a kernel in this library's anonymous namespace (Itanium mangling)."""
    m = re.search(r"_ZN12_GLOBAL__N_1(\d+)", name)
    if not m:
        return _short(name)
    kernel = name[m.end():m.end() + int(m.group(1))]
    t = re.match(r"I(DF16_|DF16b|f)?((?:L[ib]\d+E)*)", name[m.end() + int(m.group(1)):])
    if not t or not (t.group(1) or t.group(2)):
        return kernel
    args = ([{"DF16_": "f16", "DF16b": "bf16", "f": "f32"}[t.group(1)]] if t.group(1) else []) + [a[2:] for a in re.findall(r"L[ib]\d+", t.group(2))]
    return kernel + "<" + ", ".join(args) + ">"


def _grouped(rows, groups, per):
    acc = collections.OrderedDict((k, [0.0, 0.0]) for k in groups)
    other = [0.0, 0.0]
    for name, total_ns, calls in rows:
        t, c = total_ns / per / 1e3, calls / per
        for g, keys in groups.items():
            if any(k in name for k in keys):
                acc[g][0] += t
                acc[g][1] += c
                break
        else:
            other[0] += t
            other[1] += c
    out = ["  %8.1f us %6.1f launches  %s" % (t, c, g) for g, (t, c) in sorted(acc.items(), key=lambda x: -x[1][0])]
    out.append("  %8.1f us %6.1f launches  other" % tuple(other))
    return out


FORWARD_GROUPS = collections.OrderedDict([
    ("patch attention", ["patch_attn"]),
    ("sparse conv (sparse tile and tile forms, pair kernels, segment sum)",
     ["pair_gemm", "pair_wstat", "pair_segment", "subm_conv", "conv_tile", "conv_sparse"]),
    ("Linear kernels (linear_rows with GELU / BatchNorm epilogues, linear_wide, linear_ln, linear_any)",
     ["linear_rows", "linear_ln", "linear_wide", "linear_gemm", "linear_any"]),
    ("voxel hash + pair lists", ["plan_", "direct_", "vh_", "kmap", "pack_weight", "inner_"]),
    ("fused block head/tail, fused MLP", ["block_", "mlp_"]),
    ("LayerNorm / BatchNorm kernels", ["layer_norm", "bn_act"]),
    ("torch elementwise / index / cat", ["at::native", "at::cuda"]),
    ("copies (D2D residual copies, D2H counts)", ["copyBuffer", "fillBuffer"]),
    ("serialization (encode, sort, pooled orders)",
     ["scatter_kernel", "digit_totals", "zero_words", "order_", "encode", "grid_max"]),
    ("pooling / unpooling", ["pool_", "segment_reduce", "unpool", "cluster_"]),
    ("attention index tables", ["attn_slots", "pad_index", "pad_prefix"]),
    ("offset2batch", ["offset2batch"]),
])

TRAIN_GROUPS = collections.OrderedDict([
    ("attention backward (attn_bwd_q / attn_bwd_kv / fill)", ["attn_bwd"]),
    ("attention forward (keeps log-sum-exp rows)", ["patch_attn"]),
    ("weight gradients: conv (gather) and Linear (outer_rows, slab_sum)", ["outer_rows", "slab_sum", "conv_wgrad"]),
    ("sparse conv forward and input gradient (sparse tile and tile forms, pair kernels, segment sum)",
     ["pair_gemm", "pair_wstat", "pair_segment", "subm_conv", "conv_tile", "conv_sparse", "pack_weight"]),
    ("LayerNorm + residual add, forward and backward", ["add_layer_norm", "layer_norm", "scaled_add"]),
    ("parameter casts and transposes (cast_params)", ["cast_params"]),
    ("Linear forward / input gradient on the row kernels (with the MLP's GELU)", ["linear_rows", "linear_wide", "linear_any"]),
    ("library GEMMs", ["Cijk"]),
    ("BatchNorm (+ GELU) training kernels", ["bn_stats", "bn_finalize", "bn_bwd", "bn_act", "batch_norm", "zero_kernel"]),
    ("torch elementwise, reductions, optimizer", ["at::native", "at::cuda"]),
    ("voxel hash + pair lists + neighbour maps", ["plan_", "direct_", "vh_", "kmap", "inner_"]),
    ("pooling / unpooling and their backward", ["pool_", "segment_reduce", "unpool", "cluster_"]),
    ("copies / fills", ["copyBuffer", "fillBuffer"]),
    ("serialization (encode, sort, pooled orders)",
     ["scatter_kernel", "digit_totals", "zero_words", "order_", "encode", "grid_max"]),
])


# --------------------------------------------------------------------------------------------------- sections
def forward_trace(d, out_dir):
    """profiles/forward_4x100k_fp16_kernel_trace.txt"""
    trace_path = _find(os.path.join(d, "prof_csv"), "*kernel_trace.csv")
    need = [os.path.join(d, "bench.json"), os.path.join(d, "prof_bench.json")]
    if trace_path is None or not all(os.path.exists(p) for p in need):
        return "forward trace: needs bench.json, prof_bench.json and prof_csv/ (recipe lines 1-2)"
    bench, pbench = _last_json(need[0]), _last_json(need[1])
    steps = pbench["steps"]
    # per-kernel statistics over the timed forwards only: a forward starts at its offset2batch kernel; what bench.py
    # launches around the forwards (set-up, flop accounting) is left out
    trace = list(csv.DictReader(open(trace_path)))
    trace.sort(key=lambda r: int(r["Start_Timestamp"]))
    marks = [i for i, r in enumerate(trace) if "offset2batch" in r["Kernel_Name"]]
    overlapped = pbench["config"].get("plain_schedule_ms_per_step") is not None
    # bench.py's loops, in order: warm-up, the `steps` timed forwards, then (when the timed ones overlapped their index
    # prologues) 2 + steps forwards on the plain schedule, then 2 + steps with events around every launch. With a
    # prologue running beside the forward before it, `steps` marks apart is still `steps` forwards' worth of kernels.
    tail = steps + 2
    plain = trace[marks[-2 * tail + 2]:marks[-tail]] if overlapped else None
    t_first = -(2 * tail + steps) if overlapped else -(tail + steps)
    window = trace[marks[t_first]:marks[t_first + steps]]
    agg = collections.OrderedDict()
    for r in window:
        dur = int(r["End_Timestamp"]) - int(r["Start_Timestamp"])
        a = agg.setdefault(r["Kernel_Name"], [0, 0, 1 << 62, 0])
        a[0] += 1
        a[1] += dur
        a[2] = min(a[2], dur)
        a[3] = max(a[3], dur)
    rows = sorted(agg.items(), key=lambda kv: -kv[1][1])
    tot = sum(v[1] for _, v in rows)
    # from the first timed forward's first kernel to the last one's, over the forwards in between
    span = (int(trace[marks[t_first + steps - 1]]["Start_Timestamp"]) - int(window[0]["Start_Timestamp"])) / (steps - 1) / 1e3
    rf, brf = pbench["roofline"], bench["roofline"]
    out = [
        "rocprofv3 kernel-trace summary: full PTv3 forward, 4 room scenes (%d points), fp16, MI355X\n" % POINTS,
        "command (run from the repository root on the GPU box):",
        "  rocprofv3 --kernel-trace --stats --output-format csv -d DIR/prof_csv -o fwd -- python3 bench.py --no-cpu --no-other-configs --steps %d --warmup %d"
        % (steps, pbench["warmup"]),
        "source: the kernel trace of that run, the %d timed forwards (a forward = from one offset2batch kernel to the next%s); times in microseconds\n"
        % (steps, "; the index prologue of a forward runs on its own stream beside the forward before, so the window is cut "
                  "at the prologues and holds every kernel of a forward once" if overlapped else ""),
        "bench.py line of the same run: ms_per_step=%.2f  points/s=%.0f" % (pbench["ms_per_step"], pbench["value"]),
        "  roofline (HIP events inside bench.py): kernel=%s launches=%d avg_launch_us=%.1f flops_per_launch=%.3e achieved=%.1f TFLOP/s frac=%.4f"
        % (rf["kernel"], rf["launches"], rf["avg_launch_us"], rf["flops_per_launch"], rf["achieved"], rf["frac"]),
        "bench.py line without the profiler (`python3 bench.py`, same box, same build): ms_per_step=%.2f  points/s=%.0f  attention avg_launch_us=%.1f achieved=%.1f TFLOP/s frac=%.4f\n"
        % (bench["ms_per_step"], bench["value"], brf["avg_launch_us"], brf["achieved"], brf["frac"]),
        "%6s %10s %9s %8s %9s %6s  kernel" % ("calls", "total_us", "avg_us", "min_us", "max_us", "%"),
    ]
    for name, (calls, total, mn, mx) in rows[:48]:
        out.append("%6d %10.1f %9.1f %8.1f %9.1f %6.2f  %s" % (calls, total / 1e3, total / calls / 1e3, mn / 1e3, mx / 1e3,
                                                               100 * total / tot, name[:110]))
    out.append("\nall kernels: %.1f us of GPU time per forward, %d launches per forward; %.1f us from forward to forward under the profiler"
               % (tot / steps / 1e3, sum(v[0] for _, v in rows) / steps, span))
    out.append("\nper forward, by group:")
    out += _grouped([(n, v[1], v[0]) for n, v in rows], FORWARD_GROUPS, steps)
    if overlapped:
        ptot = sum(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]) for r in plain)
        pspan = (int(trace[marks[-tail - 1]]["Start_Timestamp"]) - int(plain[0]["Start_Timestamp"])) / (steps - 1) / 1e3
        out.append("\nthe plain schedule (every forward's index work in front of its own feature kernels), the %d forwards bench.py "
                   "times after the timed region: %.1f us of kernels per forward, %.1f us from forward to forward under the profiler; "
                   "bench.py's own clock: %.2f ms per forward with the profiler, %.2f ms without"
                   % (steps, ptot / steps / 1e3, pspan, pbench["config"]["plain_schedule_ms_per_step"],
                      bench["config"]["plain_schedule_ms_per_step"] or float("nan")))
    open(os.path.join(out_dir, "forward_4x100k_fp16_kernel_trace.txt"), "w").write("\n".join(out) + "\n")
    return "forward trace: %.1f us of kernels per forward, ms_per_step %.2f" % (tot / steps / 1e3, bench["ms_per_step"])


def attention_traffic(d, out_dir):
    """profiles/attention_hbm_traffic_pmc.txt and attention_traffic.json (the latter is what bench.py reads for
    roofline.traffic)."""
    global FETCH_SCALE, WRITE_SCALE
    fp, wp = _find(os.path.join(d, "pmc_fetch"), "*counter_collection.csv"), _find(os.path.join(d, "pmc_write"), "*counter_collection.csv")
    if fp is None or wp is None:
        return "attention traffic: needs pmc_fetch/ and pmc_write/ (recipe lines 3-4)"
    f, w = _counters(fp), _counters(wp)
    gib_kib = 1 << 20
    copy_f, copy_w = max(_pick(f, "copyBuffer", "FETCH_SIZE")), max(_pick(w, "copyBuffer", "WRITE_SIZE"))
    FETCH_SCALE, WRITE_SCALE = gib_kib / copy_f, gib_kib / copy_w
    af, aw = _pick(f, "patch_attn_half", "FETCH_SIZE"), _pick(w, "patch_attn_half", "WRITE_SIZE")
    fetch_b, write_b = _avg(af) * FETCH_SCALE * 1024, _avg(aw) * WRITE_SCALE * 1024
    alg = 115.5e6
    txt = [
        "rocprofv3 --pmc summary: HBM traffic of the patch attention kernel inside the full PTv3 forward",
        "(4 room scenes, %d points, fp16, MI355X)\n" % POINTS,
        "commands (run from the repository root on the GPU box, one counter per run):",
        "  rocprofv3 --pmc FETCH_SIZE --output-format csv -d DIR/pmc_fetch -o f -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --copy-calibration",
        "  rocprofv3 --pmc WRITE_SIZE --output-format csv -d DIR/pmc_write -o w -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --copy-calibration\n",
        "calibration (--copy-calibration: one 1 GiB device-to-device copy, kernel __amd_rocclr_copyBuffer):",
        "  FETCH_SIZE reads %.1f for 1,048,576 KiB read   -> scale %.4f" % (copy_f, FETCH_SCALE),
        "  WRITE_SIZE reads %.1f for 1,048,576 KiB written -> scale %.4f\n" % (copy_w, WRITE_SCALE),
        "patch_attn_half_kernel<f16>, %d dispatches (3 forwards x 22 launches of different sizes), per launch on average:" % len(af),
        "  FETCH_SIZE %.1f -> %.1f MB read" % (_avg(af), fetch_b / 1e6),
        "  WRITE_SIZE %.1f -> %.1f MB written" % (_avg(aw), write_b / 1e6),
        "  total %.1f MB per launch" % ((fetch_b + write_b) / 1e6),
        "algorithmic minimum (qkv rows read once, output rows written once: 8*C bytes per point, averaged over the 22",
        "launches of a forward): %.1f MB per launch -> measured / algorithmic = %.2f" % (alg / 1e6, (fetch_b + write_b) / alg),
        "the (sequence, head) items of the last, partly filled round of resident work-groups are cut into up to four",
        "query ranges, one work-group each, and every range stages the keys and values of its sequence; the ranges of",
        "an item, and the heads of a sequence (which read neighbouring 32-byte pieces of the same lines), are placed on",
        "one XCD one after the other, so those repeats are served by that XCD's L2 (with the ranges spread over the",
        "XCDs the same run read 171 MB and the ratio was 1.74).",
    ]
    open(os.path.join(out_dir, "attention_hbm_traffic_pmc.txt"), "w").write("\n".join(txt) + "\n")
    json.dump({"kernel": "patch_attn_half_kernel<f16>", "workload_points": POINTS, "dispatches": len(af),
               "fetch_size_kib_avg": _avg(af), "write_size_kib_avg": _avg(aw), "fetch_scale": FETCH_SCALE,
               "write_scale": WRITE_SCALE, "traffic_bytes_per_launch": fetch_b + write_b},
              open(os.path.join(out_dir, "attention_traffic.json"), "w"), indent=1)
    return "attention traffic: %.1f MB per launch, %.2f x algorithmic" % ((fetch_b + write_b) / 1e6, (fetch_b + write_b) / alg)


def attention_counters(d, out_dir):
    """profiles/attention_config2_sq_counters.txt"""
    paths = glob.glob(os.path.join(d, "pmc_attn", "**", "*counter_collection.csv"), recursive=True)
    cfg_path = os.path.join(d, "attn_cfg2.json")
    if not paths or not os.path.exists(cfg_path):
        return "attention counters: needs attn_cfg2.json and pmc_attn/ (recipe lines 5-7)"
    cfg2, c = _last_json(cfg_path), {}
    for path in paths:                      # the counter sets of the separate runs, merged
        agg = _counters(path)
        for k in (SQ_A + " " + SQ_B).split():
            v = _pick(agg, "patch_attn_half", k)
            if v:
                c[k] = _avg(v)
    missing = [k for k in (SQ_A + " " + SQ_B).split() if k not in c]
    if missing:
        return "attention counters: pmc_attn/ lacks " + " ".join(missing) + " (recipe lines 6-7)"
    seqs, heads = cfg2["sequences"], cfg2["heads"]
    iters = cfg2["flops"] / (4.0 * 64 * 32 * 16)   # 64-key x 32-query steps of one wave: 4*64*32*16 flops each
    cyc = c["SQ_CYCLES"] / 32.0
    valu_busy = c["SQ_ACTIVE_INST_VALU"] * 4
    trans, valu = c["SQ_INSTS_VALU_TRANS_F32"], c["SQ_INSTS_VALU"]
    t = [
        "rocprofv3 --pmc summary: instruction mix and issue utilisation of the patch attention kernel at baseline",
        "config 2 (one room scene, %d points, Hilbert order, patch 1024, C=512, 32 heads, fp16), MI355X\n" % cfg2["points"],
        "commands (run from the repository root on the GPU box):",
        "  python3 bench.py --attention-config2 20",
        "  rocprofv3 --pmc %s --output-format csv -d DIR/pmc_attn -o a -- python3 bench.py --attention-config2 3" % SQ_A,
        "  rocprofv3 --pmc %s --output-format csv -d DIR/pmc_attn -o b -- python3 bench.py --attention-config2 3\n" % SQ_B,
        "without the profiler: %.1f us per launch, %.1f TFLOP/s = %.1f %% of the 2.5 PFLOP/s dense fp16 peak"
        % (cfg2["us"], cfg2["tflops"], 100 * cfg2["frac_mfma_peak"]),
        "work: %d sequences x %d heads = %d work-groups of 8 waves; %.4g wave steps (64 keys x 32 queries: 2 QK^T + 4 PV MFMAs, 2048 scores)\n"
        % (seqs, heads, seqs * heads, iters),
        "counter averages per dispatch (summed over the chip):",
    ]
    t += ["  %-28s %.5g" % (k, v) for k, v in c.items()]
    t += [
        "\nderived:",
        "  kernel length: SQ_CYCLES / 32 shader engines = %.0f cycles; at %.1f us that is a shader clock of %.2f GHz" % (cyc, cfg2["us"], cyc / cfg2["us"] / 1e3),
        "  per wave step: %.1f VALU instructions, of them %.1f v_exp_f32, %.1f conversions, %.1f MFMA; %.1f LDS, %.1f scalar"
        % (valu / iters, trans / iters, c["SQ_INSTS_VALU_CVT"] / iters, c["SQ_INSTS_MFMA"] / iters, c["SQ_INSTS_LDS"] / iters, c["SQ_INSTS_SALU"] / iters),
        "  VALU issue time: SQ_ACTIVE_INST_VALU x 4 = %.4g cycles = %.1f cycles per VALU instruction on average" % (valu_busy, valu_busy / valu),
        "  (8 cycles per v_exp_f32, 4 per other instruction: (%.1f x 8 + %.1f x 4) / %.1f = %.2f)"
        % (trans / iters, (valu - trans) / iters, valu / iters, (trans * 8 + (valu - trans) * 4) / valu),
        "  VALU issue utilisation: %.4g / (1024 SIMDs x %.0f cycles) = %.1f %%" % (valu_busy, cyc, 100 * valu_busy / (1024 * cyc)),
        "  wave occupancy: SQ_WAVE_CYCLES x 4 / (4096 wave slots x %.0f cycles) = %.1f %%" % (cyc, 100 * c["SQ_WAVE_CYCLES"] * 4 / (4096 * cyc)),
        "  useful MFMA cycles per wave step: 4 x 32 (QK^T 2 x 32, PV 4 x 32 of which half the rows are padding) against %.0f VALU cycles" % (valu_busy / iters),
    ]
    open(os.path.join(out_dir, "attention_config2_sq_counters.txt"), "w").write("\n".join(t) + "\n")
    return "attention counters: VALU issue %.1f %%, clock %.2f GHz" % (100 * valu_busy / (1024 * cyc), cyc / cfg2["us"] / 1e3)


def kernel_rooflines(d, out_dir):
    """profiles/kernel_rooflines.txt"""
    path = os.path.join(d, "kernel_rooflines.json")
    if not os.path.exists(path):
        return "kernel rooflines: needs kernel_rooflines.json (recipe line 8)"
    rows = json.load(open(path))
    k = [
        "per-kernel measurements at the sizes of the baseline configurations (and at 16x the points for the index kernels), MI355X\n",
        "command (run from the repository root on the GPU box):",
        "  python3 bench.py --no-cpu --no-other-configs --steps 5 --warmup 2 --kernels DIR/kernel_rooflines.json",
        "each kernel is called alone 20 times back to back through the Python wrapper and timed with HIP events, so",
        "the figure includes output allocation, launch overhead and, where the wrapper reads a count back, that",
        "synchronisation: kernels that run for a few microseconds are overhead-bound here; their own durations are",
        "in the rocprofv3 trace summary.\n",
        "%-28s %9s %10s %-8s %7s  workload / algorithmic work" % ("kernel", "us", "achieved", "unit", "% peak"),
    ]
    for r in rows:
        k.append("%-28s %9.1f %10.1f %-8s %6.1f%%  %s; %.4g %s" % (r["kernel"], r["us"], r["achieved"], r["unit"], 100 * r["frac"],
                                                                  r["workload"], r["work"], r["work_unit"]))
    open(os.path.join(out_dir, "kernel_rooflines.txt"), "w").write("\n".join(k) + "\n")
    return "kernel rooflines: %d rows" % len(rows)


def index_kernel_counters(d, out_dir):
    """profiles/index_kernels_hbm_counters.txt: per kernel and launch size, duration, HBM bytes and L2 requests of
    the serialization, sort, voxel-hash / pair-list, pooling and voxelisation kernels of a --kernels run."""
    base = os.path.join(d, "kern_pmc")
    tp, fp, wp = _find(base, "t_kernel_trace.csv"), _find(base, "f_counter_collection.csv"), _find(base, "w_counter_collection.csv")
    if tp is None or fp is None or wp is None:
        return "index kernel counters: needs kern_pmc/ (recipe lines 9-11)"
    want = ("encode_kernel", "decode_kernel", "digit_totals_kernel", "scatter_kernel", "zero_words_kernel", "vh_insert_kernel",
            "vh_fill_kernel", "direct_count_kernel", "direct_fill_kernel", "plan_scan_kernel", "kmap_kernel", "kmap_build",
            "order_count_kernel", "order_assign_kernel", "pool_gather_kernel", "segment_reduce_kernel", "pool_", "voxel", "scene_min",
            "pad_index", "attn_slots", "plan_", "cluster_", "unpool")

    def load(path):
        rows = collections.defaultdict(lambda: collections.defaultdict(list))
        for r in csv.DictReader(open(path)):
            if any(x in r["Kernel_Name"] for x in want):
                rows[(_template_args(r["Kernel_Name"]), int(r["Grid_Size"]))][r["Counter_Name"]].append(float(r["Counter_Value"]))
        return rows
    f, w = load(fp), load(wp)
    dur = collections.defaultdict(list)
    for r in csv.DictReader(open(tp)):
        if any(x in r["Kernel_Name"] for x in want):
            grid = int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
            dur[(_template_args(r["Kernel_Name"]), grid)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    out = [
        "rocprofv3 summary: HBM traffic and L2 requests of the serialization, radix sort, voxel-hash / pair-list, pooling and",
        "voxelisation kernels at the sizes bench.py --kernels runs them (4 room scenes of %d points; the same 16 times over;" % POINTS,
        "baseline config 3's 200,000 voxels; the levels of the benchmark batch), MI355X\n",
        "commands (run from the repository root on the GPU box; each counter set in a run of its own):",
        "  rocprofv3 --kernel-trace --output-format csv -d DIR/kern_pmc -o t -- python3 bench.py --no-cpu --no-other-configs --steps 2 --warmup 1 --kernels DIR/kr_t.json",
        "  rocprofv3 --pmc FETCH_SIZE TCC_HIT_sum --output-format csv -d DIR/kern_pmc -o f -- (the same bench.py line)",
        "  rocprofv3 --pmc WRITE_SIZE TCC_REQ_sum TCC_MISS_sum --output-format csv -d DIR/kern_pmc -o w -- (the same bench.py line)\n",
        "Per kernel and launch size (grid = threads launched): n launches in the run, median duration under the kernel trace,",
        "FETCH_SIZE x %.4f KiB read and WRITE_SIZE x %.4f KiB written (the factors a 1 GiB device-to-device copy gives)," % (FETCH_SCALE, WRITE_SCALE),
        "their sum over the duration, and the L2's requests, hits and misses. Launches shorter than 8 us are left out",
        "(launch and ramp-up set their time, not traffic).\n",
    ]
    for key in sorted(dur, key=lambda k: (k[0], -k[1])):
        if len(dur[key]) < 3:
            continue
        us = sorted(dur[key])[len(dur[key]) // 2]
        if us < 8:
            continue
        fb = _avg(f.get(key, {}).get("FETCH_SIZE", [])) * 1024 * FETCH_SCALE
        wb = _avg(w.get(key, {}).get("WRITE_SIZE", [])) * 1024 * WRITE_SCALE
        hit, req, miss = (_avg(f.get(key, {}).get("TCC_HIT_sum", [])), _avg(w.get(key, {}).get("TCC_REQ_sum", [])),
                          _avg(w.get(key, {}).get("TCC_MISS_sum", [])))
        out.append(f"{key[0]:44s} grid {key[1]:>10d} n={len(dur[key]):3d} {us:8.1f} us  read {fb / 1e6:8.1f} MB  written {wb / 1e6:8.1f} MB  "
                   f"{(fb + wb) / us / 1e6:5.2f} TB/s  L2 req {req:.3g} hit {hit:.3g} miss {miss:.3g}")
    open(os.path.join(out_dir, "index_kernels_hbm_counters.txt"), "w").write("\n".join(out) + "\n")
    return "index kernel counters: %d rows" % (len(out) - 11)


def training_trace(d, out_dir):
    """profiles/training_step_4x100k_bf16_kernel_trace.txt"""
    stats = _find(os.path.join(d, "train_prof"), "*kernel_stats.csv")
    need = [os.path.join(d, n) for n in ("train_bench.json", "train_bench_f16.json", "train_prof_bench.json")]
    if stats is None or not all(os.path.exists(p) for p in need):
        return "training trace: needs train_bench.json, train_bench_f16.json, train_prof_bench.json and train_prof/ (recipe lines 12-14)"
    tb, tb16, tp = (_last_json(p) for p in need)
    rows = list(csv.DictReader(open(stats)))
    nstep = tp["steps"] + tp["warmup"]
    tot = sum(float(r["TotalDurationNs"]) for r in rows)
    o = [
        "rocprofv3 kernel-trace summary: PTv3 training step (forward + backward + AdamW), default model in training mode,",
        "4 room scenes (%d points), bf16 autocast, MI355X\n" % POINTS,
        "command (run from the repository root on the GPU box):",
        "  rocprofv3 --kernel-trace --stats --output-format csv -d DIR/train_prof -o tr -- python3 bench.py --train bfloat16 --steps %d --warmup %d" % (tp["steps"], tp["warmup"]),
        "source: the kernel statistics of that run; all %d steps of the process (%d warm-up + %d timed), figures divided by %d; times in microseconds\n"
        % (nstep, tp["warmup"], tp["steps"], nstep),
        "bench.py --train line of the same run: ms_per_step=%.2f  points/s=%.0f" % (tp["ms_per_step"], tp["value"]),
        "without the profiler (same box, same build): bf16 ms_per_step=%.2f  points/s=%.0f  peak memory %.1f GiB;  f16 ms_per_step=%.2f\n"
        % (tb["ms_per_step"], tb["value"], tb["peak_memory_gib"], tb16["ms_per_step"]),
        "%8s %11s %9s %6s  kernel" % ("calls/st", "us/step", "avg_us", "%"),
    ]
    for r in rows[:50]:
        t = float(r["TotalDurationNs"])
        o.append("%8.1f %11.1f %9.1f %6.2f  %s" % (int(r["Calls"]) / nstep, t / nstep / 1e3, float(r["AverageNs"]) / 1e3, 100 * t / tot, r["Name"][:110]))
    o.append("\nall kernels: %.1f us of GPU time per step, %.0f launches per step" % (tot / nstep / 1e3, sum(int(r["Calls"]) for r in rows) / nstep))
    o.append("\nper step, by group:")
    o += _grouped([(r["Name"], float(r["TotalDurationNs"]), int(r["Calls"])) for r in rows], TRAIN_GROUPS, nstep)
    open(os.path.join(out_dir, "training_step_4x100k_bf16_kernel_trace.txt"), "w").write("\n".join(o) + "\n")
    return "training trace: bf16 %.2f ms per step, f16 %.2f" % (tb["ms_per_step"], tb16["ms_per_step"])


def conv_counters(d, out_dir):
    """profiles/conv_<workload>_counters.txt, one per workload whose raw files are there."""
    keep = ("conv_sparse", "conv_tile", "pair_wstat", "pair_gemm", "subm_conv_pairs", "pair_segment_sum")
    done = []
    for wl in CONV_CASES:
        base, line_path = os.path.join(d, f"conv_{wl}"), os.path.join(d, f"conv_{wl}.json")
        if not os.path.isdir(base) or not os.path.exists(line_path):
            continue
        line = _last_json(line_path)
        ctr = collections.defaultdict(lambda: collections.defaultdict(list))
        for path in glob.glob(os.path.join(base, "**", "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(path)):
                if any(x in r["Kernel_Name"] for x in keep):
                    ctr[_template_args(r["Kernel_Name"])][r["Counter_Name"]].append(float(r["Counter_Value"]))
        dur = collections.defaultdict(list)
        for path in glob.glob(os.path.join(base, "**", "*kernel_trace.csv"), recursive=True):
            for r in csv.DictReader(open(path)):
                if any(x in r["Kernel_Name"] for x in keep):
                    dur[_template_args(r["Kernel_Name"])].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
        out = [
            f"rocprofv3 summary: the 3x3x3 submanifold convolution of one level alone -- {line['workload']}, fp16, MI355X",
            f"{line['voxels']} voxels, {line['channels']} channels, {line['pairs']} active pairs ({line['pairs_per_voxel']:.2f} per voxel), form: {line['form']}",
            "",
            "commands (run from the repository root on the GPU box; each counter set in a run of its own):",
            f"  python3 bench.py --conv {wl} --reps 20",
            f"  rocprofv3 --kernel-trace --stats --output-format csv -d DIR/conv_{wl} -o t -- python3 bench.py --conv {wl} --reps 5",
            f"  rocprofv3 --pmc {CONV_A} --output-format csv -d DIR/conv_{wl} -o a -- python3 bench.py --conv {wl} --reps 3",
            f"  rocprofv3 --pmc FETCH_SIZE TCC_HIT_sum --output-format csv -d DIR/conv_{wl} -o f -- python3 bench.py --conv {wl} --reps 3",
            f"  rocprofv3 --pmc WRITE_SIZE TCC_MISS_sum TCC_REQ_sum --output-format csv -d DIR/conv_{wl} -o w -- python3 bench.py --conv {wl} --reps 3",
            "",
            f"without the profiler (HIP events, 20 calls): {line['us']:.1f} us per convolution = {line['tflops']:.1f} TFLOP/s of useful work "
            f"(2 * pairs * Cin * Cout = {line['flops']:.3e} FLOP) = {100 * line['frac_mfma_peak']:.1f} % of the 2.5 PFLOP/s dense fp16 peak;",
            f"algorithmic bytes (rows in and out once, weights once, 4 B per pair) {line['min_bytes'] / 1e6:.1f} MB -> {line['gbs']:.0f} GB/s = "
            f"{100 * line['frac_hbm_peak']:.1f} % of 8 TB/s",
            "",
            "FETCH_SIZE / WRITE_SIZE are in KiB; scaled by what the same counters read for a 1 GiB device-to-device copy",
            f"(FETCH_SIZE x {FETCH_SCALE:.4f}, WRITE_SIZE x {WRITE_SCALE:.4f})",
        ]
        for k in sorted(dur, key=lambda k: -sum(dur[k])):
            c = ctr.get(k, {})
            avg = lambda n: _avg(c.get(n, []))
            us = _avg(dur[k])
            cyc = avg("SQ_CYCLES") / 32
            out += ["", f"{k}: {us:.1f} us per launch under the trace ({len(dur[k])} launches)",
                    f"  kernel length SQ_CYCLES / 32 = {cyc:.0f} cycles; SQ_INSTS_MFMA {avg('SQ_INSTS_MFMA'):.4g}, SQ_INSTS_VALU {avg('SQ_INSTS_VALU'):.4g}"]
            if avg("SQ_INSTS_MFMA") > 0:
                out.append(f"  MFMA pipe busy: SQ_VALU_MFMA_BUSY_CYCLES {avg('SQ_VALU_MFMA_BUSY_CYCLES'):.4g} / (1024 SIMDs x {cyc:.0f}) = "
                           f"{100 * avg('SQ_VALU_MFMA_BUSY_CYCLES') / (1024 * cyc):.1f} %")
            fb, wb = avg("FETCH_SIZE") * 1024 * FETCH_SCALE, avg("WRITE_SIZE") * 1024 * WRITE_SCALE
            out += [
                f"  waves resident: SQ_WAVE_CYCLES x 4 / (256 CUs x {cyc:.0f}) = {avg('SQ_WAVE_CYCLES') * 4 / (256 * cyc):.1f} per CU",
                f"  LDS: SQ_ACTIVE_INST_LDS x 4 / (256 CUs x {cyc:.0f}) = {100 * avg('SQ_ACTIVE_INST_LDS') * 4 / (256 * cyc):.1f} % of the kernel; "
                f"SQ_LDS_BANK_CONFLICT {avg('SQ_LDS_BANK_CONFLICT'):.4g} cycles",
                f"  HBM: FETCH_SIZE {avg('FETCH_SIZE'):.1f} -> {fb / 1e6:.1f} MB read, WRITE_SIZE {avg('WRITE_SIZE'):.1f} -> {wb / 1e6:.1f} MB written "
                f"({(fb + wb) / 1e6:.1f} MB, {(fb + wb) / us / 1e6:.2f} TB/s at the traced duration)",
                f"  L2: TCC_REQ_sum {avg('TCC_REQ_sum'):.4g} requests, TCC_HIT_sum {avg('TCC_HIT_sum'):.4g}, TCC_MISS_sum {avg('TCC_MISS_sum'):.4g} "
                f"(hit rate {100 * avg('TCC_HIT_sum') / max(avg('TCC_HIT_sum') + avg('TCC_MISS_sum'), 1):.0f} %)",
            ]
        name = {"config3": "conv_config3_200k_voxels_64ch_fp16_counters.txt"}.get(wl, f"conv_{wl}_4x100k_fp16_counters.txt")
        open(os.path.join(out_dir, name), "w").write("\n".join(out) + "\n")
        done.append(wl)
    return "conv counters: " + (", ".join(done) if done else "needs conv_<case>.json and conv_<case>/ (recipe: the --conv lines)")


def dense_counters(d, out_dir):
    """profiles/dense_block_kernels_sq_counters.txt"""
    cases = [c for c in DENSE_CASES if os.path.exists(os.path.join(d, f"dense_{c}.json")) and os.path.isdir(os.path.join(d, f"dense_{c}"))]
    if not cases:
        return "dense counters: needs dense_<case>.json and dense_<case>/ (recipe: the --dense lines)"
    out = [
        "rocprofv3 --pmc summary: the fused dense kernels of a transformer block, each alone at the rows and width of a level of the",
        "benchmark batch (4 room scenes, fp16), MI355X",
        "",
        "commands (run from the repository root on the GPU box; CASE = " + ", ".join(DENSE_CASES) + "; each counter set in a run of its own):",
        "  python3 bench.py --dense CASE --reps 20",
        f"  rocprofv3 --pmc {DENSE_A} --output-format csv -d DIR/dense_CASE -o a -- python3 bench.py --dense CASE --reps 3",
        f"  rocprofv3 --pmc {DENSE_B} --output-format csv -d DIR/dense_CASE -o b -- python3 bench.py --dense CASE --reps 3",
        "",
        "busy figures are fractions of the kernel's length (SQ_CYCLES / 32 shader engines): VALU issue = SQ_ACTIVE_INST_VALU x 4 / 1024 SIMDs,",
        "MFMA = SQ_VALU_MFMA_BUSY_CYCLES / 1024 SIMDs, LDS = SQ_ACTIVE_INST_LDS x 4 / 256 CUs; waves = SQ_WAVE_CYCLES x 4 / 256 CUs;",
        "waiting = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES",
        "",
    ]
    for c in cases:
        j = _last_json(os.path.join(d, f"dense_{c}.json"))
        agg = collections.defaultdict(list)
        for path in glob.glob(os.path.join(d, f"dense_{c}", "**", "*counter_collection.csv"), recursive=True):
            for r in csv.DictReader(open(path)):
                if DENSE_KERNEL[c] in r["Kernel_Name"]:
                    agg[r["Counter_Name"]].append(float(r["Counter_Value"]))
        a = {k: _avg(v) for k, v in agg.items()}
        cyc = a["SQ_CYCLES"] / 32
        out += [
            f"{c}: {DENSE_KERNEL[c]}, {j['rows']} rows x {j['channels']} channels: {j['us']:.1f} us without the profiler = {j['tflops']:.0f} TFLOP/s of useful work "
            f"({100 * j['frac_mfma_peak']:.1f} % of 2.5 PFLOP/s), rows in and out once {j['min_bytes'] / 1e6:.0f} MB -> {j['gbs'] / 1e3:.2f} TB/s "
            f"({100 * j['frac_hbm_peak']:.0f} % of 8 TB/s)",
            f"  kernel length {cyc:.0f} cycles; VALU issue {100 * a['SQ_ACTIVE_INST_VALU'] * 4 / 1024 / cyc:.0f} %, MFMA {100 * a['SQ_VALU_MFMA_BUSY_CYCLES'] / 1024 / cyc:.0f} %, "
            f"LDS {100 * a['SQ_ACTIVE_INST_LDS'] * 4 / 256 / cyc:.0f} %, waves per CU {a['SQ_WAVE_CYCLES'] * 4 / 256 / cyc:.1f}, "
            f"waiting {100 * a['SQ_WAIT_INST_ANY'] / a['SQ_WAVE_CYCLES']:.0f} %",
            f"  SQ_INSTS_VALU {a['SQ_INSTS_VALU']:.4g} (transcendental {a['SQ_INSTS_VALU_TRANS_F32']:.4g}, conversions {a['SQ_INSTS_VALU_CVT']:.4g}), "
            f"SQ_INSTS_MFMA {a['SQ_INSTS_MFMA']:.4g}, SQ_INSTS_LDS {a['SQ_INSTS_LDS']:.4g}, SQ_LDS_BANK_CONFLICT {a['SQ_LDS_BANK_CONFLICT']:.4g}",
        ]
        if j["gelu_evaluations"]:
            g = j["gelu_evaluations"] / 64.0
            out.append(f"  per GELU evaluation (64 to a wave instruction): {a['SQ_INSTS_VALU'] / g:.1f} VALU instructions in the whole kernel, "
                       f"{a['SQ_INSTS_VALU_TRANS_F32'] / g:.2f} of them transcendental")
        out.append("")
    open(os.path.join(out_dir, "dense_block_kernels_sq_counters.txt"), "w").write("\n".join(out))
    return "dense counters: " + ", ".join(cases)


def micro_reports(d, out_dir):
    """profiles/micro_issue.txt, micro_loads.txt: the microbenchmark reports as printed, under their commands."""
    done = []
    for which in ("issue", "loads"):
        path = os.path.join(d, f"micro_{which}.txt")
        if not os.path.exists(path):
            continue
        body = [l for l in open(path).read().splitlines() if "amdgpu.ids" not in l]
        head = [f"microbenchmark of the part (libptv3_micro.so, pointtransformerv3_amd/csrc/micro.hip), MI355X",
                f"command (run from the repository root on the GPU box): python3 bench.py --micro {which}", ""]
        open(os.path.join(out_dir, f"micro_{which}.txt"), "w").write("\n".join(head + body) + "\n")
        done.append(which)
    return "micro reports: " + (", ".join(done) if done else "needs micro_issue.txt / micro_loads.txt (recipe: the --micro lines)")


SECTIONS = (forward_trace, attention_traffic, attention_counters, kernel_rooflines, index_kernel_counters, training_trace,
            conv_counters, dense_counters, micro_reports)


def summarise(d, out_dir):
    os.makedirs(out_dir, exist_ok=True)
    for section in SECTIONS:
        print(section(d, out_dir))

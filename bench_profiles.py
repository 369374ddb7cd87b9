"""Collects the rocprofv3 evidence for the fused kernels and reduces it to the short summaries under profiles/.

    python bench_profiles.py collect      (on the MI355X; raw profiler output goes to RAW/prof_*)
    python bench_profiles.py summarize    (reads RAW/prof_*, writes profiles/*.txt)

Every profiler run is a child process of its own (`rocprofv3 ... -- python3 bench.py ...`), one counter set per run;
the commands are repeated at the top of each summary.  Summaries are named for the kernels and workload they cover.
"""
from __future__ import annotations

import collections
import csv
import json
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
RAW = os.path.join(ROOT, "gpurun_out")
OUT = os.path.join(ROOT, "profiles")

QUIET = "--no-cpu-baseline --no-parity --no-other-configs"
SQ_COUNTERS = ("GRBM_GUI_ACTIVE SQ_VALU_MFMA_BUSY_CYCLES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_INSTS_MFMA SQ_WAIT_ANY "
               "SQ_ACTIVE_INST_ANY SQ_INSTS_LDS")
# name -> (rocprofv3 arguments, bench.py arguments, seconds)
RUNS = {
    "trace_layer": ("--kernel-trace --stats", f"--steps 20 --warmup 5 {QUIET}", 300),
    "fetch_layer": ("--pmc FETCH_SIZE", f"--steps 3 --warmup 1 {QUIET} --no-kernel-timing --calibration-copy", 120),
    "write_layer": ("--pmc WRITE_SIZE", f"--steps 3 --warmup 1 {QUIET} --no-kernel-timing --calibration-copy", 120),
    "sq_layer": (f"--pmc {SQ_COUNTERS}", f"--steps 3 --warmup 1 {QUIET} --no-kernel-timing", 120),
    "sq_layer_fp16": (f"--pmc {SQ_COUNTERS}", "--workload layer_fp16 --steps 3 --warmup 1", 180),
    "sq_config4": (f"--pmc {SQ_COUNTERS}", "--workload config4 --steps 3 --warmup 1 --no-kernel-timing", 180),
    "sq_config5": (f"--pmc {SQ_COUNTERS}", "--workload config5 --steps 3 --warmup 1 --no-kernel-timing", 180),
    "trace_config4": ("--kernel-trace --stats", "--workload config4 --steps 10 --warmup 3", 240),
    "trace_config5": ("--kernel-trace --stats", "--workload config5 --steps 10 --warmup 3", 240),
    "trace_yardsticks": ("--kernel-trace --stats", "--yardsticks", 240),
}


def command(name):
    prof, bench, _ = RUNS[name]
    return f"rocprofv3 {prof} --output-format csv -d gpurun_out/prof_{name} -o p -- python3 bench.py {bench}"


def collect(names):
    for name in names:
        cmd = command(name)
        print("[collect]", cmd, flush=True)
        log = open(os.path.join(RAW, f"prof_{name}.log"), "w")
        err = open(os.path.join(RAW, f"prof_{name}.err"), "w")
        subprocess.run(["rm", "-rf", os.path.join(RAW, f"prof_{name}")], check=False)
        rc = subprocess.run(["timeout", "-s", "KILL", str(RUNS[name][2])] + cmd.split(), cwd=ROOT, stdout=log, stderr=err).returncode
        print("[collect] exit", rc, flush=True)
        if rc != 0:
            sys.exit(rc)  # nothing more is started on the GPU after a failed or killed step


# ---------------------------------------------------------------------------------------------------------------
def short(n):
    n = re.sub(r"\(anonymous namespace\)::", "", n)
    n = re.sub(r"^void ", "", n)
    m = re.match(r"_ZN12_GLOBAL__N_1\d+([a-z_0-9]+?)I", n)
    if m:
        n = m.group(1)
    return n.split("(")[0].split("<")[0][:44]


def find(name, suffix):
    base = os.path.join(RAW, f"prof_{name}")
    for d, _, files in os.walk(base):
        for f in files:
            if f.endswith(suffix):
                return os.path.join(d, f)
    raise FileNotFoundError(f"{base}: no *{suffix}")


def bench_line(name):
    for line in open(os.path.join(RAW, f"prof_{name}.log")):
        if line.startswith("{"):
            return json.loads(line)
    return {}


def wgs(r, key="Grid_Size"):
    g = int(r.get(key) or r.get("Grid_Size_X"))
    w = int(r.get("Workgroup_Size") or r.get("Workgroup_Size_X") or 256)
    return g // max(1, w)


def is_gemm(n):
    return "gptq_lora_fwd" in n or "gptq_lora_bwd_dx" in n


def trace_summary(name, title, steps, first_timed, out_file, launches_key):
    """Per-kernel time per step over the timed steps of a --kernel-trace run.  `launches_key`: (kernel, workgroups) of a
    launch that happens exactly once per step, used to cut the trace into steps."""
    trace = list(csv.DictReader(open(find(name, "kernel_trace.csv"))))
    trace.sort(key=lambda r: int(r["Start_Timestamp"]))
    bj = bench_line(name)
    idx = [i for i, r in enumerate(trace) if launches_key[0] in r["Kernel_Name"] and wgs(r, "Grid_Size_X") == launches_key[1]]
    seg = trace[idx[first_timed]:idx[first_timed + steps]]
    wall = (int(trace[idx[first_timed + steps]]["Start_Timestamp"]) - int(seg[0]["Start_Timestamp"])) / 1e6 / steps
    agg = collections.defaultdict(lambda: [0, 0.0])
    for r in seg:
        d = (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
        k = (short(r["Kernel_Name"]), wgs(r, "Grid_Size_X"))
        agg[k][0] += 1
        agg[k][1] += d
    busy = sum(v[1] for v in agg.values()) / steps / 1e3
    lines = [f"command: {command(name)}", "", title,
             f"line printed by this run: ms_per_step {bj.get('ms_per_step', float('nan')):.3f}, {bj.get('tflops', float('nan')):.1f} TFLOP/s = "
             f"{100 * bj.get('frac_bf16_mfma_peak', float('nan')):.1f} % of 2516.6",
             f"kernel trace over the {steps} timed steps: {wall:.3f} ms/step wall, {busy:.3f} ms/step of kernel time", "",
             f"{'kernel':44s} {'workgroups':>10s} {'launches/step':>13s} {'us/step':>9s} {'avg us':>9s}"]
    for k, v in sorted(agg.items(), key=lambda kv: -kv[1][1])[:20]:
        lines.append(f"{k[0]:44s} {k[1]:10d} {v[0] / steps:13.1f} {v[1] / steps:9.1f} {v[1] / v[0]:9.1f}")
    gemm = sum(v[1] for k, v in agg.items() if is_gemm(k[0])) / steps
    lines += ["", f"fused dequant-GEMM launches: {gemm:.1f} us/step; everything else (rank-r products, adapter gradients, packs, "
              f"permutes): {busy * 1e3 - gemm:.1f} us/step"]
    if "kernels" in bj:
        lines += ["", "the same launches as bench.py's events on the launch stream see them (a second pass of the same steps):"]
        for label, v in bj["kernels"].items():
            lines.append(f"  {label:50s} {v['ms'] * 1e3:8.1f} us   {v['tflops']:7.1f} TFLOP/s = {100 * v['tflops'] / 2516.6:4.1f} %")
    if "roofline" in bj:
        rl = bj["roofline"]
        lines += ["", f"roofline kernel of the bench line: {rl['kernel']}: {rl['avg_launch_ms'] * 1e3:.1f} us/launch (events), "
                  f"{rl['achieved']:.1f} TFLOP/s = {100 * rl['frac']:.1f} % of peak"]
    open(os.path.join(OUT, out_file), "w").write("\n".join(lines) + "\n")
    print("\n".join(lines), "\n")
    return agg


def counter_rows(name):
    return list(csv.DictReader(open(find(name, "counter_collection.csv"))))


def sq_table(name, note, labeller):
    """Per launch (in dispatch order, one step's worth: the median over the steps of the run): duration, shader clock,
    MFMA busy, VALU and LDS instructions per MFMA."""
    rows = [r for r in counter_rows(name) if is_gemm(r["Kernel_Name"])]
    per = collections.OrderedDict()
    for r in rows:
        d = per.setdefault(r["Dispatch_Id"], {"kernel": short(r["Kernel_Name"]), "wgs": wgs(r),
                                               "dur": int(r["End_Timestamp"]) - int(r["Start_Timestamp"])})
        d[r["Counter_Name"]] = float(r["Counter_Value"])
    launches = [per[k] for k in sorted(per, key=int)]  # dispatch order
    labels = labeller(launches)
    by_label = collections.OrderedDict()
    for lab, d in zip(labels, launches):
        by_label.setdefault(lab, []).append(d)
    out = [f"command: {command(name)}", "", note,
           "per launch (median over the steps of the run): duration under the counter run, shader clock = GRBM_GUI_ACTIVE / 8 XCDs /",
           "duration, MFMA pipe busy = SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs x cycles), share of wave time waiting (SQ_WAIT_ANY /",
           "SQ_WAVE_CYCLES) and issuing (SQ_ACTIVE_INST_ANY / SQ_WAVE_CYCLES), other vector-ALU and LDS instructions per MFMA", "",
           f"{'launch':52s} {'wgs':>5s} {'us':>8s} {'GHz':>6s} {'MFMA busy':>10s} {'waiting':>8s} {'issuing':>8s} {'VALU/MFMA':>10s} {'LDS/MFMA':>9s}"]
    table = {}
    for lab, ds in by_label.items():
        def med(key):
            v = sorted(d[key] for d in ds)
            return v[len(v) // 2]
        dur, cyc = med("dur"), med("GRBM_GUI_ACTIVE") / 8
        row = {"us": dur / 1e3, "ghz": cyc / dur, "busy": med("SQ_VALU_MFMA_BUSY_CYCLES") / (1024 * cyc),
               "valu": (med("SQ_INSTS_VALU") - med("SQ_INSTS_MFMA")) / med("SQ_INSTS_MFMA"), "lds": med("SQ_INSTS_LDS") / med("SQ_INSTS_MFMA")}
        table[lab] = row
        out.append(f"{lab:52s} {ds[0]['wgs']:5d} {row['us']:8.1f} {row['ghz']:6.2f} {100 * row['busy']:9.1f}% "
                   f"{100 * med('SQ_WAIT_ANY') / med('SQ_WAVE_CYCLES'):7.1f}% {100 * med('SQ_ACTIVE_INST_ANY') / med('SQ_WAVE_CYCLES'):7.1f}% "
                   f"{row['valu']:10.2f} {row['lds']:9.2f}")
    return out, table


def period(seq):
    """Smallest p with seq[i] == seq[i + p] throughout: the launches of one step."""
    for p in range(1, len(seq) + 1):
        if len(seq) % p == 0 and all(seq[i] == seq[i + p] for i in range(len(seq) - p)):
            return p
    return len(seq)


def _by_position(launches):
    """(period, per position of the step: (kind, workgroups, median duration))."""
    seq = [("fwd" if "fwd" in d["kernel"] else "bwd", d["wgs"]) for d in launches]
    p = period(seq)
    pos = []
    for i in range(p):
        durs = sorted(d["dur"] for d in launches[i::p])
        pos.append((*seq[i], durs[len(durs) // 2]))
    return p, pos


def label_layer(launches):
    """The headline step's eight GEMM launches.  Launches of one kind and grid (o_proj and down forward; the three input
    gradients over 4096 columns) are told apart by their duration."""
    p, pos = _by_position(launches)
    names = {("fwd", 768): ["fwd q,k,v (K 4096, N 6144)"], ("fwd", 3584): ["fwd gate/up + SwiGLU (K 4096, N 2 x 14336)"],
             ("fwd", 512): ["fwd o (K 4096, N 4096)", "fwd down (K 14336, N 4096)"],
             ("bwd", 1792): ["dh + SwiGLU backward (N 4096 -> 14336 columns)"],
             ("bwd", 512): ["dX o (N 4096)", "dX q,k,v (N 6144)", "dX gate+up (N 2 x 14336 -> 4096 columns)"]}
    lab = [None] * p
    for key, options in names.items():
        idx = sorted((i for i in range(p) if pos[i][:2] == key), key=lambda i: pos[i][2])
        for i, name in zip(idx, options):
            lab[i] = name
    lab = [x or f"launch {i}: {pos[i][0]} [{pos[i][1]} workgroups]" for i, x in enumerate(lab)]
    return [lab[i % p] for i in range(len(launches))]


def label_mlp(launches):
    """An MLP step's launches in their order inside the step, named by kind and grid."""
    p, pos = _by_position(launches)
    lab = [f"launch {i + 1} of {p}: {'forward' if k == 'fwd' else 'input gradient'}, {w} workgroups" for i, (k, w, _) in enumerate(pos)]
    return [lab[i % p] for i in range(len(launches))]


def summarize():
    os.makedirs(OUT, exist_ok=True)
    sys.path.insert(0, ROOT)
    import bench

    # ---- kernel traces ------------------------------------------------------------------------------
    trace_summary("trace_layer", "Llama-3-8B layer step (LoRA_QKV + LoRA_W(o) + LoRA_MLP forward + backward, 8192 tokens, bf16); the run does 5 warm-up, "
                  "20 timed and 20 event-bracketed steps: the 20 timed ones are summarised", 20, 5,
                  "bench_llama3_8b_layer_kernel_trace.txt", ("gptq_lora_fwd", 3584))
    for name, title, out_file in (
            ("trace_config4", "Llama-2-70B MLP step with act-order GPTQ weights (4096 tokens, 8192 <-> 28672, r = 64, one permutation per projection): "
             "3 warm-up, 10 timed and 10 event-bracketed steps: the 10 timed ones are summarised", "bench_config4_act_order_mlp_kernel_trace.txt"),
            ("trace_config5", "Mistral-7B MLP step with NF4 weights (16384 tokens, 4096 <-> 14336, r = 8): 3 warm-up, 10 timed and 10 event-bracketed "
             "steps: the 10 timed ones are summarised", "bench_config5_nf4_mlp_kernel_trace.txt")):
        try:
            # a launch that happens once per step: the down-projection forward (512 workgroups) / the gate+up forward (7168)
            trace_summary(name, title, 10, 3, out_file, ("gptq_lora_fwd", 512 if name == "trace_config4" else 7168))
        except (FileNotFoundError, IndexError) as exc:
            print(f"[summarize] {name}: skipped ({exc})")

    # ---- traffic counters ---------------------------------------------------------------------------
    def load(name, counter):
        out = collections.OrderedDict()
        for r in counter_rows(name):
            if r["Counter_Name"] != counter:
                continue
            n = r["Kernel_Name"]
            if is_gemm(n):
                out[int(r["Dispatch_Id"])] = (short(n), wgs(r), float(r["Counter_Value"]))
            elif "copyBuffer" in n and int(r["Grid_Size"]) > out.get("copy", ("", 0, 0.0))[1]:
                # the 1 GiB calibration copy is the largest copy of the run (the step's own small copies, e.g. the
                # one-time tables of a prepared weight, come after it)
                out["copy"] = ("copyBuffer", int(r["Grid_Size"]), float(r["Counter_Value"]))
        return out
    fe, wr = load("fetch_layer", "FETCH_SIZE"), load("write_layer", "WRITE_SIZE")
    gib_kib = 1048576.0
    cf, cw = gib_kib / fe["copy"][2], gib_kib / wr["copy"][2]
    fl = [fe[k] for k in sorted(k for k in fe if k != "copy")]  # dispatch order
    wl = [wr[k] for k in sorted(k for k in wr if k != "copy")]
    # (told apart by the bytes they fetch, which rank like their durations)
    labels = label_layer([{"kernel": a[0], "wgs": a[1], "dur": a[2]} for a in fl])
    per = collections.OrderedDict()
    for lab, a, b in zip(labels, fl, wl):
        per.setdefault(lab, []).append((a[2] * cf * 1024, b[2] * cw * 1024, a[1]))
    L = ["commands (one counter per run):", f"  {command('fetch_layer')}", f"  {command('write_layer')}", "",
         "calibration: the 1 GiB device copy of --calibration-copy (__amd_rocclr_copyBuffer) reads 1048576 KiB and writes 1048576 KiB;",
         f"  FETCH_SIZE reads {fe['copy'][2]:.0f} KiB for it -> factor {cf:.3f};  WRITE_SIZE reads {wr['copy'][2]:.0f} KiB -> factor {cw:.3f}", "",
         "traffic between L2 and the fabric (MALL / HBM) per launch, median over the steps of the run, scaled by those factors:", "",
         f"{'launch':52s} {'workgroups':>10s} {'fetch MB':>10s} {'write MB':>10s} {'total MB':>10s}"]
    tot = {}
    for lab, v in per.items():
        f_ = sorted(x[0] for x in v)[len(v) // 2] / 1e6
        w_ = sorted(x[1] for x in v)[len(v) // 2] / 1e6
        tot[lab] = (f_ + w_) * 1e6
        L.append(f"{lab:52s} {v[0][2]:10d} {f_:10.1f} {w_:10.1f} {f_ + w_:10.1f}")
    L += ["", "figures bench.py reads (bytes per launch, fetch + write; the label is the launch's name on the bench line):",
          f"roofline_traffic_bytes gptq_lora_fwd<swiglu> K=4096 N=14336+14336 = {tot['fwd gate/up + SwiGLU (K 4096, N 2 x 14336)']:.0f}",
          f"roofline_traffic_bytes gptq_lora_bwd_dx<linear> K=4096 N=14336+14336 = {tot['dX gate+up (N 2 x 14336 -> 4096 columns)']:.0f}",
          f"kernel_sources_sha256 = {bench.kernel_sources_digest()}"]
    open(os.path.join(OUT, "gptq_lora_gemms_llama3_8b_hbm_traffic_pmc.txt"), "w").write("\n".join(L) + "\n")
    print("\n".join(L), "\n")

    # ---- SQ counters --------------------------------------------------------------------------------
    S, layer = sq_table("sq_layer", "Llama-3-8B layer step, bf16 (the headline workload).", label_layer)
    S += ["", "what the machine sustains with nothing but MFMAs (zero / random operands) is in yardsticks_bf16_gemm_and_mfma_loop.txt"]
    open(os.path.join(OUT, "gptq_lora_gemms_llama3_8b_mfma_busy_pmc.txt"), "w").write("\n".join(S) + "\n")
    print("\n".join(S), "\n")
    for name, note, labeller, out_file in (
            ("sq_layer_fp16", "Llama-3-8B layer step in float16 (the reference's own arithmetic for this path).", label_layer,
             "gptq_lora_gemms_llama3_8b_fp16_mfma_busy_pmc.txt"),
            ("sq_config4", "Llama-2-70B MLP step, act-order GPTQ weights with one permutation per projection (4096 tokens, r = 64).", label_mlp,
             "gptq_lora_gemms_config4_act_order_mfma_busy_pmc.txt"),
            ("sq_config5", "Mistral-7B MLP step, NF4 weights (code-book flavours of the kernels; 16384 tokens, r = 8).", label_mlp,
             "gptq_lora_gemms_config5_nf4_mfma_busy_pmc.txt")):
        try:
            T, _ = sq_table(name, note, labeller)
        except FileNotFoundError as exc:
            print(f"[summarize] {name}: skipped ({exc})")
            continue
        open(os.path.join(OUT, out_file), "w").write("\n".join(T) + "\n")
        print("\n".join(T), "\n")

    # ---- per-launch residual: where each launch of the headline step stands against the peak -----------
    tl = bench_line("trace_layer")
    if "kernels" in tl:
        names = {"fwd q,k,v (K 4096, N 6144)": "gptq_lora_fwd<linear> K=4096 N=4096+1024+1024", "fwd o (K 4096, N 4096)": "gptq_lora_fwd<linear> K=4096 N=4096",
                 "fwd gate/up + SwiGLU (K 4096, N 2 x 14336)": "gptq_lora_fwd<swiglu> K=4096 N=14336+14336", "fwd down (K 14336, N 4096)": "gptq_lora_fwd<linear> K=14336 N=4096",
                 "dh + SwiGLU backward (N 4096 -> 14336 columns)": "gptq_lora_bwd_dx<swiglu> K=14336 N=4096",
                 "dX gate+up (N 2 x 14336 -> 4096 columns)": "gptq_lora_bwd_dx<linear> K=4096 N=14336+14336", "dX o (N 4096)": "gptq_lora_bwd_dx<linear> K=4096 N=4096",
                 "dX q,k,v (N 6144)": "gptq_lora_bwd_dx<linear> K=4096 N=4096+1024+1024"}
        R = ["per-launch residual of the headline step: duration and TFLOP/s from bench.py's events in the kernel-trace run", f"  ({command('trace_layer')}),",
             "MFMA busy, clock and instruction ratios from the counter run", f"  ({command('sq_layer')}).",
             "at-clock = MFMA busy x clock / 2.4 GHz: the share of the 2516.6 TFLOP/s peak the matrix pipe delivers; the rest of the busy time computes",
             "nothing new (every launch also carries its rank-r LoRA MFMAs, < 1 %).", "",
             f"{'launch':52s} {'us':>8s} {'TFLOP/s':>8s} {'% peak':>7s} {'MFMA busy':>10s} {'GHz':>6s} {'at-clock':>9s} {'VALU/MFMA':>10s} {'LDS/MFMA':>9s}"]
        tot_us = 0.0
        for lab, row in layer.items():
            k = tl["kernels"].get(names[lab])
            if not k:
                continue
            tot_us += k["ms"] * 1e3
            R.append(f"{lab:52s} {k['ms'] * 1e3:8.1f} {k['tflops']:8.1f} {100 * k['tflops'] / 2516.6:6.1f}% {100 * row['busy']:9.1f}% {row['ghz']:6.2f} "
                     f"{100 * row['busy'] * row['ghz'] / 2.4:8.1f}% {row['valu']:10.2f} {row['lds']:9.2f}")
        R += ["", f"sum of the eight launches: {tot_us:.1f} us of the {tl['ms_per_step'] * 1e3:.1f} us step ({tl['tflops']:.1f} TFLOP/s = "
              f"{100 * tl['frac_bf16_mfma_peak']:.1f} % of peak); 50 % of peak would be {bench.layer_flops(bench.M_TOKENS) / 2516.6e12 / 0.5 * 1e6:.0f} us for the whole step"]
        open(os.path.join(OUT, "llama3_8b_layer_per_launch_residual.txt"), "w").write("\n".join(R) + "\n")
        print("\n".join(R), "\n")

    # ---- yardsticks ---------------------------------------------------------------------------------
    try:
        yj = bench_line("trace_yardsticks")["yardsticks"]
        ys = list(csv.DictReader(open(find("trace_yardsticks", "kernel_stats.csv"))))
    except (FileNotFoundError, KeyError) as exc:
        print(f"[summarize] yardsticks: skipped ({exc})")
        return
    Y = [f"command: {command('trace_yardsticks')}", "", "line printed by the run (events on the launch stream):"]
    for k, v in yj.items():
        Y.append(f"  {k:68s} {v['ms']:9.3f} ms  {v['tflops']:8.1f} TFLOP/s = {100 * v['tflops'] / 2516.6:5.1f} % of 2516.6" + (f"   {v['shape']}" if "shape" in v else ""))
    Y += ["", "kernels of the same run by total time (rocprofv3 --stats):", f"{'kernel':60s} {'calls':>6s} {'avg us':>10s}"]
    for r in ys[:6]:
        Y.append(f"{short(r['Name'])[:60]:60s} {r['Calls']:>6s} {float(r['AverageNs']) / 1e3:10.1f}")
    Y += ["", "library_bf16_gemm: torch.matmul (hipBLASLt) of the gate/up shape, bf16 in and out: no dequantisation, no LoRA term, no SwiGLU.",
          "mfma_loop_*: the probe library (csrc/probe.hip), 1024 workgroups x 4 waves x 20000 x 16 MFMA 32x32x16 bf16 out of registers: all-zero",
          "operands run at the clock limit; random operands at what the power limit leaves; the third line adds one 1 KB direct-to-LDS load per",
          "wave and 8 MFMAs (the GEMM kernels' ratio of X-tile loads), which one wave per SIMD cannot hide; the fourth also takes the A operands",
          "out of LDS (one 1 KB fragment read per wave and 2 MFMAs, a workgroup barrier per 64 MFMAs): the operand traffic of the GEMM",
          "kernels' main loop with no unpacking, no epilogue and no tile turnaround."]
    open(os.path.join(OUT, "yardsticks_bf16_gemm_and_mfma_loop.txt"), "w").write("\n".join(Y) + "\n")
    print("\n".join(Y))


if __name__ == "__main__":
    if len(sys.argv) < 2 or sys.argv[1] not in ("collect", "summarize"):
        print(__doc__)
        sys.exit(2)
    if sys.argv[1] == "collect":
        os.makedirs(RAW, exist_ok=True)
        collect(sys.argv[2:] or list(RUNS))
    else:
        summarize()

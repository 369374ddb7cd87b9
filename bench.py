#!/usr/bin/env python3
"""Benchmark of the fused GPTQ-LoRA layer (forward + backward) on one MI355X.

One step = LoRA_QKV + LoRA_W(o_proj) + LoRA_MLP forward and backward at Llama-3-8B layer shape
(8192 tokens, hidden 4096, intermediate 14336, 32 query / 8 KV heads x 128, GPTQ 4-bit group 128,
LoRA rank 16), driven through the same `apply_lora_*` entry points the model patcher installs.
Inputs are synthetic (seeded normal activations / gradients, N(0, 0.02) weights RTN-quantised)
and already resident in HBM when the timed region starts.

Before anything is timed the tensors of one step (every output, every input gradient, every dA and
dB) are compared with the CPU oracle's unfused fp32 path on the same inputs; a failed comparison
ends the run.  The same oracle runs are the CPU baseline.

Prints ONE JSON line: whole-layer tokens/s, the parity figures, the roofline of the dominant kernel
(measured live with events on the launch stream), the unfused PyTorch CPU baseline and the timings
of the other configurations of the baseline description (MLP alone, act-order at Llama-2-70B MLP
shape, NF4 at Mistral-7B MLP shape).
"""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "fms-acceleration_amd"))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6  # MI355X dense bf16 MFMA: 256 CU x 4096 FLOP/clk/CU x 2.4 GHz
PEAK_HBM_GBS = 8000.0

M_TOKENS, HIDDEN, INTER, N_HEADS, N_KV, HEAD_DIM = 8192, 4096, 14336, 32, 8, 128
RANK, GROUP = 16, 128
ALPHA_MLP, ALPHA_ATTN = 16.0, 32.0
TOL_OUT, TOL_GRAD = 1e-2, 2e-2  # max |out - ref| / max |ref| per tensor: outputs and dX; dA and dB (sums over 8192 tokens)

# L2 <-> fabric bytes per launch come from the committed counter summary (rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE, scaled by a device copy of known size): lines `roofline_traffic_bytes <kernel label> = <bytes>`,
# and `kernel_sources_sha256 = <digest>` of the two GEMM sources the counters were taken with.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gptq_lora_gemms_llama3_8b_hbm_traffic_pmc.txt")
GEMM_SOURCES = [os.path.join(ROOT, "fms-acceleration_amd", "csrc", f) for f in ("gemm_fwd.hip", "gemm_bwd.hip", "gemm_bwd_t.hip", "common.h")]

_W_BYTES = HIDDEN * INTER // 2 + (HIDDEN // GROUP) * INTER * 2 + (HIDDEN // GROUP) * INTER // 2  # packed + scales + zeros
# algorithmic bytes of the launches that can be the dominant one
ALGORITHMIC_BYTES = {
    # X once, gate and up weights once, U and B, the three outputs e, g, h
    "gptq_lora_fwd<swiglu> K=4096 N=14336+14336":
        M_TOKENS * HIDDEN * 2 + 2 * _W_BYTES + 2 * (M_TOKENS * RANK * 2 + INTER * RANK * 2) + 3 * M_TOKENS * INTER * 2,
    # d_g and d_e once, the transposed twins of the up and gate weights + their fp32 scale and offset tables once, T and
    # A^T, the mask source X, dX
    "gptq_lora_bwd_dx<linear> K=4096 N=14336+14336":
        2 * M_TOKENS * INTER * 2 + 2 * (HIDDEN * INTER // 2 + 2 * (HIDDEN // GROUP) * INTER * 4)
        + 2 * (M_TOKENS * RANK * 2 + HIDDEN * RANK * 2) + 2 * M_TOKENS * HIDDEN * 2,
}


def kernel_sources_digest():
    h = hashlib.sha256()
    for f in GEMM_SOURCES:
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def traffic_from_profile(label):
    """(bytes or None, note): the counter summary's figure for `label`, None when the summary is absent,
    has no such line, or was taken with other kernel sources than the ones in the tree."""
    if not os.path.exists(TRAFFIC_PROFILE):
        return None, "no counter summary in profiles/"
    value, digest = None, None
    for line in open(TRAFFIC_PROFILE):
        if line.startswith("roofline_traffic_bytes ") and "=" in line:
            name, _, num = line[len("roofline_traffic_bytes "):].rpartition("=")
            if name.strip() == label:
                value = float(num)
        elif line.startswith("kernel_sources_sha256"):
            digest = line.split("=")[1].strip()
    if value is None:
        return None, f"{os.path.basename(TRAFFIC_PROFILE)} has no line for this launch"
    if digest != kernel_sources_digest():
        print(f"bench.py: {os.path.basename(TRAFFIC_PROFILE)} was taken with other GEMM sources than the tree holds; "
              "roofline.traffic is left out until the counters are collected again", file=sys.stderr)
        return None, "counter summary is older than the kernel sources"
    algorithmic = ALGORITHMIC_BYTES.get(label)
    if algorithmic and not 0.5 * algorithmic <= value <= 32 * algorithmic:
        # fewer bytes than the operands hold, or more than any re-read pattern of this tiling produces: the counters
        # were scaled by the wrong calibration dispatch
        print(f"bench.py: {os.path.basename(TRAFFIC_PROFILE)} reads {value:.3g} bytes for {label}, implausible against "
              f"{algorithmic:.3g} algorithmic bytes; roofline.traffic is left out", file=sys.stderr)
        return None, "counter summary is implausible (calibration)"
    return value, os.path.relpath(TRAFFIC_PROFILE, ROOT)


def proj_flops(M, K, N, r):
    """Algorithmic FLOPs of one projection, forward + backward: base fwd + base dX (frozen W has no
    dW) plus the LoRA terms (fwd, dA incl. T = dY B, dB incl. U = X A^T, dX-LoRA)."""
    return 4 * M * K * N + 2 * M * r * (3 * (K + N) + K)


def mlp_flops(M, H, I, r):
    return 2 * proj_flops(M, H, I, r) + proj_flops(M, I, H, r)


def layer_flops(M):
    q = proj_flops(M, HIDDEN, N_HEADS * HEAD_DIM, RANK)
    kv = 2 * proj_flops(M, HIDDEN, N_KV * HEAD_DIM, RANK)
    o = proj_flops(M, N_HEADS * HEAD_DIM, HIDDEN, RANK)
    return q + kv + o + mlp_flops(M, HIDDEN, INTER, RANK)


# --------------------------------------------------------------------------------------------------
# the layer and its step
# --------------------------------------------------------------------------------------------------
def _lora_gptq(K, N, r, alpha, gen, device, lseed, group=GROUP, g_idx=None):
    import torch
    from fms_acceleration_peft import LoraLinear
    from fms_acceleration_peft.quantizer import quantize_linear

    W = torch.randn(N, K, generator=gen, device=device) * 0.02
    ql = quantize_linear(W, group, g_idx=g_idx).to(device)
    del W
    lin = LoraLinear(ql, r, alpha).to(device)
    g2 = torch.Generator().manual_seed(lseed)
    lin.lora_B["default"].weight.data.copy_(torch.randn(N, r, generator=g2) * 0.02)
    return lin


def build_layer(device, seed=0):
    """attn (q/k/v/o) and mlp (gate/up/down) containers of LoraLinear(QuantLinear)."""
    import torch

    gen = torch.Generator(device=device).manual_seed(seed)
    attn, mlp = torch.nn.Module(), torch.nn.Module()
    attn.q_proj = _lora_gptq(HIDDEN, N_HEADS * HEAD_DIM, RANK, ALPHA_ATTN, gen, device, 1)
    attn.k_proj = _lora_gptq(HIDDEN, N_KV * HEAD_DIM, RANK, ALPHA_ATTN, gen, device, 2)
    attn.v_proj = _lora_gptq(HIDDEN, N_KV * HEAD_DIM, RANK, ALPHA_ATTN, gen, device, 3)
    attn.o_proj = _lora_gptq(N_HEADS * HEAD_DIM, HIDDEN, RANK, ALPHA_ATTN, gen, device, 4)
    mlp.gate_proj = _lora_gptq(HIDDEN, INTER, RANK, ALPHA_MLP, gen, device, 5)
    mlp.up_proj = _lora_gptq(HIDDEN, INTER, RANK, ALPHA_MLP, gen, device, 6)
    mlp.down_proj = _lora_gptq(INTER, HIDDEN, RANK, ALPHA_MLP, gen, device, 7)
    return attn, mlp


def make_step(attn, mlp, M, device, dtype, io=None):
    """The timed step.  `io`, when given, receives the step's inputs once and its outputs after every call."""
    import torch
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import (
        apply_lora_mlp,
        apply_lora_o_v2,
        apply_lora_qkv,
    )

    gen = torch.Generator(device=device).manual_seed(2)
    rn = lambda *s: torch.randn(*s, generator=gen, device=device).to(dtype)  # noqa: E731
    x_attn = rn(1, M, HIDDEN).requires_grad_(True)
    x_o = rn(1, M, N_HEADS * HEAD_DIM).requires_grad_(True)
    x_mlp = rn(1, M, HIDDEN).requires_grad_(True)
    dQ, dK, dV = rn(1, M, N_HEADS * HEAD_DIM), rn(1, M, N_KV * HEAD_DIM), rn(1, M, N_KV * HEAD_DIM)
    dO, dY = rn(1, M, HIDDEN), rn(1, M, HIDDEN)
    params = [p for mod in (attn, mlp) for p in mod.parameters() if p.requires_grad]
    if io is not None:
        io.update(x_attn=x_attn, x_o=x_o, x_mlp=x_mlp, dQ=dQ, dK=dK, dV=dV, dO=dO, dY=dY)

    def step():
        for t in (x_attn, x_o, x_mlp, *params):
            t.grad = None
        Q, K, V = apply_lora_qkv(attn, x_attn)
        O = apply_lora_o_v2(attn.o_proj, x_o)
        Y = apply_lora_mlp(mlp, x_mlp)
        torch.autograd.backward([Q, K, V, O, Y], [dQ, dK, dV, dO, dY])
        if io is not None:
            io.update(Q=Q, K=K, V=V, O=O, Y=Y)

    return step


PROJ_NAMES = (("q", "attn", "q_proj"), ("k", "attn", "k_proj"), ("v", "attn", "v_proj"), ("o", "attn", "o_proj"),
              ("gate", "mlp", "gate_proj"), ("up", "mlp", "up_proj"), ("down", "mlp", "down_proj"))


def gpu_results(attn, mlp, io, rows=None):
    """Every tensor one step produced, on the CPU in fp32 (`rows`: only those token rows of the row-wise ones)."""
    mods = {"attn": attn, "mlp": mlp}
    sel = (lambda t: t[0]) if rows is None else (lambda t: t[0][rows.to(t.device)])
    out = {k: sel(io[k].detach()).float().cpu() for k in ("Q", "K", "V", "O", "Y")}
    out.update({"dX_attn": sel(io["x_attn"].grad).float().cpu(), "dX_o": sel(io["x_o"].grad).float().cpu(),
                "dX_mlp": sel(io["x_mlp"].grad).float().cpu()})
    for name, holder, attr in PROJ_NAMES:
        lin = getattr(mods[holder], attr)
        out[f"dA_{name}"] = lin.lora_A["default"].weight.grad.detach().float().cpu()
        out[f"dB_{name}"] = lin.lora_B["default"].weight.grad.detach().float().cpu()
    return out


# --------------------------------------------------------------------------------------------------
# the oracle's unfused path on the same inputs: parity reference and CPU baseline
# --------------------------------------------------------------------------------------------------
def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.lower().startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def oracle_step(attn, mlp, io, act_dtype, rows=None):
    """A callable running the reference's UNFUSED path as restated by the oracle (dense dequant inside the call,
    x @ W, PEFT-style LoRA, HF SwiGLU MLP, torch.autograd backward) in fp32 on the host, on the inputs and packed
    weights of the GPU step (all tokens, or the token rows `rows`); returns the same dict gpu_results() returns."""
    import torch

    from oracle import gptq as ogptq
    from oracle import lora as olora

    mods = {"attn": attn, "mlp": mlp}
    packed = {}
    for name, holder, attr in PROJ_NAMES:
        lin = getattr(mods[holder], attr)
        base = lin.base_layer
        # the kernels see the adapters rounded to the activation type (matmul_lora casts them, UL/gptq/fast_lora.py:167)
        A = lin.lora_A["default"].weight.detach().to(act_dtype).float().cpu()
        B = lin.lora_B["default"].weight.detach().to(act_dtype).float().cpu()
        packed[name] = (base.qweight.cpu(), base.scales.cpu(), base.qzeros.cpu(), base.g_idx.cpu(), A, B, float(lin.scaling["default"]))
    take = (lambda t: t[0]) if rows is None else (lambda t: t[0][rows.to(t.device)])
    cpu = {k: take(io[k].detach()).float().cpu() for k in ("x_attn", "x_o", "x_mlp", "dQ", "dK", "dV", "dO", "dY")}

    def dense(name):
        qw, sc, qz, gi, A, B, s = packed[name]
        return ogptq.dequant_torch(qw, sc, qz, gi), A, B, s

    def zero_rows(x):
        return torch.nonzero((x == 0).any(dim=1)).flatten()

    def run():
        dq, dk, dv, do = dense("q"), dense("k"), dense("v"), dense("o")
        (Q, K, V), dxa, gq = olora.lora_qkv_autograd(cpu["x_attn"], [dq, dk, dv], [cpu["dQ"], cpu["dK"], cpu["dV"]])
        O, dxo, dAo, dBo = olora.lora_w_autograd(cpu["x_o"], *do, cpu["dO"])
        dg, du, dd = dense("gate"), dense("up"), dense("down")
        Y, dxm, gm, _ = olora.lora_mlp_autograd(cpu["x_mlp"], dg, du, dd, cpu["dY"])
        # The fused backward keeps the reference's `(X != 0)` factor on the LoRA part of dX
        # (UL/gptq/fast_lora.py:391,398,662-674,831), which autograd of the unfused graph does not have: the two differ
        # exactly where an input entry is 0.0.  Rows that hold such an entry take dX from the oracle's statement of the
        # hand-derived backward instead (a handful of rows of seeded normal inputs, if any).
        zr = zero_rows(cpu["x_attn"])
        if len(zr):
            dxa[zr] = olora.lora_qkv_manual(cpu["x_attn"][zr], [dq, dk, dv], [cpu["dQ"][zr], cpu["dK"][zr], cpu["dV"][zr]])[0]
        zr = zero_rows(cpu["x_o"])
        if len(zr):
            dxo[zr] = olora.lora_w_manual(cpu["x_o"][zr], *do, cpu["dO"][zr])[0]
        zr = zero_rows(cpu["x_mlp"])
        if len(zr):
            dxm[zr] = olora.lora_mlp_manual(cpu["x_mlp"][zr], dg, du, dd, cpu["dY"][zr])[0]
        out = {"Q": Q, "K": K, "V": V, "O": O, "Y": Y, "dX_attn": dxa, "dX_o": dxo, "dX_mlp": dxm, "dA_o": dAo, "dB_o": dBo}
        for n, (dA, dB) in zip(("q", "k", "v"), gq):
            out[f"dA_{n}"], out[f"dB_{n}"] = dA, dB
        for n, (dA, dB) in zip(("gate", "up", "down"), gm):
            out[f"dA_{n}"], out[f"dB_{n}"] = dA, dB
        return out

    return run


def parity_report(got, ref, what):
    """Per-tensor figures, worst ones on top: max |out - ref| / max |ref| (the gate) and the element-wise relative
    error over the entries with |ref| > 1e-2 max |ref| (reported)."""
    from oracle import lora as olora

    worst = {"outputs_dX": (0.0, ""), "dA_dB": (0.0, "")}
    ew_max, ew_mean, ok = 0.0, 0.0, True
    per = {}
    for k, r in ref.items():
        e = olora.max_rel_err(got[k], r)
        m, a = olora.elementwise_rel_err(got[k], r, 1e-2)
        per[k] = round(e, 6)
        cls = "dA_dB" if k.startswith(("dA_", "dB_")) else "outputs_dX"
        if e >= worst[cls][0]:
            worst[cls] = (e, k)
        ew_max, ew_mean = max(ew_max, m), max(ew_mean, a)
        ok = ok and e <= (TOL_GRAD if cls == "dA_dB" else TOL_OUT)
    return {
        "ok": ok, "checked": what, "tensors": len(ref),
        "max_rel_err": worst["outputs_dX"][0], "max_rel_err_tensor": worst["outputs_dX"][1], "tolerance": TOL_OUT,
        "max_rel_err_dA_dB": worst["dA_dB"][0], "max_rel_err_dA_dB_tensor": worst["dA_dB"][1], "tolerance_dA_dB": TOL_GRAD,
        "elementwise_rel_err_over_1e-2": {"max": ew_max, "mean_of_worst_tensor": ew_mean},
        "per_tensor_max_rel_err": per,
    }


def cpu_threads():
    """Host threads for the oracle: the box's CPU share (OMP_NUM_THREADS is set to it there), else every core."""
    env = os.environ.get("OMP_NUM_THREADS")
    return int(env) if env and env.isdigit() and int(env) > 0 else (os.cpu_count() or 1)


def cpu_baseline_and_reference(attn, mlp, io, act_dtype, reps=3):
    """Times the oracle's unfused path at the full shape (1 warm-up + `reps` repetitions) and keeps the tensors of
    the last repetition as the parity reference.  A repetition over 60 s falls back to 1024 tokens, and says so."""
    import torch

    threads = cpu_threads()
    torch.set_num_threads(threads)
    M = io["x_attn"].shape[1]
    run = oracle_step(attn, mlp, io, act_dtype)
    t0 = time.perf_counter()
    ref = run()  # warm-up
    warm = time.perf_counter() - t0
    rows = None
    if warm > 60.0:
        rows = torch.arange(1024)
        run = oracle_step(attn, mlp, io, act_dtype, rows)
        ref = run()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        ref = run()
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[len(times) // 2]
    m_used = M if rows is None else len(rows)
    sample = (f"all {M} tokens" if rows is None else f"the first {m_used} of {M} tokens (a full repetition took {warm:.0f} s)")
    base = {
        "value": m_used / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"{sample} of the same layer and inputs (full-size weights, dequantisation inside the timed region), fp32, "
                  f"1 warm-up + {reps} repetitions, median {dt:.2f} s; {threads} threads of {os.cpu_count()} logical CPUs",
        "cpu_model": cpu_model_name(), "seconds_per_step": dt, "gflops": layer_flops(m_used) / dt / 1e9,
    }
    return base, ref, rows


# --------------------------------------------------------------------------------------------------
# per-launch timing
# --------------------------------------------------------------------------------------------------
class LaunchTimer:
    """Brackets every fused-GEMM launch of the step with a pair of events recorded on the stream the
    kernel is launched on (torch's current stream), by wrapping the two ctypes entry points."""

    def __init__(self, M):
        import fmsa_hip

        self.mod, self.M, self.records = fmsa_hip, M, []
        self._fwd, self._bwd = fmsa_hip.gptq_lora_fwd, fmsa_hip.gptq_lora_bwd_dx

    def _timed(self, label, flop, fn, *args, **kw):
        import torch

        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        out = fn(*args, **kw)
        e.record()
        self.records.append((label, flop, s, e))
        return out

    def __enter__(self):
        mod, M = self.mod, self.M

        def fwd(x2d, projs, mode=mod.FWD_LINEAR, **kw):
            K, Ns = projs[0]["w"].K, [p["w"].N for p in projs]
            flop = sum(2.0 * M * K * n + 2.0 * M * p["r"] * n for n, p in zip(Ns, projs))
            kind = "swiglu" if mode == mod.FWD_SWIGLU else "linear"
            return self._timed(f"gptq_lora_fwd<{kind}> K={K} N={'+'.join(map(str, Ns))}", flop, self._fwd, x2d, projs, mode, **kw)

        def bwd(projs, M_, K, mode=mod.BWD_LINEAR, **kw):
            Ns = [p["w"].N for p in projs]
            flop = sum(2.0 * M * K * n + 2.0 * M * p["r"] * K for n, p in zip(Ns, projs))
            kind = "swiglu" if mode == mod.BWD_SWIGLU else "linear"
            return self._timed(f"gptq_lora_bwd_dx<{kind}> K={K} N={'+'.join(map(str, Ns))}", flop, self._bwd, projs, M_, K, mode, **kw)

        mod.gptq_lora_fwd, mod.gptq_lora_bwd_dx = fwd, bwd
        return self

    def __exit__(self, *exc):
        self.mod.gptq_lora_fwd, self.mod.gptq_lora_bwd_dx = self._fwd, self._bwd

    def summary(self):
        """label -> (average ms per launch, algorithmic FLOP per launch, launches)."""
        acc = {}
        for label, flop, s, e in self.records:
            t = acc.setdefault(label, [0.0, flop, 0])
            t[0] += s.elapsed_time(e)
            t[2] += 1
        return {k: (v[0] / v[2], v[1], v[2]) for k, v in acc.items()}


def time_steps(step, steps, warmup):
    import torch

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


# --------------------------------------------------------------------------------------------------
# the other configurations of the baseline description: MLP forward + backward only, timed for reference
# --------------------------------------------------------------------------------------------------
def _timed_mlp(op, mlp, M, H, I, r, note, device, dtype, steps, warmup, launch_timing=False):
    import torch

    gen = torch.Generator(device=device).manual_seed(2)
    x = torch.randn(M, H, generator=gen, device=device).to(dtype).requires_grad_(True)
    dy = torch.randn(M, H, generator=gen, device=device).to(dtype)
    params = [p for p in mlp.parameters() if p.requires_grad]

    def step():
        for t in (x, *params):
            t.grad = None
        op(mlp, x).backward(dy)

    dt = time_steps(step, steps, warmup)
    fl = mlp_flops(M, H, I, r)
    out = {"ms_per_step": dt * 1e3, "tokens_per_s": M / dt, "tflops": fl / dt / 1e12,
           "frac_bf16_mfma_peak": fl / dt / 1e12 / PEAK_BF16_TFLOPS, "workload": note}
    if launch_timing:
        with LaunchTimer(M) as timer:
            for _ in range(steps):
                step()
            torch.cuda.synchronize()
        out["kernels"] = {k: {"ms": v[0], "tflops": v[1] / v[0] / 1e9} for k, v in timer.summary().items()}
    return out


def build_act_order_mlp(device, shared):
    """Config 4: Llama-2-70B MLP shape, desc_act GPTQ: g_idx is a seeded random permutation of the group assignments
    along K; act-order GPTQ gives projections quantised on the same input one permutation (`shared`), the description
    draws one each."""
    import torch

    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp

    H, I, r, alpha = 8192, 28672, 64, 128.0
    gen = torch.Generator(device=device).manual_seed(0)
    mlp = torch.nn.Module()
    for i, (name, K, N) in enumerate((("gate_proj", H, I), ("up_proj", H, I), ("down_proj", I, H))):
        pseed = 1234 + K if shared else 40 + i
        perm = torch.randperm(K, generator=torch.Generator().manual_seed(pseed))
        g_idx = (torch.arange(K) // GROUP)[perm].to(torch.int32).to(device)
        setattr(mlp, name, _lora_gptq(K, N, r, alpha, gen, device, 20 + i, g_idx=g_idx))
    note = ("LoRA_MLP fwd+bwd, 4096 tokens, 8192<->28672, GPTQ g128 desc_act, r=64, "
            + ("gate and up share their permutation" if shared else "one random permutation per projection"))
    return apply_lora_mlp, mlp, 4096, H, I, r, note


def build_nf4_mlp(device, dtype):
    """Config 5: Mistral-7B MLP shape, NF4 with double-quantised statistics, 16384 packed tokens."""
    import torch

    from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_mlp_swiglu
    from fms_acceleration_peft import Linear4bit, LoraLinear

    H, I, r, alpha = 4096, 14336, 8, 16.0
    gen = torch.Generator(device=device).manual_seed(0)
    mlp = torch.nn.Module()
    for i, (name, K, N) in enumerate((("gate_proj", H, I), ("up_proj", H, I), ("down_proj", I, H))):
        W = torch.randn(N, K, generator=gen, device=device) * 0.02
        lin = LoraLinear(Linear4bit.from_dense(W, compute_dtype=dtype), r, alpha).to(device)
        lin.lora_B["default"].weight.data.copy_(torch.randn(N, r, generator=torch.Generator().manual_seed(30 + i)) * 0.02)
        setattr(mlp, name, lin)
        del W
    return (apply_lora_mlp_swiglu, mlp, 16384, H, I, r,
            "LoRA_MLP fwd+bwd, 16384 packed tokens, 4096<->14336, NF4 b64 + 8-bit absmax b256, r=8")


def other_configs(device, dtype, mlp_layer, steps=10, warmup=3):
    import torch

    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp

    out = {"config2_llama3_8b_mlp": _timed_mlp(apply_lora_mlp, mlp_layer, M_TOKENS, HIDDEN, INTER, RANK,
                                               "LoRA_MLP fwd+bwd, 8192 tokens, 4096<->14336, GPTQ g128, r=16",
                                               device, dtype, steps, warmup)}
    out["config4_llama2_70b_mlp_act_order"] = _timed_mlp(*build_act_order_mlp(device, False), device, dtype, steps, warmup)
    torch.cuda.empty_cache()
    out["config4_shared_permutation"] = _timed_mlp(*build_act_order_mlp(device, True), device, dtype, steps, warmup)
    torch.cuda.empty_cache()
    out["config5_mistral_7b_mlp_nf4"] = _timed_mlp(*build_nf4_mlp(device, dtype), device, dtype, steps, warmup)
    return out


def qkv_rope_config(device, dtype, attn, steps=200, warmup=20):
    """Forward of the Q / K / V projections with the rotary embedding of Q and K: applied in the epilogue of the
    projection launch (apply_lora_qkv_rope) against the projections followed by the in-place rotary kernel on Q and
    on K (what the reference's fast_rope_embedding does after its fused projections)."""
    import torch

    import fmsa_hip
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv, apply_lora_qkv_rope

    attn.head_dim = HEAD_DIM
    x = torch.randn(1, M_TOKENS, HIDDEN, generator=torch.Generator(device=device).manual_seed(5), device=device).to(dtype)
    ang = torch.outer(torch.arange(M_TOKENS).float(), 1.0 / (10000 ** (torch.arange(0, HEAD_DIM, 2).float() / HEAD_DIM)))
    emb = torch.cat([ang, ang], -1)
    cos, sin = emb.cos().to(dtype).to(device), emb.sin().to(dtype).to(device)

    def plain():
        with torch.no_grad():
            apply_lora_qkv(attn, x)

    def separate():
        with torch.no_grad():
            Q, K, _ = apply_lora_qkv(attn, x)
            fmsa_hip.rope_embedding_(Q.view(M_TOKENS, -1), cos, sin, N_HEADS, HEAD_DIM)
            fmsa_hip.rope_embedding_(K.view(M_TOKENS, -1), cos, sin, N_KV, HEAD_DIM)

    def fused():
        with torch.no_grad():
            apply_lora_qkv_rope(attn, x, cos, sin)

    us = {k: time_steps(f, steps, warmup) * 1e6 for k, f in (("projections_only", plain), ("separate_passes", separate), ("in_epilogue", fused))}
    return {"workload": "LoRA_QKV forward + rotary embedding of Q and K, 8192 tokens, 32 + 8 heads of 128, bf16 tables",
            "us_projections_only": us["projections_only"], "us_with_separate_rope_passes": us["separate_passes"],
            "us_with_rope_in_epilogue": us["in_epilogue"]}


def attention_config(device, dtype, attn, steps=20, warmup=5):
    """The attention half of the layer alone (the baseline description's third configuration): LoRA_QKV + LoRA_W(o_proj)
    forward + backward at the Llama-3-8B shape."""
    import torch

    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_o_v2, apply_lora_qkv

    gen = torch.Generator(device=device).manual_seed(3)
    rn = lambda *s: torch.randn(*s, generator=gen, device=device).to(dtype)  # noqa: E731
    x_attn, x_o = rn(1, M_TOKENS, HIDDEN).requires_grad_(True), rn(1, M_TOKENS, N_HEADS * HEAD_DIM).requires_grad_(True)
    grads = [rn(1, M_TOKENS, N_HEADS * HEAD_DIM), rn(1, M_TOKENS, N_KV * HEAD_DIM), rn(1, M_TOKENS, N_KV * HEAD_DIM), rn(1, M_TOKENS, HIDDEN)]
    params = [p for p in attn.parameters() if p.requires_grad]

    def step():
        for t in (x_attn, x_o, *params):
            t.grad = None
        Q, K, V = apply_lora_qkv(attn, x_attn)
        O = apply_lora_o_v2(attn.o_proj, x_o)
        torch.autograd.backward([Q, K, V, O], grads)

    dt = time_steps(step, steps, warmup)
    fl = layer_flops(M_TOKENS) - mlp_flops(M_TOKENS, HIDDEN, INTER, RANK)
    return {"ms_per_step": dt * 1e3, "tokens_per_s": M_TOKENS / dt, "tflops": fl / dt / 1e12,
            "frac_bf16_mfma_peak": fl / dt / 1e12 / PEAK_BF16_TFLOPS,
            "workload": "LoRA_QKV + LoRA_W(o_proj) fwd+bwd, 8192 tokens, 32 + 8 heads of 128, GPTQ g128, r=16"}


def fp16_layer_config(device, attn, mlp, M, steps, warmup):
    """The same layer step in float16, the reference's own arithmetic for the GPTQ path (its dequantisation always emits
    fp16 and its GPTQ-LoRA benchmarks run in fp16: scripts/benchmarks/scenarios.yaml:111-112): outputs and dX of one step
    on 128 sampled token rows against the fp32 oracle first, then the timed steps and the per-launch figures."""
    import torch

    dtype = torch.float16
    io = {}
    step = make_step(attn, mlp, M, device, dtype, io)
    step()
    torch.cuda.synchronize()
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(11))[:128].sort().values
    torch.set_num_threads(cpu_threads())
    ref = oracle_step(attn, mlp, io, dtype, rows)()
    got = gpu_results(attn, mlp, io, rows)
    keep = [k for k in ref if not k.startswith(("dA_", "dB_"))]
    parity = parity_report({k: got[k] for k in keep}, {k: ref[k] for k in keep},
                           "outputs and dX of one float16 step on 128 sampled token rows against the fp32 oracle")
    del got, ref, io
    out = {"workload": "the headline layer step in float16 (LoRA_QKV + LoRA_W(o_proj) + LoRA_MLP fwd+bwd, 8192 tokens)",
           "dtype": "f16", "parity": {k: parity[k] for k in ("ok", "checked", "max_rel_err", "max_rel_err_tensor", "tolerance")}}
    if not parity["ok"]:
        out["error"] = "parity check failed, not timed"
        return out
    step = make_step(attn, mlp, M, device, dtype)
    dt = time_steps(step, steps, warmup)
    fl = layer_flops(M)
    out.update({"ms_per_step": dt * 1e3, "tokens_per_s": M / dt, "tflops": fl / dt / 1e12,
                "frac_f16_mfma_peak": fl / dt / 1e12 / PEAK_BF16_TFLOPS})  # fp16 and bf16 dense MFMA peaks are equal
    with LaunchTimer(M) as timer:
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
    out["kernels"] = {k: {"ms": v[0], "tflops": v[1] / v[0] / 1e9} for k, v in timer.summary().items()}
    return out


def yardsticks(device):
    """What the machine at hand sustains, next to the fused kernels' figures: the vendor library's plain bf16 GEMM of
    the gate/up shape (no dequantisation, no LoRA, no SwiGLU), and the register-only MFMA loop of the library with
    zero operands, random operands, and random operands plus the GEMM kernels' ratio of direct-to-LDS loads."""
    import torch

    import fmsa_hip

    def ev_time(fn, n, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        for _ in range(n):
            fn()
        e.record()
        torch.cuda.synchronize()
        return s.elapsed_time(e) / n * 1e-3

    # the MFMA-loop probe is a library of its own (fms-acceleration_amd/csrc/probe.hip -> lib/libfmsa_probe.so), not part of
    # the product's C ABI
    import ctypes

    probe_path = os.path.join(os.path.dirname(os.path.abspath(fmsa_hip.__file__)), "..", "lib", "libfmsa_probe.so")
    probe_lib = ctypes.CDLL(os.path.abspath(probe_path))
    probe_lib.fmsa_probe_mfma.restype = ctypes.c_int
    probe_lib.fmsa_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]

    def probe_mfma(mode, iters, n_workgroups, dev):
        out = torch.empty(n_workgroups * 256, dtype=torch.float32, device=dev)
        # bf16 pairs in +-[1, 2), the kind of operand the loop keeps in registers (mode 3 feeds them to the MFMAs through LDS)
        src = (torch.randint(0, 1 << 32, (1 << 18,), dtype=torch.int64, device=dev) & 0x807F807F | 0x3F803F80).to(torch.int32)
        rc = probe_lib.fmsa_probe_mfma(mode, iters, n_workgroups, out.data_ptr(), src.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, f"fmsa_probe_mfma returned {rc}"
        return float(n_workgroups) * 4 * iters * 16 * 32768.0

    gen = torch.Generator(device=device).manual_seed(0)
    x = torch.randn(M_TOKENS, HIDDEN, generator=gen, device=device).to(torch.bfloat16)
    w = (torch.randn(HIDDEN, 2 * INTER, generator=gen, device=device) * 0.02).to(torch.bfloat16)
    y = torch.empty(M_TOKENS, 2 * INTER, dtype=torch.bfloat16, device=device)
    t = ev_time(lambda: torch.matmul(x, w, out=y), 30, 10)
    out = {"library_bf16_gemm": {"shape": f"[{M_TOKENS}, {HIDDEN}] x [{HIDDEN}, {2 * INTER}]", "ms": t * 1e3,
                                 "tflops": 2.0 * M_TOKENS * HIDDEN * 2 * INTER / t / 1e12}}
    del x, w, y
    for mode, name in ((0, "mfma_loop_zero_operands"), (1, "mfma_loop_random_operands"), (2, "mfma_loop_random_operands_with_direct_loads"),
                       (3, "mfma_loop_random_operands_with_direct_loads_and_lds_fragment_reads")):
        flop = [0.0]

        def run():
            flop[0] = probe_mfma(mode, 20000, 1024, device)

        t = ev_time(run, 5, 2)  # 5 x about 40 ms: long enough for the clocks to settle under the power limit
        out[name] = {"ms": t * 1e3, "tflops": flop[0] / t / 1e12}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--tokens", type=int, default=M_TOKENS)
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the CPU baseline; the parity gate then checks a sample of token rows instead of every token")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true")
    ap.add_argument("--workload", default="layer", choices=["layer", "layer_fp16", "config4", "config4_shared", "config5"],
                    help="profiling runs: time ONE of the other workloads (its own JSON line: step time and per-launch figures; "
                         "parity of these is the business of tests/test_gpu_full_size.py) instead of the headline layer")
    ap.add_argument("--no-parity", action="store_true", help="profiling runs only: skip the parity gate (the line says so)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one device copy of 1 GiB (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--yardsticks", action="store_true",
                    help="instead of the benchmark: time the vendor library's bf16 GEMM of the gate/up shape and the "
                         "register-only MFMA loop, and print them as one JSON line")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the fused-LoRA path is data parallel over tokens and this build "
              "has no multi-GPU leg; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no GPU is visible (there is no CPU fallback for the fused path)", file=sys.stderr)
        sys.exit(3)
    device, dtype, M = torch.device("cuda:0"), torch.bfloat16, args.tokens
    if args.yardsticks:
        print(json.dumps({"yardsticks": yardsticks(device), "peak_bf16_tflops": PEAK_BF16_TFLOPS}))
        return

    if args.workload != "layer":
        if args.workload == "layer_fp16":
            attn, mlp = build_layer(device)
            out = fp16_layer_config(device, attn, mlp, M, args.steps, args.warmup)
        else:
            built = (build_nf4_mlp(device, dtype) if args.workload == "config5"
                     else build_act_order_mlp(device, args.workload == "config4_shared"))
            out = _timed_mlp(*built, device, dtype, args.steps, args.warmup, launch_timing=not args.no_kernel_timing)
        print(json.dumps({"workload_only": args.workload, **out}))
        return

    attn, mlp = build_layer(device)
    io = {}
    step = make_step(attn, mlp, M, device, dtype, io)

    # ---- parity gate (and CPU baseline): nothing is timed on the GPU before this passes ----------------
    cpu_base, parity = None, {"ok": None, "checked": "skipped (--no-parity)"}
    if not args.no_parity:
        step()
        torch.cuda.synchronize()
        if not args.no_cpu_baseline:
            got = gpu_results(attn, mlp, io)
            cpu_base, ref, rows = cpu_baseline_and_reference(attn, mlp, io, dtype)
            if rows is not None:  # fallback sample: row-wise tensors only
                got = gpu_results(attn, mlp, io, rows)
                ref = {k: v for k, v in ref.items() if not k.startswith(("dA_", "dB_"))}
            parity = parity_report(got, ref, "every output, dX, dA and dB of one step against the fp32 oracle on "
                                   + ("all tokens" if rows is None else f"{len(rows)} token rows (outputs and dX only)"))
        else:
            rows = torch.randperm(M, generator=torch.Generator().manual_seed(7))[:128].sort().values
            torch.set_num_threads(cpu_threads())
            ref = oracle_step(attn, mlp, io, dtype, rows)()
            got = gpu_results(attn, mlp, io, rows)
            parity = parity_report({k: got[k] for k in ref if not k.startswith(("dA_", "dB_"))},
                                   {k: v for k, v in ref.items() if not k.startswith(("dA_", "dB_"))},
                                   "outputs and dX of one step on 128 sampled token rows against the fp32 oracle "
                                   "(dA / dB are sums over all tokens: checked only with the CPU baseline on)")
        del got, ref
        if not parity["ok"]:
            print(json.dumps({"error": "parity gate failed, nothing was timed", "parity": parity}))
            sys.exit(1)

    if args.calibration_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    io_keep, io = io, None
    step = make_step(attn, mlp, M, device, dtype)  # the timed step keeps no references to its outputs
    del io_keep
    dt = time_steps(step, args.steps, args.warmup)

    flops = layer_flops(M)
    result = {
        "metric": "fused GPTQ-LoRA layer fwd+bwd tokens/s + % bf16 MFMA peak, Llama-3-8B shape",
        "value": M / dt,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": dt * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "llama3-8b layer: LoRA_QKV + LoRA_W(o_proj) + LoRA_MLP(SwiGLU) fwd+bwd "
                        "(BASELINE configs[1]+configs[2])",
            "tokens": M, "hidden": HIDDEN, "intermediate": INTER, "q_heads": N_HEADS, "kv_heads": N_KV,
            "head_dim": HEAD_DIM, "quant": "gptq-4bit-g128", "lora_rank": RANK,
        },
        "tflops": flops / dt / 1e12,
        "frac_bf16_mfma_peak": flops / dt / 1e12 / PEAK_BF16_TFLOPS,
        "algorithmic_tflop_per_step": flops / 1e12,
        "parity": parity,
    }
    if not args.no_kernel_timing:
        # the same K steps once more, every fused-GEMM launch bracketed by events on its stream (kept
        # out of the pass that produced `value`: the event packets serialise the queue a little)
        with LaunchTimer(M) as timer:
            for _ in range(args.steps):
                step()
            torch.cuda.synchronize()
        kt = timer.summary()
        per_step = {k: v[0] * v[2] / args.steps for k, v in kt.items()}
        dominant = max(per_step, key=per_step.get)
        ms, fl, _ = kt[dominant]
        traffic, traffic_note = traffic_from_profile(dominant)
        result["roofline"] = {
            "kernel": dominant, "bound": "mfma", "achieved": fl / ms / 1e9, "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s", "frac": fl / ms / 1e9 / PEAK_BF16_TFLOPS, "traffic": traffic, "traffic_source": traffic_note,
            "avg_launch_ms": ms, "algorithmic_flop_per_launch": fl,
            "algorithmic_bytes_per_launch": ALGORITHMIC_BYTES.get(dominant),
        }
        result["kernels"] = {k: {"ms": v[0], "tflops": v[1] / v[0] / 1e9, "launches_per_step": v[2] / args.steps}
                             for k, v in kt.items()}
        # spread of the step time: the K steps a third time with one event per step boundary
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
        marks[0].record()
        for i in range(args.steps):
            step()
            marks[i + 1].record()
        torch.cuda.synchronize()
        per = sorted(a.elapsed_time(b) for a, b in zip(marks[:-1], marks[1:]))
        q = lambda p: per[min(len(per) - 1, int(round(p * (len(per) - 1))))]  # noqa: E731
        result["ms_per_step_quantiles"] = {"p10": q(0.1), "p50": q(0.5), "p90": q(0.9)}
    if cpu_base is not None:
        result["cpu_baseline"] = cpu_base
    if not args.no_other_configs:
        del step
        fp16_cfg = fp16_layer_config(device, attn, mlp, M, args.steps, args.warmup)
        rope_cfg = qkv_rope_config(device, dtype, attn)
        attn_cfg = attention_config(device, dtype, attn)
        attn = None
        torch.cuda.empty_cache()
        result["other_configs"] = other_configs(device, dtype, mlp)
        result["other_configs"]["config3_llama3_8b_attention"] = attn_cfg
        result["other_configs"]["qkv_with_rope_llama3_8b"] = rope_cfg
        result["other_configs"]["llama3_8b_layer_fp16"] = fp16_cfg
    print(json.dumps(result))


if __name__ == "__main__":
    main()

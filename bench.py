#!/usr/bin/env python3
"""Benchmark of the fused GPTQ-LoRA layer (forward + backward) on one MI355X.

One step = LoRA_QKV + LoRA_W(o_proj) + LoRA_MLP forward and backward at Llama-3-8B layer shape
(8192 tokens, hidden 4096, intermediate 14336, 32 query / 8 KV heads x 128, GPTQ 4-bit group 128,
LoRA rank 16), driven through the same `apply_lora_*` entry points the model patcher installs.
Inputs are synthetic (seeded normal activations / gradients, N(0, 0.02) weights RTN-quantised)
and already resident in HBM when the timed region starts.

Prints ONE JSON line: whole-layer tokens/s, the roofline of the dominant kernel (measured live with
events on the launch stream) and the unfused PyTorch CPU baseline on a bounded sample.
"""
from __future__ import annotations

import argparse
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

# Bytes per launch that cross between L2 and the fabric (MALL / HBM) for the two launches that can
# be the dominant one: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, each scaled by what the
# same counter reads for the 1 GiB device copy of --calibration-copy (factors 2.000 and 1.000);
# profiles/gptq_lora_gemms_llama3_8b_hbm_traffic_pmc.txt holds the runs.
ROOFLINE_TRAFFIC_BYTES = {
    "gptq_lora_fwd<swiglu> K=4096 N=14336+14336": 1447.5e6 + 719.5e6,
    "gptq_lora_bwd_dx<linear> K=4096 N=14336+14336": 1532.6e6 + 67.1e6,
}
_W_BYTES = HIDDEN * INTER // 2 + (HIDDEN // GROUP) * INTER * 2 + (HIDDEN // GROUP) * INTER // 2  # packed + scales + zeros
# algorithmic bytes of the same launches
ALGORITHMIC_BYTES = {
    # X once, gate and up weights once, U and B, the three outputs e, g, h
    "gptq_lora_fwd<swiglu> K=4096 N=14336+14336":
        M_TOKENS * HIDDEN * 2 + 2 * _W_BYTES + 2 * (M_TOKENS * RANK * 2 + INTER * RANK * 2) + 3 * M_TOKENS * INTER * 2,
    # d_g and d_e once, up and gate weights + fp32 offset tables once, T and A^T, the mask source X, dX
    "gptq_lora_bwd_dx<linear> K=4096 N=14336+14336":
        2 * M_TOKENS * INTER * 2 + 2 * (_W_BYTES + (HIDDEN // GROUP) * INTER * 4) + 2 * (M_TOKENS * RANK * 2 + HIDDEN * RANK * 2)
        + 2 * M_TOKENS * HIDDEN * 2,
}

def proj_flops(M, K, N, r):
    """Algorithmic FLOPs of one projection, forward + backward: base fwd + base dX (frozen W has no
    dW) plus the LoRA terms (fwd, dA incl. T = dY B, dB incl. U = X A^T, dX-LoRA)."""
    return 4 * M * K * N + 2 * M * r * (3 * (K + N) + K)


def layer_flops(M):
    q = proj_flops(M, HIDDEN, N_HEADS * HEAD_DIM, RANK)
    kv = 2 * proj_flops(M, HIDDEN, N_KV * HEAD_DIM, RANK)
    o = proj_flops(M, N_HEADS * HEAD_DIM, HIDDEN, RANK)
    mlp = 2 * proj_flops(M, HIDDEN, INTER, RANK) + proj_flops(M, INTER, HIDDEN, RANK)
    return q + kv + o + mlp


def build_layer(device, seed=0):
    """attn (q/k/v/o) and mlp (gate/up/down) containers of LoraLinear(QuantLinear)."""
    import torch
    from fms_acceleration_peft import LoraLinear
    from fms_acceleration_peft.quantizer import quantize_linear

    gen = torch.Generator(device=device).manual_seed(seed)

    def lora_gptq(K, N, alpha, lseed):
        W = torch.randn(N, K, generator=gen, device=device) * 0.02
        ql = quantize_linear(W, GROUP).to(device)
        lin = LoraLinear(ql, RANK, alpha).to(device)
        g2 = torch.Generator().manual_seed(lseed)
        lin.lora_B["default"].weight.data.copy_(torch.randn(N, RANK, generator=g2) * 0.02)
        return lin

    attn, mlp = torch.nn.Module(), torch.nn.Module()
    attn.q_proj = lora_gptq(HIDDEN, N_HEADS * HEAD_DIM, ALPHA_ATTN, 1)
    attn.k_proj = lora_gptq(HIDDEN, N_KV * HEAD_DIM, ALPHA_ATTN, 2)
    attn.v_proj = lora_gptq(HIDDEN, N_KV * HEAD_DIM, ALPHA_ATTN, 3)
    attn.o_proj = lora_gptq(N_HEADS * HEAD_DIM, HIDDEN, ALPHA_ATTN, 4)
    mlp.gate_proj = lora_gptq(HIDDEN, INTER, ALPHA_MLP, 5)
    mlp.up_proj = lora_gptq(HIDDEN, INTER, ALPHA_MLP, 6)
    mlp.down_proj = lora_gptq(INTER, HIDDEN, ALPHA_MLP, 7)
    return attn, mlp


def make_step(attn, mlp, M, device, dtype):
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

    def step():
        for t in (x_attn, x_o, x_mlp, *params):
            t.grad = None
        Q, K, V = apply_lora_qkv(attn, x_attn)
        O = apply_lora_o_v2(attn.o_proj, x_o)
        Y = apply_lora_mlp(mlp, x_mlp)
        torch.autograd.backward([Q, K, V, O, Y], [dQ, dK, dV, dO, dY])

    return step


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

        def fwd(x2d, projs, mode=mod.FWD_LINEAR):
            K, Ns = projs[0]["w"].K, [p["w"].N for p in projs]
            flop = sum(2.0 * M * K * n + 2.0 * M * p["r"] * n for n, p in zip(Ns, projs))
            kind = "swiglu" if mode == mod.FWD_SWIGLU else "linear"
            return self._timed(f"gptq_lora_fwd<{kind}> K={K} N={'+'.join(map(str, Ns))}", flop, self._fwd, x2d, projs, mode)

        def bwd(projs, M_, K, mode=mod.BWD_LINEAR, e=None, g=None):
            Ns = [p["w"].N for p in projs]
            flop = sum(2.0 * M * K * n + 2.0 * M * p["r"] * K for n, p in zip(Ns, projs))
            kind = "swiglu" if mode == mod.BWD_SWIGLU else "linear"
            return self._timed(f"gptq_lora_bwd_dx<{kind}> K={K} N={'+'.join(map(str, Ns))}", flop, self._bwd, projs, M_, K, mode, e=e, g=g)

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


def cpu_baseline(sample_tokens: int):
    """The reference's UNFUSED path restated by the oracle (dense dequant inside the timed region,
    x @ W, PEFT-style LoRA, HF SwiGLU MLP, torch.autograd backward), fp32, on the host cores."""
    import torch

    from oracle import gptq as ogptq
    from oracle import lora as olora
    from fms_acceleration_peft.quantizer import rtn_quantize

    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    torch.set_num_threads(threads)
    M = sample_tokens
    gen = torch.Generator().manual_seed(0)

    def qproj(K, N, alpha, seed):
        buf = rtn_quantize(torch.randn(N, K, generator=gen) * 0.02, 4, GROUP)
        A, B = olora.make_lora(K, N, RANK, seed)
        return buf, A, B, alpha / RANK

    projs = {
        "q": qproj(HIDDEN, N_HEADS * HEAD_DIM, ALPHA_ATTN, 1), "k": qproj(HIDDEN, N_KV * HEAD_DIM, ALPHA_ATTN, 2),
        "v": qproj(HIDDEN, N_KV * HEAD_DIM, ALPHA_ATTN, 3), "o": qproj(N_HEADS * HEAD_DIM, HIDDEN, ALPHA_ATTN, 4),
        "gate": qproj(HIDDEN, INTER, ALPHA_MLP, 5), "up": qproj(HIDDEN, INTER, ALPHA_MLP, 6),
        "down": qproj(INTER, HIDDEN, ALPHA_MLP, 7),
    }
    x = torch.randn(M, HIDDEN, generator=gen)
    xo = torch.randn(M, N_HEADS * HEAD_DIM, generator=gen)
    d_h = torch.randn(M, HIDDEN, generator=gen)
    d_q = torch.randn(M, N_HEADS * HEAD_DIM, generator=gen)
    d_kv = torch.randn(M, N_KV * HEAD_DIM, generator=gen)

    def dense(name):
        buf, A, B, s = projs[name]
        W = ogptq.dequant_torch(buf["qweight"], buf["scales"], buf["qzeros"], buf["g_idx"])
        return W, A, B, s

    def step():
        olora.lora_qkv_autograd(x, [dense("q"), dense("k"), dense("v")], [d_q, d_kv, d_kv])
        olora.lora_w_autograd(xo, *dense("o"), d_h)
        olora.lora_mlp_autograd(x, dense("gate"), dense("up"), dense("down"), d_h)

    step()  # warm-up
    reps, t0 = 2, time.perf_counter()
    for _ in range(reps):
        step()
    dt = (time.perf_counter() - t0) / reps
    return {
        "value": M / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
        "sample": f"{M} of {M_TOKENS} tokens of the same layer (full-size weights, dequant inside the timed "
                  f"region), fp32, 1 warm-up + {reps} reps, {dt:.2f} s/rep",
        "gflops": layer_flops(M) / dt / 1e9,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--tokens", type=int, default=M_TOKENS)
    ap.add_argument("--cpu-sample-tokens", type=int, default=4096)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one device copy of 1 GiB (a kernel of known traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
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

    attn, mlp = build_layer(device)
    step = make_step(attn, mlp, M, device, dtype)
    if args.calibration_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=device).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps

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
        result["roofline"] = {
            "kernel": dominant, "bound": "mfma", "achieved": fl / ms / 1e9, "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s", "frac": fl / ms / 1e9 / PEAK_BF16_TFLOPS, "traffic": ROOFLINE_TRAFFIC_BYTES.get(dominant),
            "avg_launch_ms": ms, "algorithmic_flop_per_launch": fl,
            "algorithmic_bytes_per_launch": ALGORITHMIC_BYTES.get(dominant),
        }
        result["kernels"] = {k: {"ms": v[0], "tflops": v[1] / v[0] / 1e9, "launches_per_step": v[2] / args.steps}
                             for k, v in kt.items()}
    if not args.no_kernel_timing:
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
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.cpu_sample_tokens)
    print(json.dumps(result))


if __name__ == "__main__":
    main()

"""Writes tests/golden/hot_path_small.npz: small seeded inputs of every operator of the path together
with the outputs the CPU oracle computes for them.

    python tests/golden/make_fixtures.py

The file pins two things.  On the CPU: the oracle itself (tests/test_golden.py recomputes every entry
and, for the dequantised weights, re-derives sampled entries from the bit layout with plain loops).
On the GPU: the HIP kernels reproduce the stored outputs (tests/test_gpu_golden.py), bit for bit
where the result is a rounded exact product (dequantised weights, NF4, the SwiGLU rounding points)
and within the stated tolerance elsewhere.  16-bit tensors are stored as their bit patterns
(uint16); nothing in the file needs pickle.  The reference holds no numeric vectors for this path
(its parity tests load hub models), so these vectors come from the oracle, whose formulas are pinned
separately in tests/test_oracle_*.py.
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import cross_entropy as oce  # noqa: E402
from oracle import gptq as ogptq  # noqa: E402
from oracle import lora as olora  # noqa: E402
from oracle import nf4 as onf4  # noqa: E402
from oracle import norm_rope as onr  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hot_path_small.npz")


def bits(t: torch.Tensor) -> np.ndarray:
    """Bit pattern of a bf16 / fp16 tensor."""
    assert t.dtype in (torch.bfloat16, torch.float16)
    return t.contiguous().view(torch.int16).numpy().view(np.uint16).copy()


def randn(shape, seed, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def gptq_case(K, N, group_size, seed, act_order=False):
    W = randn((N, K), seed, 0.02).numpy()
    g_idx = ogptq.act_order_g_idx(K, group_size, seed=seed + 4) if act_order else None
    return ogptq.quantize_and_pack(W, group_size, g_idx=g_idx)


def build() -> dict:
    d = {}
    # ---- A: dequantisation (layout + one rounding), identity / act-order / v1 zero points -----------
    for tag, act in (("deq", False), ("deq_act", True)):
        b = gptq_case(256, 64, 64, seed=1, act_order=act)
        for k in ("qweight", "qzeros", "scales", "g_idx"):
            d[f"{tag}.{k}"] = b[k]
        d[f"{tag}.W_fp16"] = bits(ogptq.dequant(b["qweight"], b["scales"], b["qzeros"], b["g_idx"], out="fp16"))
        d[f"{tag}.W_bf16"] = bits(ogptq.dequant(b["qweight"], b["scales"], b["qzeros"], b["g_idx"], out="bf16"))
    d["deq.qzeros_v1"] = ogptq.to_v1_zeros(d["deq.qzeros"])

    # ---- B: one LoRA projection, forward and backward (fp64 autograd of the unfused graph) ----------
    K, N, r, s = 256, 64, 16, 2.0
    b = gptq_case(K, N, 64, seed=2)
    W = ogptq.dequant(b["qweight"], b["scales"], b["qzeros"], b["g_idx"], out="fp32").double()
    A, B = olora.make_lora(K, N, r, seed=3)
    A16, B16 = A.to(torch.bfloat16), B.to(torch.bfloat16)
    x, dy = randn((40, K), 4).to(torch.bfloat16), randn((40, N), 5).to(torch.bfloat16)
    y, dx, dA, dB = olora.lora_w_autograd(x.double(), W, A16.double(), B16.double(), s, dy.double())
    for k in ("qweight", "qzeros", "scales", "g_idx"):
        d[f"lora_w.{k}"] = b[k]
    d.update({"lora_w.A": bits(A16), "lora_w.B": bits(B16), "lora_w.s": np.float64(s), "lora_w.x": bits(x), "lora_w.dy": bits(dy),
              "lora_w.y": y.numpy(), "lora_w.dx": dx.numpy(), "lora_w.dA": dA.numpy(), "lora_w.dB": dB.numpy()})

    # ---- C: the SwiGLU MLP (gate / up / down), forward and backward --------------------------------
    H, I, r, s = 256, 128, 8, 2.0
    projs = []
    for i, (name, (Kp, Np)) in enumerate((("gate", (H, I)), ("up", (H, I)), ("down", (I, H)))):
        b = gptq_case(Kp, Np, 64, seed=10 + i)
        Wp = ogptq.dequant(b["qweight"], b["scales"], b["qzeros"], b["g_idx"], out="fp32").double()
        Ap, Bp = olora.make_lora(Kp, Np, r, seed=20 + i)
        Ap, Bp = Ap.to(torch.bfloat16), Bp.to(torch.bfloat16)
        for k in ("qweight", "qzeros", "scales", "g_idx"):
            d[f"mlp.{name}.{k}"] = b[k]
        d[f"mlp.{name}.A"], d[f"mlp.{name}.B"] = bits(Ap), bits(Bp)
        projs.append((Wp, Ap.double(), Bp.double(), s))
    x, dy = randn((48, H), 30).to(torch.bfloat16), randn((48, H), 31).to(torch.bfloat16)
    out, dx, grads, _ = olora.lora_mlp_autograd(x.double(), *projs, dy.double())
    d.update({"mlp.s": np.float64(s), "mlp.x": bits(x), "mlp.dy": bits(dy), "mlp.out": out.numpy(), "mlp.dx": dx.numpy()})
    for name, (ga, gb) in zip(("gate", "up", "down"), grads):
        d[f"mlp.{name}.dA"], d[f"mlp.{name}.dB"] = ga.numpy(), gb.numpy()

    # ---- D: SwiGLU rounding points (bit-exact) ------------------------------------------------------
    for dt, tag in ((torch.bfloat16, "bf16"), (torch.float16, "fp16")):
        e, g, dh = (randn((8, 128), 40 + i, 2.0).to(dt) for i in range(3))
        h = olora.swiglu_fwd(e, g)
        h2, d_g, d_e = olora.swiglu_bwd(dh, e, g)
        assert torch.equal(h, h2)
        d.update({f"swiglu.{tag}.e": bits(e), f"swiglu.{tag}.g": bits(g), f"swiglu.{tag}.dh": bits(dh),
                  f"swiglu.{tag}.h": bits(h), f"swiglu.{tag}.d_g": bits(d_g), f"swiglu.{tag}.d_e": bits(d_e)})

    # ---- E: NF4 with double-quantised statistics ---------------------------------------------------
    q = onf4.quantize(randn((64, 256), 50, 0.02).numpy())
    d.update({"nf4.packed": q["packed"], "nf4.absmax_q": q["absmax_q"], "nf4.absmax2": q["absmax2"], "nf4.code2": q["code2"],
              "nf4.offset": np.float32(q["offset"]), "nf4.shape": np.array(q["shape"]), "nf4.blocksize": np.int64(q["blocksize"]),
              "nf4.blocksize2": np.int64(q["blocksize2"]), "nf4.W_bf16": bits(onf4.dequant(q, "bf16")),
              "nf4.W_fp16": bits(onf4.dequant(q, "fp16"))})

    # ---- F: RMS norm, rotary embedding, cross entropy ----------------------------------------------
    x, w, dy = randn((6, 128), 60).to(torch.bfloat16), (1.0 + randn((128,), 61, 0.1)).to(torch.bfloat16), randn((6, 128), 62).to(torch.bfloat16)
    yv, rr = onr.rms_fwd(x, w, 1e-5)
    d.update({"rms.x": bits(x), "rms.w": bits(w), "rms.dy": bits(dy), "rms.y": bits(yv), "rms.r": rr.numpy(),
              "rms.dx": bits(onr.rms_bwd(dy, x, w, rr))})
    qv = randn((10, 2 * 64), 63).to(torch.bfloat16)
    ang = torch.arange(10, dtype=torch.float32)[:, None] * (1.0 / 10000 ** (torch.arange(32, dtype=torch.float32) / 32))[None]
    cos, sin = torch.cos(ang), torch.sin(ang)
    d.update({"rope.q": bits(qv), "rope.cos": cos.numpy(), "rope.sin": sin.numpy(),
              "rope.fwd": bits(onr.rope(qv, cos, sin, 2, 64)), "rope.bwd": bits(onr.rope(qv, cos, sin, 2, 64, backward=True))})
    logits, labels = randn((6, 200), 64, 3.0), torch.tensor([3, 199, -100, 0, 57, 120])
    loss, lse = oce.ce_fwd(logits, labels)
    dl = torch.tensor([0.5, 1.0, 2.0, 0.25, 1.5, 1.0])
    fl, fg = oce.liger_ce(logits, labels, 0.2, 0.1)
    d.update({"ce.logits": logits.numpy(), "ce.labels": labels.numpy(), "ce.loss": loss.numpy(), "ce.lse": lse.numpy(),
              "ce.dloss": dl.numpy(), "ce.grad": oce.ce_bwd(logits, labels, lse, dl).numpy(),
              "ce.fused_loss": fl.numpy(), "ce.fused_grad": fg.numpy()})
    return d


if __name__ == "__main__":
    fixtures = build()
    np.savez_compressed(OUT, **fixtures)
    print(f"wrote {OUT}: {len(fixtures)} arrays, {os.path.getsize(OUT) / 1024:.0f} KB")

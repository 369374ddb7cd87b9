"""Per-row cross entropy on the CPU -- test infrastructure only.

Restates kernels/unsloth/cross_entropy_loss.py of the reference: forward :22-73
(logsumexp = c + log sum exp(x - c), c = max x; loss = logsumexp - x[label], 0 for label -100) and
backward :138-190 (dlogits = dloss * (exp(x - logsumexp) - onehot(label)), zero rows for -100).
Pinned in tests/test_oracle_cross_entropy.py against torch.nn.functional.cross_entropy (library
code), its autograd gradient, and closed forms (uniform logits -> log V; gradient rows sum to 0).

`liger_ce` / `fused_linear_ce` restate fused_ops/liger_ce/cross_entropy.py:33-186 (loss and logits
gradient together, label smoothing, sum / mean over the valid labels) and
fused_ops/liger_ce/fused_linear_cross_entropy_loss.py:45-160 (lm_head matmul + that kernel, chunked
over tokens; the chunking only changes the order of the sums, so it is restated unchunked), pinned
against torch.nn.functional.cross_entropy(label_smoothing=...) and autograd through F.linear."""
from __future__ import annotations

import torch


def ce_fwd(logits: torch.Tensor, labels: torch.Tensor):
    x = logits.double()
    c = x.max(dim=-1, keepdim=True).values
    lse = (c + torch.log(torch.exp(x - c).sum(dim=-1, keepdim=True))).squeeze(-1)
    keep = (labels >= 0) & (labels < x.shape[1])  # -100 and any other label outside the vocabulary: ignored row
    picked = x.gather(1, torch.where(keep, labels, torch.zeros_like(labels)).unsqueeze(1)).squeeze(1)
    loss = torch.where(keep, lse - picked, torch.zeros_like(lse))
    return loss.float(), lse.float()


def ce_bwd(logits: torch.Tensor, labels: torch.Tensor, lse: torch.Tensor, dloss: torch.Tensor):
    x = logits.double()
    y = torch.exp(x - lse.double().unsqueeze(1))
    keep = (labels >= 0) & (labels < x.shape[1])
    onehot = torch.zeros_like(y)
    onehot[keep, labels[keep]] = 1.0
    dl = torch.where(keep, dloss.double(), torch.zeros_like(dloss.double())).unsqueeze(1)
    return (dl * (y - onehot)).to(logits.dtype)


def liger_ce(logits: torch.Tensor, labels: torch.Tensor, scale: float = 1.0, label_smoothing: float = 0.0,
             ignore_index: int = -100):
    """(losses [M], dlogits [M, V]) in float64, both already multiplied by `scale` (cross_entropy.py:97-186:
    softmax - eps everywhere, a further -(1 - ls) at the label; smoothed loss :163-165)."""
    x = logits.double()
    V = x.shape[1]
    c = x.max(dim=-1, keepdim=True).values
    d = torch.exp(x - c).sum(dim=-1, keepdim=True)
    lse = (c + torch.log(d)).squeeze(-1)
    eps = label_smoothing / V
    keep = labels != ignore_index
    safe = torch.where(keep, labels, torch.zeros_like(labels))
    picked = x.gather(1, safe.unsqueeze(1)).squeeze(1)
    loss = (1.0 - label_smoothing) * (lse - picked) + (label_smoothing * lse - eps * x.sum(dim=-1))
    g = torch.exp(x - c) / d - eps
    g[torch.arange(x.shape[0]), safe] -= 1.0 - label_smoothing
    loss = torch.where(keep, loss, torch.zeros_like(loss)) * scale
    g = torch.where(keep.unsqueeze(1), g, torch.zeros_like(g)) * scale
    return loss, g


def fused_linear_ce(x: torch.Tensor, weight: torch.Tensor, target: torch.Tensor, bias=None, ignore_index: int = -100,
                    label_smoothing: float = 0.0, reduction: str = "mean"):
    """(loss, dx, dweight, dbias) in float64 (fused_linear_cross_entropy_loss.py:84-158)."""
    xd, wd = x.double(), weight.double()
    logits = xd @ wd.t()
    if bias is not None:
        logits = logits + bias.double()
    n_valid = int((target != ignore_index).sum())
    scale = (1.0 / n_valid if n_valid > 0 else 0.0) if reduction == "mean" else 1.0
    losses, g = liger_ce(logits, target, scale, label_smoothing, ignore_index)
    return losses.sum(), g @ wd, g.t() @ xd, (g.sum(dim=0) if bias is not None else None)

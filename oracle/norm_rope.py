"""RMS layer norm and rotary embedding on the CPU -- test infrastructure only.

Restates kernels/unsloth/rms_layernorm.py and rope_embedding.py of the reference in torch:
  * rms_fwd   (:36-47; gemma :99-109): r = rsqrt(mean(x32^2) + eps); y = (x32 * r).to(w.dtype) * w,
              stored in x's dtype.  gemma: fp32 throughout, weight w + 1.
  * rms_bwd   (:71-86): dX = r/n * (n * dY_W - normed * sum(dY_W * normed)), dY_W = dY * W.
  * rope      (:36-65): (q1, q2) -> (q1 cos - q2 sin, q2 cos + q1 sin) per head half, sin negated
              for the backward pass; row m takes position m % seq_len.
Pinned in tests/test_oracle_norm_rope.py against independent statements of the same mathematics:
transformers' own LlamaRMSNorm / apply_rotary_pos_emb (installed library code, not the reference),
torch.autograd of those, and closed forms (unit-norm output, rotation preserving norms, backward of
a rotation = the inverse rotation).
"""
from __future__ import annotations

import torch


def rms_fwd(x: torch.Tensor, w: torch.Tensor, eps: float, gemma: bool = False):
    x32 = x.float()
    var = x32.pow(2).mean(dim=-1, keepdim=True)
    if gemma:
        r = 1.0 / torch.sqrt(var + eps)
        y = x32 * r * (w.float() + 1.0)
    else:
        r = torch.rsqrt(var + eps)
        y = (x32 * r).to(w.dtype) * w
    return y.to(x.dtype), r.squeeze(-1)


def rms_bwd(dy: torch.Tensor, x: torch.Tensor, w: torch.Tensor, r: torch.Tensor, gemma: bool = False):
    n = x.shape[-1]
    x32, dy32, w32 = x.float(), dy.float(), w.float()
    normed = x32 * r.unsqueeze(-1)
    dy_w = dy32 * (w32 + 1.0 if gemma else w32)
    rowsum = (dy_w * normed).sum(dim=-1, keepdim=True)
    return (r.unsqueeze(-1) / n * (n * dy_w - normed * rowsum)).to(dy.dtype)


def rope(q: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, n_heads: int, head_dim: int, backward: bool = False):
    """q [M, n_heads*head_dim]; cos / sin [rows, head_dim] (first half used).  fp32 arithmetic, one
    rounding to q's dtype."""
    M = q.shape[0]
    half = head_dim // 2
    pos = torch.arange(M) % cos.shape[0]
    c = cos.float()[pos, :half].unsqueeze(1)
    s = sin.float()[pos, :half].unsqueeze(1) * (-1.0 if backward else 1.0)
    qh = q.float().view(M, n_heads, head_dim)
    q1, q2 = qh[..., :half], qh[..., half:]
    out = torch.cat([q1 * c - q2 * s, q2 * c + q1 * s], dim=-1)
    return out.view(M, n_heads * head_dim).to(q.dtype)

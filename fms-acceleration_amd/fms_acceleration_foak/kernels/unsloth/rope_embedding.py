"""Rotary position embedding on the gfx950 kernel of libfmsa_hip (drop-in for
kernels/unsloth/rope_embedding.py of the reference: `Fast_RoPE_Embedding` :68-128 and
`fast_rope_embedding(Q, K, cos, sin, position_ids=None)` :132-135).

Like the reference the rotation is applied in place on the [batch, seq, heads, head_dim] view of the
projection output and ignores `position_ids` (:131): row m of the flattened tokens takes position
m % seq_len (:60-63, with seq_len <= cos.shape[0] allowed) of a 2-D cos / sin cache, however many
positions that cache holds; a 3-D cos / sin [batch, seq, head_dim] (what recent transformers pass)
is used row by row, which is the same thing for the default positions."""
import torch

import fmsa_hip


def _rows(t, batch, seq_len):
    """cos / sin as the [rows, head_dim] table the kernel indexes with (token row % rows):
    [P, d] or [1, P, d] with P >= seq_len -> its first seq_len rows (every batch entry starts again at
    position 0); [batch, seq_len, d] -> [batch * seq_len, d]."""
    while t.dim() > 2 and t.shape[0] == 1:
        t = t[0]
    if t.dim() == 2:
        if t.shape[0] < seq_len:
            raise ValueError("cos / sin cover fewer positions than the sequence")
        t = t[:seq_len]
    elif t.dim() == 3 and t.shape[0] == batch and t.shape[1] == seq_len:
        t = t.reshape(batch * seq_len, t.shape[-1])
    else:
        raise ValueError(f"cos / sin must be [positions, head_dim] or [batch, seq, head_dim], got {tuple(t.shape)}")
    return t if t.stride(1) == 1 else t.contiguous()


class Fast_RoPE_Embedding(torch.autograd.Function):
    @staticmethod
    def forward(ctx, Q, cos, sin):
        batch, seq_len, n_heads, head_dim = Q.shape
        cos, sin = _rows(cos, batch, seq_len), _rows(sin, batch, seq_len)
        Q2 = Q.view(batch * seq_len, n_heads * head_dim)
        fmsa_hip.rope_embedding_(Q2, cos, sin, n_heads, head_dim, backward=False)
        ctx.cos, ctx.sin = cos, sin
        return Q2.view(batch, seq_len, n_heads, head_dim)

    @staticmethod
    def backward(ctx, dY):
        batch, seq_len, n_heads, head_dim = dY.shape
        dY2 = dY.reshape(batch * seq_len, n_heads * head_dim)  # reshape: dY may be non-contiguous (:111-112)
        dY2 = dY2 if dY2.stride(1) == 1 else dY2.contiguous()
        fmsa_hip.rope_embedding_(dY2, ctx.cos, ctx.sin, n_heads, head_dim, backward=True)
        return dY2.view(batch, seq_len, n_heads, head_dim), None, None


# Q / K that left a fused projection already rotated (apply_lora_qkv_rope behind the `<arch>-qkvo` rule): keyed by the
# address of Q's storage, holding both tensors so that the address cannot be reused while the entry waits for the
# attention's apply_rotary_pos_emb call, which consumes it.
_ROTATED = {}


def mark_rotated(Q, K):
    key = Q.untyped_storage().data_ptr()
    _ROTATED[key] = (Q, K)
    return key


def unmark_rotated(key) -> bool:
    """Drops a mark that was never consumed; True if it was still there."""
    return _ROTATED.pop(key, None) is not None


def fast_rope_embedding(Q, K, cos, sin, position_ids=None, unsqueeze_dim=1):
    if _ROTATED:
        done = _ROTATED.pop(Q.untyped_storage().data_ptr(), None)
        if done is not None:
            if done[1].untyped_storage().data_ptr() != K.untyped_storage().data_ptr():
                raise RuntimeError("fast_rope_embedding: Q comes rotated from the fused projection, K does not")
            return Q, K
    Q = Fast_RoPE_Embedding.apply(Q.transpose(1, 2), cos, sin).transpose(1, 2)
    K = Fast_RoPE_Embedding.apply(K.transpose(1, 2), cos, sin).transpose(1, 2)
    return Q, K

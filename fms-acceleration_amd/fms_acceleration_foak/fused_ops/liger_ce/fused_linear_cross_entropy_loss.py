"""Loss head that never holds the full [tokens, vocabulary] logits: lm_head matmul + cross entropy,
chunk of tokens by chunk of tokens, with the gradient formed during the forward pass (reference:
fused_ops/liger_ce/fused_linear_cross_entropy_loss.py:45-160 forward, :163-207 backward,
:209-276 autograd function and loss module, :278-417 `lce_forward`).

Per chunk: `logits = x_chunk @ W^T (+ bias)` through the library GEMM in the activation dtype, then ONE
launch of `fmsa_cross_entropy_fused` turns the chunk into its own gradient in place (fp32 arithmetic on the
16-bit logits, one rounding on the way back) and writes the per-token losses, then `dX_chunk = dlogits @ W`
(and `dW += dlogits^T @ x_chunk`, `dbias += sum dlogits` when those are trainable).

Differences from the reference, on purpose:
  * the mean reduction multiplies by 1 / (number of valid labels of the whole batch) inside the kernel, read
    from device memory: one rounding instead of the reference's divide-by-chunk-count, round, multiply by
    chunk-count / total, round again (:120-137), and no host synchronisation per chunk (:100);
  * chunks are as large as `MAX_CHUNK_BYTES` of logits allows (the reference sizes them so that a chunk of
    logits is no larger than the hidden states, :66-70, which at a 128k vocabulary means 256-token GEMMs);
  * the backward multiplies by grad_output unconditionally instead of synchronising to compare it with 1
    (:167).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch.nn import CrossEntropyLoss

MAX_CHUNK_BYTES = 1 << 30


def _chunk_rows(BT: int, V: int, itemsize: int) -> int:
    """Tokens per chunk: the largest power of two whose logits fit MAX_CHUNK_BYTES."""
    budget_rows = max(MAX_CHUNK_BYTES // (V * itemsize), 1)
    return min(BT, 1 << (budget_rows.bit_length() - 1))


def fused_linear_cross_entropy_forward(_input, weight, target, bias=None, ignore_index=-100, label_smoothing=0.0,
                                       reduction="mean"):
    """(loss, grad_input, grad_weight | None, grad_bias | None); `loss` is an fp32 scalar tensor."""
    import fmsa_hip  # pylint: disable=import-outside-toplevel

    if reduction not in ("mean", "sum"):
        raise ValueError(f"reduction must be 'mean' or 'sum', got {reduction!r}")
    if not _input.is_cuda:
        raise RuntimeError("the fused linear cross entropy runs on the GPU kernels only")
    dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else _input.dtype
    BT, H = _input.shape
    V = weight.shape[0]
    x = _input.detach()
    x = (x if x.dtype == dtype else x.to(dtype)).contiguous()
    w = weight.detach()
    w = (w if w.dtype == dtype else w.to(dtype)).contiguous()
    b = None if bias is None else bias.detach().to(dtype)
    target = target.contiguous()
    rows = _chunk_rows(BT, V, x.element_size())

    grad_input = torch.empty_like(x)
    grad_weight = torch.zeros_like(weight) if weight.requires_grad else None
    grad_bias = torch.zeros(V, dtype=torch.float32, device=x.device) if bias is not None else None
    loss_1d = torch.empty(BT, dtype=torch.float32, device=x.device)
    scale = None
    if reduction == "mean":
        n_valid = (target != ignore_index).sum().to(torch.float32)
        scale = torch.where(n_valid > 0, 1.0 / n_valid, torch.zeros_like(n_valid)).reshape(1)
    logits = torch.empty((rows, V), dtype=dtype, device=x.device)

    for start in range(0, BT, rows):
        end = min(start + rows, BT)
        xc, lc = x[start:end], logits[: end - start]
        if b is None:
            torch.mm(xc, w.t(), out=lc)
        else:
            torch.addmm(b, xc, w.t(), out=lc)
        fmsa_hip.cross_entropy_fused_(lc, target[start:end], scale, label_smoothing, ignore_index, losses_out=loss_1d[start:end])
        torch.mm(lc, w, out=grad_input[start:end])
        if grad_weight is not None:
            if grad_weight.dtype == dtype:
                grad_weight.addmm_(lc.t(), xc)
            else:
                grad_weight.add_(torch.mm(lc.t(), xc))
        if grad_bias is not None:
            grad_bias.add_(lc.sum(dim=0, dtype=torch.float32))
    if grad_bias is not None:
        grad_bias = grad_bias.to(bias.dtype)
    return loss_1d.sum(), grad_input.to(_input.dtype), grad_weight, grad_bias


def fused_linear_cross_entropy_backward(grad_output, grad_input, grad_weight, grad_bias):
    scale = lambda g: None if g is None else g * grad_output.to(g.dtype)  # noqa: E731
    return scale(grad_input), scale(grad_weight), scale(grad_bias)


class LigerFusedLinearCrossEntropyFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, _input, weight, target, bias=None, ignore_index=-100, label_smoothing=0.0, reduction="mean"):
        loss, grad_input, grad_weight, grad_bias = fused_linear_cross_entropy_forward(
            _input, weight, target, bias, ignore_index, label_smoothing, reduction)
        ctx.has = (grad_weight is not None, grad_bias is not None)
        ctx.save_for_backward(grad_input, *(g for g in (grad_weight, grad_bias) if g is not None))
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        saved = list(ctx.saved_tensors)
        grad_input = saved.pop(0)
        grad_weight = saved.pop(0) if ctx.has[0] else None
        grad_bias = saved.pop(0) if ctx.has[1] else None
        grad_input, grad_weight, grad_bias = fused_linear_cross_entropy_backward(grad_output, grad_input, grad_weight, grad_bias)
        return grad_input, grad_weight, None, grad_bias, None, None, None


class LigerFusedLinearCrossEntropyLoss(CrossEntropyLoss):
    def forward(self, lin_weight, _input, target, bias=None):  # pylint: disable=arguments-differ
        return LigerFusedLinearCrossEntropyFunction.apply(
            _input, lin_weight, target, bias, self.ignore_index, self.label_smoothing, self.reduction)


def lce_forward(self, input_ids=None, attention_mask=None, position_ids=None, past_key_values=None, inputs_embeds=None,
                labels: Optional[torch.LongTensor] = None, use_cache=None, logits_to_keep=0, **kwargs):
    """Forward of a `...ForCausalLM` with the loss head fused while training (reference :278-417).  Outside
    training, or without labels, it is the stock forward (lm_head on the kept positions + `loss_function`).

    The next-token shift is done on the labels (last position of each sequence ignored), so the hidden
    states are used as they are instead of being copied without their last position (:361-362).  A model
    with `config.logits_scaling` (granite) has its hidden states divided by it before the head, which the
    reference leaves out of the training branch (:386-387).  `num_items_in_batch`, when the trainer passes
    it, replaces the count of valid labels as the denominator, as in transformers' own causal-LM loss."""
    from transformers.modeling_outputs import CausalLMOutputWithPast  # pylint: disable=import-outside-toplevel

    return_dict = kwargs.pop("return_dict", None)
    outputs = self.model(input_ids=input_ids, attention_mask=attention_mask, position_ids=position_ids,
                         past_key_values=past_key_values, inputs_embeds=inputs_embeds, use_cache=use_cache, **kwargs)
    hidden_states = outputs[0]
    loss, logits = None, None
    if self.training and labels is not None:
        shift_labels = kwargs.get("shift_labels")
        if shift_labels is None:
            shift_labels = torch.nn.functional.pad(labels, (0, 1), value=-100)[..., 1:]
        shift_labels = shift_labels.reshape(-1).to(hidden_states.device)
        hidden = hidden_states.reshape(-1, hidden_states.shape[-1])
        scaling = getattr(self.config, "logits_scaling", None)
        if scaling not in (None, 1, 1.0):
            hidden = hidden / scaling
        num_items = kwargs.get("num_items_in_batch")
        lce = LigerFusedLinearCrossEntropyLoss(reduction="mean" if num_items is None else "sum")
        loss = lce(self.lm_head.weight, hidden, shift_labels, self.lm_head.bias)
        if num_items is not None:
            loss = loss / (num_items.to(loss.device) if torch.is_tensor(num_items) else num_items)
    else:
        slice_indices = slice(-logits_to_keep, None) if isinstance(logits_to_keep, int) else logits_to_keep
        logits = self.lm_head(hidden_states[:, slice_indices, :])
        scaling = getattr(self.config, "logits_scaling", None)
        if scaling not in (None, 1, 1.0):
            logits = logits / scaling
        if labels is not None:
            loss = self.loss_function(logits=logits, labels=labels, vocab_size=self.config.vocab_size, **kwargs)
    if return_dict is False:
        out = (logits,) + tuple(outputs[1:])
        return (loss,) + out if loss is not None else out
    return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=outputs.past_key_values,
                                  hidden_states=outputs.hidden_states, attentions=outputs.attentions)

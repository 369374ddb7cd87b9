"""Cross-entropy loss on the gfx950 kernels of libfmsa_hip (drop-in for
kernels/unsloth/cross_entropy_loss.py of the reference: `Fast_CrossEntropyLoss` :195-262,
`fast_cross_entropy_loss` :265-282, `FastCrossEntropyLoss` :285-296, `FastForCausalLMLoss` :302-327,
`replace_custom_loss_when_triggered` :330-346).  As in the reference the backward overwrites the
saved logits with their gradient (:259), so a graph can be back-propagated once."""
from typing import Type

import torch

import fmsa_hip


class Fast_CrossEntropyLoss(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, labels):
        if logits.stride(1) != 1:
            logits = logits.contiguous()
        labels = labels.to(torch.int64).contiguous()
        losses, logsumexp = fmsa_hip.cross_entropy_fwd(logits, labels)
        ctx.save_for_backward(logits, logsumexp, labels)
        return losses

    @staticmethod
    def backward(ctx, dlosses):
        logits, logsumexp, labels = ctx.saved_tensors
        fmsa_hip.cross_entropy_bwd_(logits, dlosses.float(), logsumexp, labels)
        return logits, None, None


def fast_cross_entropy_loss(logits, labels):
    """logits (batch, seq_len, vocab), labels (batch, seq_len) -> mean loss over labels != -100."""
    batch, seq_len, d = logits.shape
    assert labels.shape == (batch, seq_len)
    loss = Fast_CrossEntropyLoss.apply(logits.view(batch * seq_len, d), labels.view(-1))
    n_items = torch.count_nonzero(labels != -100)
    return loss.sum() / n_items


class FastCrossEntropyLoss(torch.nn.CrossEntropyLoss):
    def __init__(self):
        super().__init__()

    def forward(self, input, target):  # pylint: disable=redefined-builtin
        loss = Fast_CrossEntropyLoss.apply(input, target)
        n_items = torch.count_nonzero(target != -100)
        return loss.sum() / n_items


def FastForCausalLMLoss(logits, labels, vocab_size: int, num_items_in_batch: int = None, ignore_index: int = -100,
                        shift_labels=None, **kwargs):
    """Counterpart of transformers.loss.loss_utils.ForCausalLMLoss on the fused kernel."""
    logits = logits.float()
    if shift_labels is None:
        labels = labels.to(logits.device)
        shift_logits = logits[..., :-1, :].contiguous()
        shift_labels = labels[..., 1:].contiguous()
    else:  # newer transformers pass the labels already shifted, against the unshifted logits
        shift_logits = logits.contiguous()
    shift_logits = shift_logits.view(-1, vocab_size)
    shift_labels = shift_labels.reshape(-1).to(shift_logits.device)
    assert ignore_index == -100, "FastForCausalLMLoss currently supports only hardcoded ignore index -100."
    loss = Fast_CrossEntropyLoss.apply(shift_logits, shift_labels)
    if num_items_in_batch is not None:
        n_items = num_items_in_batch
    else:
        n_items = torch.count_nonzero(shift_labels != -100)
    return loss.sum() / n_items


def replace_custom_loss_when_triggered(module_cls: Type, custom_loss_type: str):
    """A trigger that performs the replacement itself: registers FastForCausalLMLoss under
    `custom_loss_type` in transformers' LOSS_MAPPING and points the model at it."""

    def _trigger(mod):
        if isinstance(mod, module_cls) and hasattr(mod, "loss_function"):
            from transformers.loss.loss_utils import LOSS_MAPPING  # pylint: disable=import-outside-toplevel

            LOSS_MAPPING[custom_loss_type] = FastForCausalLMLoss
            mod.loss_type = custom_loss_type
            return True
        return False

    return _trigger

"""RMS layer norm on the gfx950 kernels of libfmsa_hip (drop-in for
kernels/unsloth/rms_layernorm.py of the reference: `Fast_RMS_Layernorm` :112-181 and
`fast_rms_layernorm(layernorm, X, gemma=False)` :184-189).  As in the reference the weight gets no
gradient (:181 returns None for it) and the backward writes dX over dY (:171-180)."""
import torch

import fmsa_hip


class Fast_RMS_Layernorm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, X, W, eps, gemma=False):
        shape = X.shape
        X2 = X.reshape(-1, shape[-1])
        if X2.stride(1) != 1:
            X2 = X2.contiguous()
        Wc = W.detach()
        Wc = Wc if Wc.is_contiguous() else Wc.contiguous()
        Y, r = fmsa_hip.rms_layernorm_fwd(X2, Wc, eps, gemma)
        ctx.gemma = gemma
        ctx.save_for_backward(X2, Wc, r)
        return Y.view(*shape)

    @staticmethod
    def backward(ctx, dY):
        shape = dY.shape
        X2, W, r = ctx.saved_tensors
        dY2 = dY.reshape(-1, shape[-1])
        if dY2.stride(1) != 1 or dY2.dtype != X2.dtype:
            dY2 = dY2.to(X2.dtype).contiguous()
        dX = fmsa_hip.rms_layernorm_bwd(dY2, X2, W, r, ctx.gemma)
        return dX.view(*shape), None, None, None


def fast_rms_layernorm(layernorm, X, gemma=False):
    W = layernorm.weight
    eps = layernorm.variance_epsilon if hasattr(layernorm, "variance_epsilon") else layernorm.eps
    return Fast_RMS_Layernorm.apply(X, W, eps, gemma)

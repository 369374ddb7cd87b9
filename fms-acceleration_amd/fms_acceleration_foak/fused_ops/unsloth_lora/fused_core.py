"""What the GPTQ- and the NF4-flavoured fused LoRA functions share: the per-projection operand
bundle, adapter stacking, and the forward / backward bodies of LoRA_W, LoRA_QKV and LoRA_MLP on the
libfmsa_hip kernels (reference: fused_ops/unsloth_lora/gptq/fast_lora.py:143-435, 466-711, 742-846
and its bnb twin fused_ops/unsloth_lora/bnb/fast_lora.py).  The two flavours differ only in how a
projection's frozen base weight is described to the kernels (`_Proj.w`, an affine GPTQ weight or a
code-book weight) and in the argument lists of their autograd functions.

  forward   U = Xd A^T                 (fmsa_lora_down, streams X once)
            Y = X deq(W) + s U B^T     (fmsa_gptq_lora_fwd: nibble unpack in registers -> MFMA,
                                        LoRA / bias / SwiGLU in the epilogue)
  backward  T = dY B                   (fmsa_lora_down)
            dA = s T^T Xd, dB = s dY^T U   (fmsa_lora_grad, deterministic)
            dX = dY deq(W)^T + (Xd != 0) * T (s A)      (fmsa_gptq_lora_bwd_dx)
"""
from __future__ import annotations

import torch

import fmsa_hip


# ----------------------------------------------------------------------------------------------
# small helpers shared by the three functions
# ----------------------------------------------------------------------------------------------
def _act_dtype(X):
    if X.dtype in (torch.float16, torch.bfloat16):
        return X.dtype
    if torch.is_autocast_enabled():
        return torch.get_autocast_gpu_dtype()
    raise TypeError(f"fused GPTQ-LoRA ops compute in float16 / bfloat16, got {X.dtype} outside autocast")


def _as2d(X, dtype):
    X2 = X.reshape(-1, X.shape[-1])
    if X2.dtype != dtype:
        X2 = X2.to(dtype)
    return X2 if X2.is_contiguous() else X2.contiguous()


def _apply_dropout(X2, dropout):
    """Post-dropout input of the LoRA branch (matmul_lora :155-163).  Returns X2 itself when the
    module is absent or an identity."""
    if dropout is None or isinstance(dropout, torch.nn.Identity):
        return X2
    if isinstance(dropout, torch.Tensor):
        return X2 * dropout.reshape(X2.shape).to(X2.dtype)
    Xd = dropout(X2)
    return Xd if Xd.is_contiguous() else Xd.contiguous()


def _same(a, b):
    """Same memory seen the same way (tensors that went through save_for_backward come back as new
    objects)."""
    return a is b or (a is not None and b is not None and a.data_ptr() == b.data_ptr()
                      and a.shape == b.shape and a.stride() == b.stride())


def _dropped_inputs(X2, projs, dropouts):
    """Post-dropout input of each projection's LoRA branch; X2 itself (the same object) where no
    dropout applies, which is what lets projections share passes over it."""
    return [_apply_dropout(X2, d) if p.r else X2 for p, d in zip(projs, dropouts)]


class _Proj:
    """One projection's operands in the forms the kernels take."""

    def __init__(self, w, bias, A, B, S, dtype):
        self.w = w  # prepared weight: .struct (C-ABI view), .K, .N, .perm (act-order) and .nsz
        self.bias = None if bias is None else bias.to(dtype)
        self.A_param, self.B_param = A, B
        self.r = 0 if A is None else A.shape[0]
        self.s = 0.0 if S is None else float(S)
        self.dtype = dtype
        # activation-type copies of the adapter in the four layouts the kernels read (one launch,
        # see pack): A [r, K], A^T [K, r], B [N, r], B^T [r, N]
        self.A = self.At = self.B = self.Bt = None
        # An MLP whose down projection is act-order runs its intermediate dimension in that projection's
        # kernel order: gate / up get re-ordered output columns (col_perm: column n' is the model's column
        # col_perm[n']), down takes its input as it comes (input_ordered).
        self.col_perm = None
        self.input_ordered = False

    def with_columns(self, col_perm, key):
        """This projection producing its output columns in the order col_perm (before pack)."""
        q = _Proj(self.w.with_columns(col_perm, key), None, self.A_param, self.B_param, self.s if self.r else None, self.dtype)
        q.bias = None if self.bias is None else self.bias.index_select(0, col_perm)
        q.col_perm = col_perm
        return q

    def with_ordered_input(self):
        """This projection reading an input whose columns are already in its kernel order (before pack)."""
        q = _Proj(self.w, None, self.A_param, self.B_param, self.s if self.r else None, self.dtype)
        q.bias, q.input_ordered = self.bias, True
        return q

    def after_pack(self):
        if self.r and self.col_perm is not None:
            self.B, self.Bt = self.B.index_select(0, self.col_perm), self.Bt.index_select(1, self.col_perm)
        if self.r and self.input_ordered:
            self.A = self.A.index_select(1, self.w.perm.long())  # U = h' A'^T on the ordered input

    def natural_grads(self, dA, dB):
        """Adapter gradients back in the layouts of the parameters."""
        if dB is not None and self.col_perm is not None:
            dB = dB.index_select(0, self.w.col_inv)
        if dA is not None and self.input_ordered:
            dA = dA.index_select(1, self.w.row_inv)
        return dA, dB

    def pack(self, A16_out=None):
        _pack_projs([(self, A16_out)])

    # the kernels walk K in the repacked order for act-order weights
    def to_kernel_order(self, X2):
        return X2 if self.w.perm is None or self.input_ordered else fmsa_hip.permute_cols(X2, self.w.perm, gather=True)

    def from_kernel_order(self, dXp):
        return dXp if self.w.perm is None or self.input_ordered else fmsa_hip.permute_cols(dXp, self.w.perm, gather=False)

    def fwd_dict(self, U, interleaved=False):
        return {"w": self.w.struct_interleaved if interleaved else self.w.struct, "U": U, "B": self.B, "bias": self.bias,
                "r": self.r, "s": self.s}

    def bwd_dict(self, dY2, T, mask_src, permuted=None):
        """`permuted`: dict shared by the projections of one launch, so that a mask source they have in common
        is brought into kernel order once."""
        At = None
        if self.r:
            At = self.At  # [K, r]
            if self.w.perm is not None:
                At = At[self.w.perm.long()].contiguous()
                if mask_src is not None and not self.input_ordered:
                    key = (id(mask_src), self.w.perm_key)
                    if permuted is not None and key in permuted:
                        mask_src = permuted[key][1]
                    else:
                        pm = fmsa_hip.permute_cols(mask_src, self.w.perm, gather=True)
                        if permuted is not None:
                            permuted[key] = (mask_src, pm)  # holds the source too: its id stays taken
                        mask_src = pm
        qweight_t, scale_f32, negzp_f16 = self.w.twin
        return {"w": self.w.struct, "nsz": self.w.nsz, "dY": dY2, "T": T, "At": At, "mask_src": mask_src if self.r else None,
                "r": self.r, "s": self.s, "qweight_t": qweight_t, "scale_f32": scale_f32, "negzp_f16": negzp_f16}

    def lora_grads(self, T, Xd, U, dY2):
        """dA [r, K] = s T^T Xd and dB [N, r] = s dY^T U, in the dtypes of the parameters."""
        if not self.r:
            return None, None
        dA, dB = fmsa_hip.lora_grad_batch([(T, Xd, self.s, False, self.A_param.dtype),
                                           (U, dY2, self.s, True, self.B_param.dtype)])
        return dA, dB

    def t_and_grads(self, Xd, U, dY2):
        """(T = dY B, dA, dB).  Where it pays, T and dB come from one pass over dY and dA from a second launch
        that reads T; otherwise T from its own pass and both gradients from one launch."""
        if not self.r:
            return None, None, None
        if not _fuse_t([self], [dY2]):
            T = fmsa_hip.lora_down(dY2, self.Bt)
            return (T,) + self.lora_grads(T, Xd, U, dY2)
        T = torch.empty((dY2.shape[0], self.r), dtype=dY2.dtype, device=dY2.device)
        (dB,) = fmsa_hip.lora_grad_batch([(U, dY2, self.s, True, self.B_param.dtype, self.Bt, T)])
        (dA,) = fmsa_hip.lora_grad_batch([(T, Xd, self.s, False, self.A_param.dtype)])
        return T, dA, dB


FUSE_T_MIN_BYTES = 96 << 20


def _fuse_t(projs, dYs):
    """Whether T_p = dY_p B_p should come out of the dB launch (one pass over dY_p instead of two).  The
    dependent dA launch then cannot share the dB launch any more, which costs about 15 us of launch ramp
    and tail: measured to pay from about 100 MB of dY (q, k, v together; gate and up), not for one
    4096-wide projection."""
    if any(p.r > fmsa_hip.LORA_GRAD_T_MAX_RANK for p in projs):
        return False
    return sum(dY.numel() * dY.element_size() for dY in dYs) >= FUSE_T_MIN_BYTES


def _pack_projs(items):
    """items: (projection, A16_out or None).  One launch packs the adapters of all of them."""
    live = [(p, out) for p, out in items if p.r]
    if live:
        packed = fmsa_hip.lora_pack_batch([(p.A_param, p.B_param, out) for p, out in live], live[0][0].dtype)
        for (p, _), quad in zip(live, packed):
            p.A, p.At, p.B, p.Bt = quad
            p.after_pack()


class _Stack:
    """Adapters of projections that read the same (post-dropout) input, stacked: one pass over the
    input gives all their U = Xd A^T (forward) and, with equal scalings, all their dA = s T^T Xd
    (backward).  `cols[i]` is the column range of projection i inside the stacked [M, R] matrices."""

    def __init__(self, projs, dtype, device, also=()):
        self.R = sum(p.r for p in projs)
        self.K = projs[0].w.K
        self.A_cat = torch.empty((self.R, self.K), dtype=dtype, device=device)
        self.cols, o, items = [], 0, []
        for p in projs:
            self.cols.append((o, o + p.r))
            items.append((p, self.A_cat[o : o + p.r]))
            o += p.r
        _pack_projs(items + [(p, None) for p in also])
        self.same_s = all(p.s == projs[0].s for p in projs)


def _one_order(projs):
    """All projections walk K in the same order (none act-order, or act-order with one shared permutation, which
    is what GPTQ gives projections quantised on the same input): they can share launches."""
    return all(p.w.perm_key == projs[0].w.perm_key for p in projs)


def _pack_group(projs, Xds, dtype, also=()):
    """Packs the adapters of a group of projections (and of the projections in `also`, in the same
    launch); returns a _Stack when the group can share passes over the input (all adapted, one
    post-dropout input, total rank <= 128; the rank-r kernels work in the model's own K order, so act-order
    weights do not matter here)."""
    live = [p for p in projs if p.r]
    if (len(live) == len(projs) and len(projs) > 1 and all(_same(Xd, Xds[0]) for Xd in Xds)
            and sum(p.r for p in projs) <= 128):
        return _Stack(projs, dtype, Xds[0].device, also)
    _pack_projs([(p, None) for p in list(projs) + list(also)])
    return None


def _lora_down_all(projs, Xds, stack):
    if stack is not None:
        U_cat = fmsa_hip.lora_down(Xds[0], stack.A_cat)
        return [U_cat[:, a:b] for a, b in stack.cols]
    return [fmsa_hip.lora_down(Xd, p.A) if p.r else None for p, Xd in zip(projs, Xds)]


def _rope_in_epilogue(projs, rope, dtype):
    """Whether the forward kernel can apply the rotary embedding itself (fmsa_gptq_lora_fwd_rope): group sizes and
    K in whole 64-wide stages, heads that do not straddle its 256-column tiles, tables of the activation type or
    fp32 whose rows start on 16-byte boundaries."""
    cos2d, sin2d, head_dim, mask = rope
    K = projs[0].w.K
    esz = cos2d.element_size()
    return (K % 64 == 0 and head_dim % 16 == 0 and 256 % head_dim == 0
            and cos2d.dtype in (dtype, torch.float32) and sin2d.dtype == cos2d.dtype
            and cos2d.stride() == sin2d.stride() and (cos2d.stride(0) * esz) % 16 == 0
            and cos2d.data_ptr() % 16 == 0 and sin2d.data_ptr() % 16 == 0
            and all(p.w.group_size % 64 == 0 for p in projs)
            and all(p.w.N % head_dim == 0 for i, p in enumerate(projs) if (mask >> i) & 1))


def _interleaved(projs, dtype):
    """Whether a forward launch over these projections reads the interleaved copies of their weights (the kernel's
    packed-half unpack: fp16 activations, GPTQ weights with groups in whole stages; all projections or none)."""
    return all(getattr(p.w, "interleaved_ok", lambda _: False)(dtype) for p in projs)


def _linear_forward(projs, X2, Xds, stack=None, rope=None):
    """Y_p = X deq(W_p) + s U_p B_p^T for projections sharing X2.  One launch when the weights walk K in one
    order (on X in that order); otherwise one launch per projection on its own column-permuted copy of X.
    rope = (cos2d, sin2d, head_dim, mask): the projections named by the mask leave with the rotary embedding
    applied, in the kernel's epilogue where it can, by the in-place kernel otherwise."""
    Us = _lora_down_all(projs, Xds, stack)
    fused_rope = rope is not None and _rope_in_epilogue(projs, rope, X2.dtype)
    if _one_order(projs):
        il = not fused_rope and _interleaved(projs, X2.dtype)  # the rotating flavours read the checkpoint's nibble order
        outs = fmsa_hip.gptq_lora_fwd(projs[0].to_kernel_order(X2), [p.fwd_dict(U, il) for p, U in zip(projs, Us)],
                                      rope=rope if fused_rope else None)
    else:
        outs = []
        for i, (p, U) in enumerate(zip(projs, Us)):
            r1 = (rope[0], rope[1], rope[2], 1) if fused_rope and (rope[3] >> i) & 1 else None
            il = r1 is None and _interleaved([p], X2.dtype)
            outs.append(fmsa_hip.gptq_lora_fwd(p.to_kernel_order(X2), [p.fwd_dict(U, il)], rope=r1)[0])
    if rope is not None and not fused_rope:
        cos2d, sin2d, head_dim, mask = rope
        for i, (p, y) in enumerate(zip(projs, outs)):
            if (mask >> i) & 1:
                fmsa_hip.rope_embedding_(y, cos2d, sin2d, p.w.N // head_dim, head_dim, backward=False)
    return outs, Us


def _adapter_grads(projs, dYs, Xds, Us, stack):
    """(Ts, [(dA, dB)]) of projections sharing their input.  T_p = dY_p B_p; dA_p = s T_p^T Xd;
    dB_p = s dY_p^T U_p.  With a stack the T's are written side by side and one pass over Xd gives
    every dA."""
    if stack is not None:
        M = dYs[0].shape[0]
        T_cat = torch.empty((M, stack.R), dtype=dYs[0].dtype, device=dYs[0].device)
        Ts = [T_cat[:, a:b] for a, b in stack.cols]
        # one launch: every dB, and with it (same pass over dY) every T; a second one: every dA, which reads the T's
        stacked_dA = stack.same_s and all(p.A_param.dtype == projs[0].A_param.dtype for p in projs)
        dA_jobs = ([(T_cat, Xds[0], projs[0].s, False, projs[0].A_param.dtype)] if stacked_dA else
                   [(T, Xds[0], p.s, False, p.A_param.dtype) for p, T in zip(projs, Ts)])
        if _fuse_t(projs, dYs):
            dBs = fmsa_hip.lora_grad_batch([(U, dY, p.s, True, p.B_param.dtype, p.Bt, T)
                                            for p, dY, U, T in zip(projs, dYs, Us, Ts)])
            dAs = fmsa_hip.lora_grad_batch(dA_jobs)
        else:
            for p, dY, T in zip(projs, dYs, Ts):
                fmsa_hip.lora_down(dY, p.Bt, out=T)
            outs = fmsa_hip.lora_grad_batch(dA_jobs + [(U, dY, p.s, True, p.B_param.dtype) for p, dY, U in zip(projs, dYs, Us)])
            dAs, dBs = outs[: len(dA_jobs)], outs[len(dA_jobs) :]
        if stacked_dA:
            dAs = [dAs[0][a:b] for a, b in stack.cols]
        return Ts, list(zip(dAs, dBs))
    Ts, grads = [], []
    for p, dY, Xd, U in zip(projs, dYs, Xds, Us):
        T, dA, dB = p.t_and_grads(Xd, U, dY)
        Ts.append(T)
        grads.append((dA, dB))
    return Ts, grads


def _linear_backward_dx(projs, dYs, Ts, Xds, M, K):
    """dX = sum_p dY_p deq(W_p)^T + mask (.) sum_p s_p T_p A_p.  One launch when the projections share
    one mask source (no dropout, or one dropout module applied once) and one K order; otherwise
    one launch per projection (each with its own mask / column order) and a sum."""
    masks = [Xd for p, Xd in zip(projs, Xds) if p.r]
    one_mask = all(_same(m, masks[0]) for m in masks)
    if one_mask and _one_order(projs):
        permuted = {}
        dXk = fmsa_hip.gptq_lora_bwd_dx([p.bwd_dict(dY, T, Xd, permuted) for p, dY, T, Xd in zip(projs, dYs, Ts, Xds)], M, K)
        return projs[0].from_kernel_order(dXk)
    dX = None
    for p, dY, T, Xd in zip(projs, dYs, Ts, Xds):
        part = p.from_kernel_order(fmsa_hip.gptq_lora_bwd_dx([p.bwd_dict(dY, T, Xd)], M, K))
        dX = part.float() if dX is None else dX.add_(part)  # summed in fp32, rounded once
    return dX.to(dYs[0].dtype) if len(projs) > 1 else part


# ----------------------------------------------------------------------------------------------
# bodies of the three autograd functions; `ctx` is the function's context object
# ----------------------------------------------------------------------------------------------
def w_forward(ctx, X, p, dropout, dtype):
    X2 = _as2d(X, dtype)
    p.pack()
    Xd = _apply_dropout(X2, dropout) if p.r else X2
    (Y,), (U,) = _linear_forward([p], X2, [Xd])
    ctx.proj = p
    ctx.act_dtype = dtype
    ctx.x_shape, ctx.x_dtype = X.shape, X.dtype
    ctx.save_for_backward(Xd, U) if p.r else ctx.save_for_backward()
    return Y.view(*X.shape[:-1], p.w.N)


def w_backward(ctx, dY):
    """(dX, dA, dB)"""
    p = ctx.proj
    dY2 = _as2d(dY, ctx.act_dtype)
    M, K = dY2.shape[0], p.w.K
    dA = dB = None
    T = Xd = None
    if p.r:
        Xd, U = ctx.saved_tensors
        T, dA, dB = p.t_and_grads(Xd, U, dY2)
    dX = _linear_backward_dx([p], [dY2], [T], [Xd], M, K)
    return dX.view(ctx.x_shape).to(ctx.x_dtype), dA, dB


def qkv_forward(ctx, X, projs, dropouts, dtype, rope=None):
    """rope = (cos2d, sin2d, head_dim): Q and K leave rotated (rows of the [positions, >= head_dim / 2] tables are
    taken as token row % positions)."""
    X2 = _as2d(X, dtype)
    Xds = _dropped_inputs(X2, projs, dropouts)
    stack = _pack_group(projs, Xds, dtype)
    ctx.rope = None if rope is None else (rope[0], rope[1], rope[2], 0b011)
    outs, Us = _linear_forward(projs, X2, Xds, stack, ctx.rope)
    ctx.projs, ctx.stack = projs, stack
    ctx.act_dtype = dtype
    ctx.x_shape, ctx.x_dtype = X.shape, X.dtype
    # tensors that may be None (disabled adapters) cannot go through save_for_backward as a
    # fixed-length tuple; store how many were saved per projection
    saved, ctx.layout = [], []
    for Xd, U, p in zip(Xds, Us, projs):
        ctx.layout.append(bool(p.r))
        if p.r:
            saved += [Xd, U]
    ctx.save_for_backward(*saved)
    return tuple(y.view(*X.shape[:-1], p.w.N) for y, p in zip(outs, projs))


def qkv_backward(ctx, dQ, dK, dV):
    """(dX, [(dA, dB)] * 3)"""
    projs = ctx.projs
    saved = list(ctx.saved_tensors)
    K = projs[0].w.K
    dYs = [_as2d(dY, ctx.act_dtype) for dY in (dQ, dK, dV)]  # dK may arrive non-contiguous (gptq/fast_lora.py:631)
    if getattr(ctx, "rope", None) is not None:
        # gradients of the rotated outputs -> gradients of the projections: the inverse rotation (sin negated,
        # kernels/unsloth/rope_embedding.py:105-128), on copies where autograd handed us its own tensors
        cos2d, sin2d, head_dim, mask = ctx.rope
        for i, (dY_in, p) in enumerate(zip((dQ, dK, dV), projs)):
            if (mask >> i) & 1:
                d = dYs[i]
                if d.data_ptr() == dY_in.data_ptr():
                    d = d.clone()
                dYs[i] = fmsa_hip.rope_embedding_(d, cos2d, sin2d, p.w.N // head_dim, head_dim, backward=True)
    Xds, Us = [], []
    for has in ctx.layout:
        Xds.append(saved.pop(0) if has else None)
        Us.append(saved.pop(0) if has else None)
    Ts, grads = _adapter_grads(projs, dYs, Xds, Us, ctx.stack)
    M = dYs[0].shape[0]
    dX = _linear_backward_dx(projs, dYs, Ts, Xds, M, K)
    return dX.view(ctx.x_shape).to(ctx.x_dtype), grads


def mlp_forward(ctx, X, gate, up, down, dropouts, dtype):
    dropout_gate, dropout_up, dropout_down = dropouts
    X2 = _as2d(X, dtype)
    Xg, Xu = _dropped_inputs(X2, (gate, up), (dropout_gate, dropout_up))
    # act-order down projection: let gate / up write e, g, h in its kernel order, so that nothing between the two
    # GEMM stages is permuted and both SwiGLU epilogues stay fused (not with a dropout on h: its mask is tied to
    # the model's column order)
    no_down_dropout = dropout_down is None or isinstance(dropout_down, torch.nn.Identity) or not down.r
    if (down.w.perm is not None and no_down_dropout and hasattr(gate.w, "with_columns")
            and gate.w.N == down.w.K and up.w.N == down.w.K):
        order = down.w.perm.long()
        gate, up = gate.with_columns(order, down.w.perm_key), up.with_columns(order, down.w.perm_key)
        down = down.with_ordered_input()
    stack = _pack_group([gate, up], [Xg, Xu], dtype, also=(down,))
    fused = _one_order([gate, up])
    if fused:
        Ug, Uu = _lora_down_all([gate, up], [Xg, Xu], stack)
        il = _interleaved([gate, up], X2.dtype)
        e, g, h = fmsa_hip.gptq_lora_fwd(gate.to_kernel_order(X2), [gate.fwd_dict(Ug, il), up.fwd_dict(Uu, il)], fmsa_hip.FWD_SWIGLU)
    else:
        (e, g), (Ug, Uu) = _linear_forward([gate, up], X2, [Xg, Xu], stack)
        h = fmsa_hip.swiglu_fwd(e, g)
    hd = _apply_dropout(h, dropout_down) if down.r else h
    (out,), (Ud,) = _linear_forward([down], h, [hd])
    ctx.projs, ctx.stack = (gate, up, down), stack
    ctx.x_shape, ctx.x_dtype = X.shape, X.dtype
    ctx.down_dropped = hd is not h
    none = X2.new_empty(0)
    ctx.save_for_backward(Xg, Xu, e, g, hd if ctx.down_dropped else none,
                          Ug if gate.r else none, Uu if up.r else none, Ud if down.r else none)
    return out.view(*X.shape[:-1], down.w.N)


def mlp_backward(ctx, dY):
    """(dX, (dA_gate, dB_gate), (dA_up, dB_up), (dA_down, dB_down))"""
    gate, up, down = ctx.projs
    Xg, Xu, e, g, hd, Ug, Uu, Ud = ctx.saved_tensors
    dY2 = _as2d(dY, e.dtype)
    M, H, I = dY2.shape[0], gate.w.K, down.w.K

    # ---- down projection: dh, then SwiGLU backward in place (e <- d_g, g <- d_e) -----------
    # T_d = dY B_d is needed by the dh launch; dB_d = s dY^T U_d shares its pass over dY unless U_d has to be
    # re-formed from the recomputed h (dropout on h), which exists only after that launch
    Td = dAd = dBd = None
    if down.r:
        if ctx.down_dropped or not _fuse_t([down], [dY2]):
            Td = fmsa_hip.lora_down(dY2, down.Bt)
        else:
            Td = torch.empty((M, down.r), dtype=dY2.dtype, device=dY2.device)
            (dBd,) = fmsa_hip.lora_grad_batch([(Ud, dY2, down.s, True, down.B_param.dtype, down.Bt, Td)])
    mask_h = hd if ctx.down_dropped else None
    if down.w.perm is None or down.input_ordered:
        h = fmsa_hip.gptq_lora_bwd_dx([down.bwd_dict(dY2, Td, mask_h)], M, I, fmsa_hip.BWD_SWIGLU, e=e, g=g)
    else:
        # un-fused epilogue for a repacked (act-order) weight: dh in kernel order, scatter back,
        # then the standalone SwiGLU backward.  The mask of the LoRA part is (dropout(h) != 0).
        h_now = fmsa_hip.swiglu_fwd(e, g)
        dh = down.from_kernel_order(
            fmsa_hip.gptq_lora_bwd_dx([down.bwd_dict(dY2, Td, mask_h if mask_h is not None else h_now)], M, I))
        h = fmsa_hip.swiglu_bwd(dh, e, g)
    d_g, d_e = e, g
    if down.r:
        # the reference forms both down-projection grads from the recomputed h (gptq/fast_lora.py:369-370)
        if dBd is None:
            Ud_b = fmsa_hip.lora_down(h, down.A) if ctx.down_dropped else Ud
            dAd, dBd = down.lora_grads(Td, h, Ud_b, dY2)
        else:
            (dAd,) = fmsa_hip.lora_grad_batch([(Td, h, down.s, False, down.A_param.dtype)])

    # ---- up / gate: adapter grads, then dX over the concatenated contraction ---------------
    (Tg, Tu), ((dAg, dBg), (dAu, dBu)) = _adapter_grads([gate, up], [d_e, d_g], [Xg, Xu], [Ug, Uu], ctx.stack)
    dX = _linear_backward_dx([up, gate], [d_g, d_e], [Tu, Tg], [Xu, Xg], M, H)
    return (dX.view(ctx.x_shape).to(ctx.x_dtype), gate.natural_grads(dAg, dBg), up.natural_grads(dAu, dBu),
            down.natural_grads(dAd, dBd))

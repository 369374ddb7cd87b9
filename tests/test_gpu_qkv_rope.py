"""Q / K / V projections whose Q and K leave the fused forward kernel already rotated (fmsa_gptq_lora_fwd_rope,
LoRA_QKV_RoPE), against the CPU oracle: rope(lora_qkv(x)) forward, and the oracle's LoRA_QKV backward on the
inverse-rotated output gradients (the rotation is linear and orthogonal, kernels/unsloth/rope_embedding.py:105-128 of
the reference)."""
import pytest
import torch

from oracle import lora as olora
from oracle import norm_rope as onr
from tests.helpers import randn
from tests.model_utils import make_lora_gptq_linear

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max |out - ref| / max |ref| against the fp32 oracle, per tensor


def _q(t, dtype):
    return t.to(dtype).float()


def _cos_sin(positions, d, dtype):
    ang = torch.outer(torch.arange(positions).float(), 1.0 / (10000 ** (torch.arange(0, d, 2).float() / d)))
    emb = torch.cat([ang, ang], dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def _attn(K, Ns, r, alpha, dtype, act_order=False, group_size=128, maker=make_lora_gptq_linear, **kw):
    attn = torch.nn.Module()
    refs = []
    for i, (name, N) in enumerate(Ns.items()):
        if maker is make_lora_gptq_linear:
            lin, W, A, B = maker(K, N, r, alpha, seed=10 + i, act_order=act_order, device="cuda", group_size=group_size,
                                 order_seed=99 if act_order == "shared" else None)
        else:
            lin, W, A, B = maker(K, N, r, alpha, seed=10 + i, device="cuda", **kw)
        setattr(attn, name, lin)
        refs.append((W, _q(A, dtype), _q(B, dtype), alpha / r))
    return attn, refs


def _check(apply_rope, apply_plain, attn, refs, Ns, Bz, S, K, hd, dtype, cos, sin, cos_arg, sin_arg):
    """cos / sin: the [rows, hd] CPU tables the oracle indexes with (token row % rows); *_arg what the op is given."""
    import fmsa_hip

    x = randn((Bz, S, K), 2, dtype)
    douts = [randn((Bz, S, N), 30 + i, dtype) for i, N in enumerate(Ns.values())]
    xg = x.cuda().requires_grad_(True)
    outs = apply_rope(attn, xg, cos_arg, sin_arg)
    douts_gpu = [d.cuda() for d in douts]
    keep = [d.clone() for d in douts_gpu]
    torch.autograd.backward(outs, douts_gpu)
    for d, k in zip(douts_gpu, keep):
        assert torch.equal(d, k)  # the caller's gradient tensors are not rotated in place
    # oracle: forward
    heads = [N // hd for N in Ns.values()]
    dproj = [onr.rope(d.reshape(-1, d.shape[-1]), cos, sin, h, hd, backward=True).float() if i < 2
             else d.float().reshape(-1, d.shape[-1]) for i, (d, h) in enumerate(zip(douts, heads))]
    outs_ref, dx_ref, grads_ref = olora.lora_qkv_autograd(x.float().reshape(-1, K), refs, dproj)
    for i, (o, o_ref, h) in enumerate(zip(outs, outs_ref, heads)):
        assert o.shape == (Bz, S, h * hd) and o.dtype == dtype
        ref = onr.rope(o_ref.to(dtype), cos, sin, h, hd).float() if i < 2 else o_ref
        assert olora.max_rel_err(o.reshape(ref.shape), ref) < TOL, i
    assert olora.max_rel_err(xg.grad.reshape(-1, K), dx_ref) < TOL
    for name, (dA_ref, dB_ref) in zip(Ns, grads_ref):
        lin = getattr(attn, name)
        assert olora.max_rel_err(lin.lora_A["default"].weight.grad, dA_ref) < TOL
        assert olora.max_rel_err(lin.lora_B["default"].weight.grad, dB_ref) < TOL
    # the separate pass over the plain projections gives the same numbers (same roundings: the epilogue rotates the
    # output already rounded to the storage type); one unit in the last place is left for the order of the fp32 sums
    with torch.no_grad():
        plain = apply_plain(attn, x.cuda())
    ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10
    for i in range(2):
        sep = fmsa_hip.rope_embedding_(plain[i].reshape(Bz * S, -1).clone(), cos.cuda(), sin.cuda(), heads[i], hd)
        diff = (outs[i].reshape(Bz * S, -1).float() - sep.float()).abs()
        assert bool((diff <= ulp * sep.float().abs() + 1e-6).all()), i
    assert torch.equal(outs[2], plain[2])


@pytest.mark.parametrize("dtype,cdt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                       (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("act_order", [False, True, "shared"])
@pytest.mark.parametrize("Bz,S,hd", [(2, 96, 128), (1, 50, 64), (3, 37, 32), (2, 40, 256), (1, 33, 16)])
def test_gptq_qkv_rope(Bz, S, hd, dtype, cdt, act_order):
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv, apply_lora_qkv_rope

    K, r, alpha = 1024, 16, 32.0
    Ns = {"q_proj": 1024, "k_proj": 256, "v_proj": 256}
    attn, refs = _attn(K, Ns, r, alpha, dtype, act_order)
    attn.head_dim = hd
    cos, sin = _cos_sin(S, hd, cdt)
    # a cache longer than the sequence, as transformers' rotary module of older releases hands over
    cos_long, sin_long = _cos_sin(S + 40, hd, cdt)
    assert torch.equal(cos_long[:S], cos)
    _check(apply_lora_qkv_rope, apply_lora_qkv, attn, refs, Ns, Bz, S, K, hd, dtype, cos, sin, cos_long.cuda(), sin_long.cuda())


def test_gptq_qkv_rope_per_batch_positions():
    """cos / sin [batch, seq, head_dim] (every batch entry with positions of its own) are used row by row."""
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv, apply_lora_qkv_rope

    Bz, S, K, hd, dtype = 2, 70, 512, 64, torch.bfloat16
    Ns = {"q_proj": 512, "k_proj": 128, "v_proj": 192}
    attn, refs = _attn(K, Ns, 8, 16.0, dtype)
    attn.head_dim = hd
    cos_all, sin_all = _cos_sin(500, hd, dtype)
    pos = torch.stack([torch.arange(S), torch.arange(S) + 300])
    cos3, sin3 = cos_all[pos], sin_all[pos]  # [Bz, S, hd]
    _check(apply_lora_qkv_rope, apply_lora_qkv, attn, refs, Ns, Bz, S, K, hd, dtype,
           cos3.reshape(Bz * S, hd), sin3.reshape(Bz * S, hd), cos3.cuda(), sin3.cuda())


def test_gptq_qkv_rope_falls_back_to_the_separate_pass(monkeypatch):
    """Group size 32 is outside what the fused epilogue takes: the op still returns rotated Q / K."""
    import fmsa_hip
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_qkv, apply_lora_qkv_rope

    seen = []
    real = fmsa_hip.gptq_lora_fwd
    monkeypatch.setattr(fmsa_hip, "gptq_lora_fwd", lambda *a, **k: (seen.append(k.get("rope")), real(*a, **k))[1])
    Bz, S, K, hd, dtype = 1, 80, 256, 64, torch.float16
    Ns = {"q_proj": 256, "k_proj": 128, "v_proj": 128}
    attn, refs = _attn(K, Ns, 8, 16.0, dtype, group_size=32)
    attn.head_dim = hd
    cos, sin = _cos_sin(S, hd, dtype)
    _check(apply_lora_qkv_rope, apply_lora_qkv, attn, refs, Ns, Bz, S, K, hd, dtype, cos, sin, cos.cuda(), sin.cuda())
    assert seen and all(r is None for r in seen)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_nf4_qkv_rope(dtype):
    from fms_acceleration_foak.fused_ops.unsloth_lora.bnb.fast_lora import apply_lora_qkv, apply_lora_qkv_rope
    from tests.model_utils import make_lora_nf4_linear

    Bz, S, K, hd = 2, 75, 1024, 128
    Ns = {"q_proj": 1024, "k_proj": 256, "v_proj": 256}
    attn, refs = _attn(K, Ns, 16, 32.0, dtype, maker=make_lora_nf4_linear, compute_dtype=dtype)
    attn.head_dim = hd
    cos, sin = _cos_sin(S, hd, torch.float32)
    _check(apply_lora_qkv_rope, apply_lora_qkv, attn, refs, Ns, Bz, S, K, hd, dtype, cos, sin, cos.cuda(), sin.cuda())


def test_fwd_rope_entry_rejects_what_the_kernel_does_not_take():
    import fmsa_hip

    attn, _ = _attn(256, {"q_proj": 256}, 8, 16.0, torch.bfloat16, group_size=64)
    from fms_acceleration_foak.fused_ops.unsloth_lora import fused_core as core
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import _proj, get_lora_parameters, unpack_gptqstate

    st, bias, A, B, s, _ = get_lora_parameters(attn.q_proj)
    p = _proj((*unpack_gptqstate(st), bias, A, B, s), torch.bfloat16)
    p.pack()
    x = randn((64, 256), 1, torch.bfloat16).cuda()
    U = core._lora_down_all([p], [x], None)[0]
    cos, sin = (t.cuda() for t in _cos_sin(64, 64, torch.bfloat16))
    ok = fmsa_hip.gptq_lora_fwd(x, [p.fwd_dict(U)], rope=(cos, sin, 64, 1))[0]
    assert ok.shape == (64, 256)
    with pytest.raises(fmsa_hip.FmsaError):
        fmsa_hip.gptq_lora_fwd(x, [p.fwd_dict(U)], rope=(cos, sin, 96, 1))  # 256 % head_dim
    with pytest.raises(fmsa_hip.FmsaError):
        fmsa_hip.gptq_lora_fwd(x, [p.fwd_dict(U)], rope=(cos, sin, 64, 2))  # mask names a projection that is not there
    with pytest.raises(ValueError):
        fmsa_hip.gptq_lora_fwd(x, [p.fwd_dict(U)], rope=(cos[:, :16], sin[:, :16], 64, 1))  # table narrower than half a head

"""ModelPatcher behaviours (mirrors plugins/framework/tests/test_model_patcher.py of the reference)
and the fused-LoRA patch rules applied to real transformers modules on the CPU."""
import warnings

import pytest
import torch

from fms_acceleration.model_patcher import (
    ModelPatcher,
    ModelPatcherRule,
    ModelPatcherTrigger,
    ModelPatcherTriggerType,
    combine_functions,
    combine_triggers,
    patch_model,
)
from fms_acceleration.utils.test_utils import instantiate_model_patcher


class Leaf(torch.nn.Module):
    def forward(self, x):
        return x + 1


class Other(torch.nn.Module):
    def forward(self, x):
        return x


class Net(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.a = Leaf()
        self.b = Leaf()
        self.c = Other()

    def forward(self, x):
        return self.c(self.b(self.a(x)))


def test_trigger_typing():
    assert ModelPatcherTrigger(check=Leaf).type == ModelPatcherTriggerType.module
    assert ModelPatcherTrigger(check=lambda m: True).type == ModelPatcherTriggerType.callable
    with pytest.raises(TypeError):
        ModelPatcherTrigger(check=3)
    with pytest.raises(AssertionError):
        ModelPatcherTrigger(check=Leaf, type=ModelPatcherTriggerType.callable)
    t = ModelPatcherTrigger(check=Leaf, module_name="a")
    assert t.is_triggered(Leaf(), "a") and not t.is_triggered(Leaf(), "b") and not t.is_triggered(Other(), "a")

    def raises(m):
        raise AttributeError("no such child")

    assert not ModelPatcherTrigger(check=raises).is_triggered(Leaf())


def test_combine_triggers_and_functions():
    is_leaf = ModelPatcherTrigger(check=Leaf)
    named_a = ModelPatcherTrigger(check=lambda m: True, module_name="a")
    assert combine_triggers(is_leaf, named_a, logic="OR").is_triggered(Other(), "a") is False  # name not passed on
    assert combine_triggers(is_leaf, ModelPatcherTrigger(check=Other), logic="OR").is_triggered(Other())
    assert not combine_triggers(is_leaf, ModelPatcherTrigger(check=Other), logic="AND").is_triggered(Other())
    with pytest.raises(AssertionError):
        combine_triggers(is_leaf, logic="XOR")
    f = combine_functions(lambda m: [1], lambda m: [2, 3])
    assert f(None) == [1, 2, 3]


def test_rule_validation_and_duplicates():
    with pytest.raises(ValueError, match="at most one"):
        ModelPatcherRule("r", trigger=ModelPatcherTrigger(check=Leaf), forward=lambda s, x: x, forward_builder=lambda m: None)
    with pytest.raises(ValueError, match="trigger must be None"):
        ModelPatcherRule("r", trigger=ModelPatcherTrigger(check=Leaf), import_and_maybe_reload=("a.b", object, None))
    with instantiate_model_patcher():
        ModelPatcher.register(ModelPatcherRule("dup", trigger=ModelPatcherTrigger(check=Leaf)))
        with pytest.raises(AssertionError, match="already exists"):
            ModelPatcher.register(ModelPatcherRule("dup", trigger=ModelPatcherTrigger(check=Leaf)))
    assert "dup" not in ModelPatcher.rules  # isolation restored the singleton


def test_forward_replacement_first_rule_wins():
    with instantiate_model_patcher():
        ModelPatcher.register(ModelPatcherRule("plus10", trigger=ModelPatcherTrigger(check=Leaf), forward=lambda self, x: x + 10))
        ModelPatcher.register(ModelPatcherRule("plus100", trigger=ModelPatcherTrigger(check=Leaf), forward=lambda self, x: x + 100))
        net = Net()
        with warnings.catch_warnings(record=True) as w:
            warnings.simplefilter("always")
            patch_model(net)
        assert any("is ignored" in str(x.message) for x in w)
        assert net(torch.zeros(1)).item() == 20
        assert [h.rule_id for h in ModelPatcher.history] == ["plus10", "plus10"]
        assert "plus10" in ModelPatcher.summary() and "Leaf" in ModelPatcher.summary()
        assert len(ModelPatcher.summary(raw=True)) == 2


def test_forward_builder_list_becomes_sub_rules():
    calls = []

    def builder(mod):
        calls.append(type(mod).__name__)
        return [
            (ModelPatcherTrigger(check=Leaf, module_name="a"), lambda self, x: x + 2),
            (ModelPatcherTrigger(check=Leaf, module_name="b"), lambda self, x: x + 3),
        ]

    with instantiate_model_patcher():
        ModelPatcher.register(ModelPatcherRule("net", trigger=ModelPatcherTrigger(check=Net), forward_builder=builder))
        net = Net()
        patch_model(net)
        assert calls == ["Net"]
        assert net(torch.zeros(1)).item() == 5
        assert sorted(h.rule_id for h in ModelPatcher.history) == ["net-1", "net-2"]
        assert set(ModelPatcher.rules) == {"net"}  # temporary sub-rules are gone


def _tiny_llama_layer():
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaAttention, LlamaMLP

    from fms_acceleration_peft import LoraLinear, QuantLinear

    cfg = LlamaConfig(hidden_size=128, intermediate_size=256, num_attention_heads=4, num_key_value_heads=2,
                      num_hidden_layers=1, vocab_size=64, hidden_act="silu")
    cfg.architectures = ["LlamaForCausalLM"]

    def wrap(lin):
        return LoraLinear(QuantLinear(4, 64, lin.in_features, lin.out_features, False), r=8, lora_alpha=16)

    block = torch.nn.Module()
    block.self_attn = LlamaAttention(cfg, layer_idx=0)
    block.mlp = LlamaMLP(cfg)
    for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
        setattr(block.self_attn, name, wrap(getattr(block.self_attn, name)))
    for name in ("gate_proj", "up_proj", "down_proj"):
        setattr(block.mlp, name, wrap(getattr(block.mlp, name)))
    block.config = cfg
    return block, cfg


def test_fused_lora_rules_patch_llama_modules():
    """The FOAK plugin registers llama-qkvo / llama-mlp (and the mistral / granite twins); patching a
    Llama attention + MLP whose projections are LoRA-wrapped QuantLinears rebinds q/k/v/o and the MLP."""
    from fms_acceleration_foak import FastKernelsAccelerationPlugin
    from fms_acceleration_foak.fused_ops.unsloth_lora.gptq.fast_lora import apply_lora_mlp, apply_lora_o_v2

    block, cfg = _tiny_llama_layer()
    block.quantization_method = "gptq"
    plugin = FastKernelsAccelerationPlugin({"training": {"fused_ops_and_kernels": {"fused_lora": True, "fast_loss": True}}})
    train_args = type("T", (), {"bf16": True, "fp16": False})()
    with instantiate_model_patcher():
        plugin.augmentation(block, train_args, ())
        archs = ["llama", "mistral", "granite", "mixtral", "granitemoe", "granitemoeshared", "granitemoehybrid"]
        loss_ids = {f"{a}-custom-loss" for a in archs}  # transformers >= 4.46 here
        assert set(ModelPatcher.rules) == loss_ids | {
            "llama-qkvo", "llama-mlp", "mistral-qkvo", "mistral-mlp", "granite-qkvo", "granite-mlp",
            "mixtral-qkvo", "granitemoe-qkvo", "granitemoeshared-qkvo", "granitemoehybrid-qkvo"}
        patch_model(block)
        ids = sorted(h.rule_id for h in ModelPatcher.history)
        assert ids == ["llama-mlp", "llama-qkvo-1", "llama-qkvo-2", "llama-qkvo-3", "llama-qkvo-4"]
        assert block.mlp.forward.__func__ is apply_lora_mlp
        assert block.self_attn.o_proj.forward.__func__ is apply_lora_o_v2
        for name in ("q_proj", "k_proj", "v_proj"):
            assert "forward" in vars(getattr(block.self_attn, name))  # instance-level rebinding
        assert plugin.get_callbacks_and_ready_for_train(block, None) == []
    # without a quantised base the fused-LoRA rules are not registered at all
    block2, _ = _tiny_llama_layer()
    with instantiate_model_patcher():
        plugin.augmentation(block2, train_args, ())
        assert set(ModelPatcher.rules) == loss_ids
    # `fast_loss: fused_ce_liger` selects the fused loss head, for the dense-attention families only
    liger = FastKernelsAccelerationPlugin({"training": {"fused_ops_and_kernels": {"fast_loss": "fused_ce_liger"}}})
    with instantiate_model_patcher():
        liger.augmentation(block2, train_args, ())
        assert set(ModelPatcher.rules) == {"llama-fused-lce", "mistral-fused-lce", "granite-fused-lce"}
    # mixed precision is mandatory on a quantised base
    with instantiate_model_patcher():
        with pytest.raises(AssertionError, match="mixed precision"):
            plugin.augmentation(block, type("T", (), {"bf16": False, "fp16": False})(), ())


def test_mlp_rule_dropped_for_non_silu_activation():
    from fms_acceleration_foak.models import llama

    cfg = type("C", (), {"hidden_act": "gelu", "architectures": ["LlamaForCausalLM"]})()
    with warnings.catch_warnings(record=True):
        warnings.simplefilter("always")
        ids = [r.rule_id for r in llama.get_mp_rules("auto_gptq", cfg)]
    assert ids == ["llama-qkvo", "llama-fused-lce", "llama-custom-loss", "llama-rms", "llama-rope"]


def test_partial_lora_follows_the_reference_rule_logic():
    """The qkvo trigger is an OR of "q, k, v all LoRA" and "o is LoRA", and its builder APPENDs the
    sub-rules of both branches (models/llama.py:75-108 of the reference): with an adapter-less k_proj
    the rule still fires through o_proj, and the per-projection sub-rules then patch exactly the
    children that are LoRA layers (q, v, o).  Same behaviour as the reference, kept as is."""
    from fms_acceleration_foak.models import llama

    block, cfg = _tiny_llama_layer()
    block.self_attn.k_proj = block.self_attn.k_proj.base_layer  # k loses its adapter
    with instantiate_model_patcher():
        for r in llama.get_mp_rules("auto_gptq", cfg):
            ModelPatcher.register(r)
        patch_model(block)
        ids = sorted(h.rule_id for h in ModelPatcher.history)
        assert ids == ["llama-mlp", "llama-qkvo-1", "llama-qkvo-3", "llama-qkvo-4"]


def test_qkv_wrapper_protocol():
    from fms_acceleration_foak.models.utils import _build_fused_forwards

    calls = []

    def fused(attn, X):
        calls.append(1)
        return X + 1, X + 2, X + 3

    fwd = dict(_build_fused_forwards(None, fused, ["q_proj", "k_proj", "v_proj"]))
    x = torch.zeros(1)
    assert fwd["q_proj"](None, x).item() == 1
    assert fwd["k_proj"](None, x).item() == 2
    with pytest.raises(AssertionError):
        fwd["k_proj"](None, x)  # k called twice before v
    assert fwd["v_proj"](None, x).item() == 3
    assert fwd["v_proj"](None, x).item() == 3 and len(calls) == 2  # a new round starts with whoever comes first


def test_qkv_wrapper_with_rope_tables():
    """With a rope operation the wrapper keeps the position_embeddings the attention is called with, hands them to the
    fused call, and marks Q / K so that fast_rope_embedding passes exactly those tensors through, once."""
    from fms_acceleration_foak.kernels.unsloth import rope_embedding as re_mod
    from fms_acceleration_foak.models.utils import _build_fused_forwards

    names = ["q_proj", "k_proj", "v_proj"]

    class Attn(torch.nn.Module):
        def forward(self, hidden_states, position_embeddings=None):
            q, k, v = (fwd[n](None, hidden_states) for n in names)
            q, k = q.view(1, 2, 1, 4).transpose(1, 2), k.view(1, 2, 1, 4).transpose(1, 2)
            cos, sin = position_embeddings if position_embeddings is not None else (None, None)
            return re_mod.fast_rope_embedding(q, k, cos, sin), v

    seen = []
    plain = lambda attn, X: (X + 1, X + 2, X + 3)  # noqa: E731

    def with_rope(attn, X, cos, sin):
        seen.append((cos, sin))
        return X + 10, X + 20, X + 30

    attn = Attn()
    fwd = dict(_build_fused_forwards(attn, plain, names, with_rope))
    x = torch.zeros(1, 2, 4)
    (q, k), v = attn(x, position_embeddings=("c", "s"))
    assert seen == [("c", "s")] and q.flatten()[0] == 10 and k.flatten()[0] == 20 and v.flatten()[0] == 30
    assert not re_mod._ROTATED  # consumed by the pass-through
    # a Q the fused call did not produce is not passed through (the kernel is asked for, which a CPU tensor cannot do)
    with pytest.raises(Exception):
        re_mod.fast_rope_embedding(q.clone(), k.clone(), torch.ones(2, 4), torch.zeros(2, 4))
    # Q marked, K from elsewhere: refuses instead of rotating one of them twice
    re_mod.mark_rotated(q, k)
    with pytest.raises(RuntimeError, match="K does not"):
        re_mod.fast_rope_embedding(q, k.clone(), None, None)
    assert not re_mod._ROTATED
    # an attention that is given tables but never rotates: refused when that very forward returns, not a call later
    class NoRope(torch.nn.Module):
        boom = False

        def forward(self, hidden_states, position_embeddings=None):
            q = fwd2["q_proj"](None, hidden_states)
            if self.boom:
                raise MemoryError("inside the forward")
            return [q] + [fwd2[n](None, hidden_states) for n in names[1:]]

    lazy = NoRope()
    fwd2 = dict(_build_fused_forwards(lazy, plain, names, with_rope))
    with pytest.raises(RuntimeError, match="rotated twice"):
        lazy(x, position_embeddings=("c", "s"))
    assert not re_mod._ROTATED
    # an exception between the fused call and the rotation leaves neither a mark nor pending outputs: the retry is clean
    lazy.boom = True
    with pytest.raises(MemoryError):
        lazy(x, position_embeddings=("c", "s"))
    assert not re_mod._ROTATED
    lazy.boom = False
    assert [o.flatten()[0].item() for o in lazy(x)] == [1, 2, 3]  # no tables: the plain operation, protocol intact
    # without tables the plain fused operation runs and nothing is marked
    for n in names:
        out = fwd[n](None, x)
    assert out.flatten()[0] == 3 and not re_mod._ROTATED and len(seen) == 3  # (the three calls with tables above)


def test_fast_rope_embeddings_fused_qkv_is_accepted():
    from fms_acceleration_foak import FastKernelsAccelerationPlugin

    plugin = FastKernelsAccelerationPlugin({"training": {"fused_ops_and_kernels": {
        "fused_lora": True, "fast_rope_embeddings": "fused_qkv"}}})
    assert plugin.configurations["fast_rope_embeddings"] == "fused_qkv"
    with pytest.raises(Exception):
        FastKernelsAccelerationPlugin({"training": {"fused_ops_and_kernels": {"fast_rope_embeddings": "other"}}})


def test_filter_mp_rules():
    from fms_acceleration_foak.utils import filter_mp_rules

    rules = [ModelPatcherRule(rule_id=i) for i in ("a-qkvo", "a-mlp", "a-rms")]
    assert [r.rule_id for r in filter_mp_rules(rules, {"qkvo", "mlp"})] == ["a-qkvo", "a-mlp"]
    assert [r.rule_id for r in filter_mp_rules(rules, {"mlp"}, drop=True)] == ["a-qkvo", "a-rms"]


def test_rms_and_rope_rules_registered_and_applied():
    """fast_rms_layernorm / fast_rope_embeddings select the `<arch>-rms` / `<arch>-rope` rules: the
    norm modules get the new forward, the modelling module's apply_rotary_pos_emb is replaced."""
    import transformers.models.llama.modeling_llama as ml
    from transformers import LlamaConfig
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    from fms_acceleration_foak import FastKernelsAccelerationPlugin
    from fms_acceleration_foak.kernels.unsloth import fast_rms_layernorm, fast_rope_embedding

    cfg = LlamaConfig(hidden_size=64, intermediate_size=128, num_attention_heads=4, num_hidden_layers=1, vocab_size=32)
    cfg.architectures = ["LlamaForCausalLM"]
    from transformers import LlamaForCausalLM

    model = LlamaForCausalLM(cfg)  # the import rule only applies to models defined under the patched module path
    plugin = FastKernelsAccelerationPlugin(
        {"training": {"fused_ops_and_kernels": {"fast_rms_layernorm": True, "fast_rope_embeddings": True}}})
    original = ml.apply_rotary_pos_emb
    try:
        with instantiate_model_patcher():
            plugin.augmentation(model, type("T", (), {"bf16": True, "fp16": False})(), ())
            ids = set(ModelPatcher.rules)
            assert {"llama-rms", "llama-rope", "mistral-rms", "granite-rope", "mixtral-rms", "granitemoe-rope"} <= ids
            assert not any(i.endswith(("qkvo", "mlp")) for i in ids)
            patch_model(model)
            norms = [m for m in model.modules() if isinstance(m, LlamaRMSNorm)]
            assert len(norms) == 3 and all(m.forward.__func__ is fast_rms_layernorm for m in norms)
            assert ml.apply_rotary_pos_emb is fast_rope_embedding
    finally:
        ml.apply_rotary_pos_emb = original

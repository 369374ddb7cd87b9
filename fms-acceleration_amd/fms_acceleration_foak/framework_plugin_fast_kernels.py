"""FastKernelsAccelerationPlugin: turns the `fused_ops_and_kernels` configuration into registered
ModelPatcher rules (reference: fms_acceleration_foak/framework_plugin_fast_kernels.py:31-222).

Switches with kernels behind them in this build: `fused_lora` (rule suffixes "qkvo", "mlp"),
`fast_rms_layernorm` ("rms"), `fast_rope_embeddings` ("rope"), `fast_loss: true` ("cross-ent",
"custom-loss") and `fast_loss: fused_ce_liger` ("fused-lce": llama, mistral and granite, as in the
reference).  One value beyond the reference's: `fast_rope_embeddings: fused_qkv` registers the same "rope" rule and,
with `fused_lora` on a quantised base, lets the fused Q / K / V projection of llama, mistral and granite apply the
rotary embedding in its own launch (the separate pass then finds Q and K marked as done and passes them through).
"""
from __future__ import annotations

from typing import Dict, Set, Tuple

from fms_acceleration import AccelerationPlugin, AccelerationPluginConfigError

from .utils import filter_mp_rules


def register_foak_model_patch_rules(base_type: str, filter_endswith: Set[str] = None, config=None, qkv_rope: bool = False):
    from fms_acceleration.model_patcher import ModelPatcher  # pylint: disable=import-outside-toplevel

    # pylint: disable=import-outside-toplevel
    from .models import granite, granitemoe, granitemoehybrid, granitemoeshared, llama, mistral, mixtral

    rules = [
        *granite.get_mp_rules(base_type, config, qkv_rope),
        *granitemoe.get_mp_rules(base_type),
        *granitemoeshared.get_mp_rules(base_type),
        *granitemoehybrid.get_mp_rules(base_type),
        *llama.get_mp_rules(base_type, config, qkv_rope),
        *mistral.get_mp_rules(base_type, config, qkv_rope),
        *mixtral.get_mp_rules(base_type),
    ]
    if filter_endswith:
        rules = filter_mp_rules(rules, filter_endswith)
    for rule in rules:
        ModelPatcher.register(rule)


FILTER_MAP = {
    "fused_lora": {"qkvo", "mlp"},
    "fast_loss": {True: {"cross-ent", "custom-loss"}, "fused_ce_liger": "fused-lce"},
    "fast_rms_layernorm": "rms",
    "fast_rope_embeddings": {True: "rope", "fused_qkv": "rope"},
}


class FastKernelsAccelerationPlugin(AccelerationPlugin):
    restricted_model_archs = [
        "GraniteForCausalLM",
        "GraniteMoeForCausalLM",
        "GPTBigCodeForCausalLM",
        "MixtralForCausalLM",
        "LlamaForCausalLM",
        "MistralForCausalLM",
        "GraniteMoeSharedForCausalLM",
        "GraniteMoeHybridForCausalLM",
    ]

    def __init__(self, configurations: Dict[str, Dict]):
        super().__init__(configurations)
        try:
            self.configurations = self._check_config_and_maybe_check_values(key="training.fused_ops_and_kernels")
        except AccelerationPluginConfigError:
            self.configurations = self._check_config_and_maybe_check_values(
                key="peft.quantization.fused_ops_and_kernels"
            )
        for key, values in (
            ("base_layer", ["auto_gptq", "bitsandbytes"]),
            ("fused_lora", [False, True]),
            ("fast_loss", [False, True, "fused_ce_liger"]),
            ("fast_rms_layernorm", [False, True]),
            ("fast_rope_embeddings", [False, True, "fused_qkv"]),
        ):
            default = "auto_gptq" if key == "base_layer" else False
            self.configurations[key] = self._check_config_and_maybe_check_values(key=key, values=values, default=default)

    @property
    def requires_augmentation(self):
        return True

    def augmentation(self, model, train_args, modifiable_args: Tuple):
        has_quant = getattr(model, "quantization_method", None)
        if has_quant:
            assert train_args.bf16 is True or train_args.fp16 is True, (
                f"{self.__class__} requires mixed precision argument `--fp16` or `--bf16`"
            )
        omitted = set()
        if has_quant is None:
            omitted.add("fused_lora")  # the fused LoRA rules only make sense on a quantised base
        terms = set()
        for key, value in self.configurations.items():
            if (isinstance(value, bool) and value is False) or key not in FILTER_MAP or key in omitted:
                continue
            selected = FILTER_MAP[key]
            if isinstance(selected, dict) and value in selected:
                selected = selected[value]
            terms.update({selected} if isinstance(selected, str) else selected)
        register_foak_model_patch_rules(
            base_type=self.configurations["base_layer"], filter_endswith=terms, config=model.config,
            qkv_rope=self.configurations["fast_rope_embeddings"] == "fused_qkv" and "fused_lora" not in omitted
            and bool(self.configurations["fused_lora"]),
        )
        return model, modifiable_args

    def get_callbacks_and_ready_for_train(self, model=None, accelerator=None):
        # One GPU: the reference's FSDP adapter-gradient hooks (:189-212) have nothing to attach to.
        return []


AccelerationPlugin.register_plugin(
    FastKernelsAccelerationPlugin,
    configuration_or_paths=["training.fused_ops_and_kernels", "peft.quantization.fused_ops_and_kernels"],
)

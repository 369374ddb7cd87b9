"""A minimal LoRA wrapper with exactly the attributes the fused operators read from a PEFT
`LoraLayer` (see get_lora_parameters, fused-ops-and-kernels/.../unsloth_lora/gptq/fast_lora.py:94-116):
`base_layer`, `lora_A` / `lora_B` (ModuleDicts of bias-free nn.Linear), `scaling`, `lora_dropout`,
`active_adapters`, `disable_adapters`, `merged`.  peft is not installed where this is built, so this
class stands in for `peft.tuners.lora.gptq.QuantLinear` / `GPTQLoraLinear`; a real PEFT layer is
accepted by the fused operators just the same (duck typing, FOAK models/utils.py:46-49).

`forward` is PEFT's unfused computation: result = base(x); result += lora_B(lora_A(dropout(x))) * scaling.
"""
from __future__ import annotations

import math

import torch
from torch import nn


class LoraLinear(nn.Module):
    def __init__(self, base_layer: nn.Module, r: int, lora_alpha: float, lora_dropout: float = 0.0,
                 adapter_name: str = "default", dtype=torch.float32):
        super().__init__()
        self.base_layer = base_layer
        in_f = getattr(base_layer, "infeatures", None) or base_layer.in_features  # QuantLinear / Linear4bit
        out_f = getattr(base_layer, "outfeatures", None) or base_layer.out_features
        self.in_features, self.out_features = in_f, out_f
        self.r = {adapter_name: r}
        self.lora_alpha = {adapter_name: lora_alpha}
        self.scaling = {adapter_name: lora_alpha / r}
        self.lora_dropout = nn.ModuleDict({adapter_name: nn.Dropout(p=lora_dropout) if lora_dropout > 0.0 else nn.Identity()})
        self.lora_A = nn.ModuleDict({adapter_name: nn.Linear(in_f, r, bias=False, dtype=dtype)})
        self.lora_B = nn.ModuleDict({adapter_name: nn.Linear(r, out_f, bias=False, dtype=dtype)})
        nn.init.kaiming_uniform_(self.lora_A[adapter_name].weight, a=math.sqrt(5))
        nn.init.zeros_(self.lora_B[adapter_name].weight)
        self._active_adapter = [adapter_name]
        self._disable_adapters = False
        self.merged_adapters = []
        for p in base_layer.parameters():
            p.requires_grad_(False)

    @property
    def active_adapters(self):
        return self._active_adapter

    @property
    def active_adapter(self):
        return self._active_adapter[0]

    @property
    def disable_adapters(self):
        return self._disable_adapters

    @property
    def merged(self):
        return bool(self.merged_adapters)

    def enable_adapters(self, enabled: bool):
        self._disable_adapters = not enabled

    def forward(self, x):
        result = self.base_layer(x)
        if self.disable_adapters:
            return result
        for name in self.active_adapters:
            A, B = self.lora_A[name], self.lora_B[name]
            xd = self.lora_dropout[name](x).to(A.weight.dtype)
            result = result + (B(A(xd)) * self.scaling[name]).to(result.dtype)
        return result


# peft's per-architecture defaults for `target_modules=None` (peft.utils.constants:
# TRANSFORMERS_MODELS_TO_LORA_TARGET_MODULES_MAPPING) for the architectures the fused-LoRA rules cover
DEFAULT_TARGET_MODULES = {
    "llama": ["q_proj", "v_proj"],
    "mistral": ["q_proj", "v_proj"],
    "mixtral": ["q_proj", "v_proj"],
    "granite": ["q_proj", "v_proj"],
    "granitemoe": ["q_proj", "v_proj"],
    "granitemoeshared": ["q_proj", "v_proj"],
    "granitemoehybrid": ["q_proj", "v_proj"],
}


def _config_get(peft_config, key, default=None):
    return peft_config.get(key, default) if isinstance(peft_config, dict) else getattr(peft_config, key, default)


def _target_matcher(model, targets):
    """peft's matching of `target_modules` against a module's dotted name (peft.tuners.tuners_utils:
    check_target_module_exists): a string is a regular expression that must match the whole name (except
    "all-linear": every base layer but the output embedding), a list matches a name that equals an entry or
    ends with "." + entry; None falls back to the default of the model type."""
    import re  # pylint: disable=import-outside-toplevel

    if targets is None:
        model_type = getattr(getattr(model, "config", None), "model_type", None)
        if model_type not in DEFAULT_TARGET_MODULES:
            raise ValueError(f"peft_config has no target_modules and the model type {model_type!r} has no default: name them")
        targets = DEFAULT_TARGET_MODULES[model_type]
    if isinstance(targets, str):
        if targets == "all-linear":
            out = getattr(model, "get_output_embeddings", lambda: None)()
            return (lambda name, mod: mod is not out), "all-linear"
        pattern = re.compile(targets)
        return (lambda name, mod: pattern.fullmatch(name) is not None), targets
    targets = list(targets)
    return (lambda name, mod: any(name == t or name.endswith("." + t) for t in targets)), sorted(targets)


def install_lora_adapters(model, peft_config, base_classes, adapter_name="default"):
    """Wraps every module of `model` that is an instance of `base_classes` and is named by
    `peft_config.target_modules` in a LoraLinear (what peft's get_peft_model does with its own LoRA layer),
    then freezes every other parameter.  The matching runs first: a configuration that matches nothing raises
    and leaves the model untouched.  Returns the dotted names of the wrapped modules."""
    r, alpha = _config_get(peft_config, "r"), _config_get(peft_config, "lora_alpha")
    dropout = float(_config_get(peft_config, "lora_dropout", 0.0) or 0.0)
    if not r or alpha is None:
        raise ValueError("peft_config needs `r` and `lora_alpha` to install LoRA adapters")
    match, shown = _target_matcher(model, _config_get(peft_config, "target_modules"))
    found = []
    for parent_name, parent in model.named_modules():
        for child_name, child in parent.named_children():
            full = f"{parent_name}.{child_name}" if parent_name else child_name
            if isinstance(child, base_classes) and match(full, child):
                found.append((parent, child_name, child, full))
    if not found:
        names = ", ".join(c.__name__ for c in (base_classes if isinstance(base_classes, tuple) else (base_classes,)))
        raise ValueError(f"no {names} module matches target_modules={shown}: nothing to train "
                         "(was the model loaded through this plugin's model_loader?)")
    for p in model.parameters():
        p.requires_grad_(False)
    for parent, child_name, child, _ in found:
        wrapped = LoraLinear(child, int(r), float(alpha), dropout, adapter_name=adapter_name)
        device = next((t.device for t in list(child.parameters()) + list(child.buffers())), None)
        setattr(parent, child_name, wrapped.to(device) if device is not None else wrapped)
    return [full for *_, full in found]

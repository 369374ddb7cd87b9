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

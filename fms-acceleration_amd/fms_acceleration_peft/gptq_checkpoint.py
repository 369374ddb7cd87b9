"""GPTQ checkpoints: the on-disk format (safetensors with the QuantLinear tensors + a
`quantize_config.json`), the v1 -> v2 zero-point conversion, and loading into a model whose
linears become `QuantLinear` modules.

Mirrors the checkpoint side of the reference's vendored gptqmodel: `QuantizeConfig`
(gptqmodel/quantization/config.py:35-110: fields, the `checkpoint_format` JSON key, the `w_bit` /
`q_group_size` synonyms), `convert_gptq_v1_to_v2_format` (gptqmodel/utils/model.py:205-237: v1
files store zero-1, so `qzeros += 0x11111111` for 4 bits) and the load order of
`from_quantized` (gptqmodel/models/base.py:1218-1258: replace the linears, load the tensors,
convert when the file says `gptq`).  No hub access, no accelerate dispatch: a local directory in,
a model on one device out.
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, field
from typing import Dict, Iterable, Optional

import torch
from torch import nn

from .qlinear import QuantLinear

QUANT_CONFIG_FILENAME = "quantize_config.json"
QUANT_CONFIG_FILENAME_COMPAT = [QUANT_CONFIG_FILENAME, "quant_config.json", "config.json"]
FORMAT_GPTQ, FORMAT_GPTQ_V2 = "gptq", "gptq_v2"
_SYNONYMS = {"w_bit": "bits", "q_group_size": "group_size", "checkpoint_format": "format"}
_V1_TO_V2 = {2: 0x55555555, 4: 0x11111111, 8: 0x01010101}


@dataclass
class QuantizeConfig:
    bits: int = 4
    group_size: int = -1
    damp_percent: float = 0.01
    desc_act: bool = True
    static_groups: bool = False
    sym: bool = True
    true_sequential: bool = True
    lm_head: bool = False
    quant_method: str = "gptq"
    format: str = FORMAT_GPTQ  # the reference's default: v1 files for compatibility with other loaders
    meta: Optional[Dict] = field(default=None)

    def __post_init__(self):
        if self.bits not in (2, 3, 4, 8):
            raise ValueError(f"only support quantize to [2, 3, 4, 8] bits, got {self.bits}")
        if self.group_size != -1 and self.group_size <= 0:
            raise ValueError("unless equal to -1, group_size must greater than 0.")
        if self.format not in (FORMAT_GPTQ, FORMAT_GPTQ_V2, "triton"):
            raise ValueError(f"unknown checkpoint format {self.format!r}")

    @classmethod
    def from_quant_config(cls, cfg: Dict):
        known = {f for f in cls.__dataclass_fields__}  # pylint: disable=no-member
        out = {}
        for key, val in cfg.items():
            key = _SYNONYMS.get(key, key)
            if key in known:
                out[key] = val
        if "format" not in out:
            out["format"] = FORMAT_GPTQ  # files written before the field existed are v1
        return cls(**out)

    @classmethod
    def from_pretrained(cls, save_dir: str):
        for name in QUANT_CONFIG_FILENAME_COMPAT:
            path = os.path.join(save_dir, name)
            if not os.path.isfile(path):
                continue
            with open(path, "r", encoding="utf-8") as fh:
                cfg = json.load(fh)
            if name == "config.json":  # transformers-style: the quantisation block lives inside
                cfg = cfg.get("quantization_config")
                if cfg is None:
                    continue
            return cls.from_quant_config(cfg)
        raise FileNotFoundError(f"no {QUANT_CONFIG_FILENAME_COMPAT} with a quantisation config in {save_dir}")

    def to_dict(self):
        d = asdict(self)
        d["checkpoint_format"] = d.pop("format")
        return d

    def save_pretrained(self, save_dir: str):
        with open(os.path.join(save_dir, QUANT_CONFIG_FILENAME), "w", encoding="utf-8") as fh:
            json.dump(self.to_dict(), fh, indent=2)


def _quant_linears(model: nn.Module) -> Iterable[QuantLinear]:
    return (m for m in model.modules() if isinstance(m, QuantLinear))


def convert_gptq_v1_to_v2_format(model: nn.Module, quantize_config: QuantizeConfig):
    """v1 files store (zero - 1) per nibble; the kernels take the zero itself.  Every v1 nibble is
    <= maxq - 1, so the packed addition never carries into the neighbouring nibble."""
    inc = _V1_TO_V2.get(quantize_config.bits)
    if inc is None:
        raise NotImplementedError("Only 2,4,8 bits are supported.")
    for mod in _quant_linears(model):
        mod.qzeros.data += inc
    return model


def convert_gptq_v2_to_v1_format(model: nn.Module, quantize_config: QuantizeConfig):
    inc = _V1_TO_V2.get(quantize_config.bits)
    if inc is None:
        raise NotImplementedError("Only 2,4,8 bits are supported.")
    for mod in _quant_linears(model):
        mod.qzeros.data -= inc
    return model


def _set_submodule(model: nn.Module, name: str, new: nn.Module):
    parent = model
    parts = name.split(".")
    for p in parts[:-1]:
        parent = getattr(parent, p)
    setattr(parent, parts[-1], new)


def make_quant(model: nn.Module, names: Iterable[str], quantize_config: QuantizeConfig):
    """Replace the nn.Linear modules called `names` by empty QuantLinear modules of the same shape
    (gptqmodel/utils/model.py:150-202)."""
    wanted = set(names)
    for name, mod in list(model.named_modules()):
        if name in wanted and isinstance(mod, nn.Linear):
            ql = QuantLinear(quantize_config.bits, quantize_config.group_size, mod.in_features, mod.out_features,
                             mod.bias is not None)
            _set_submodule(model, name, ql)
    return model


def _checkpoint_files(save_dir: str):
    index = os.path.join(save_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as fh:
            return sorted({os.path.join(save_dir, f) for f in json.load(fh)["weight_map"].values()})
    files = sorted(os.path.join(save_dir, f) for f in os.listdir(save_dir) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors file in {save_dir}")
    return files


def load_quantized(model: nn.Module, save_dir: str, device: str = "cpu", strict: bool = True):
    """Turn every linear of `model` that the checkpoint holds in packed form into a QuantLinear, load
    all tensors of the checkpoint, convert v1 zero points, and mark the model as GPTQ-quantised.
    Returns (model, QuantizeConfig)."""
    from safetensors import safe_open  # pylint: disable=import-outside-toplevel

    qcfg = QuantizeConfig.from_pretrained(save_dir)
    if qcfg.bits != 4:
        raise NotImplementedError(f"the gfx950 kernels cover 4-bit GPTQ only (checkpoint has bits={qcfg.bits})")
    files = _checkpoint_files(save_dir)
    keys = {}
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as fh:
            for k in fh.keys():
                keys[k] = path
    quant_names = sorted(k[: -len(".qweight")] for k in keys if k.endswith(".qweight"))
    make_quant(model, quant_names, qcfg)
    state = dict(model.state_dict())
    missing = [k for k in state if k not in keys and not k.endswith(".g_idx")]
    unexpected = [k for k in keys if k not in state]
    if strict and (missing or unexpected):
        raise KeyError(f"checkpoint / model mismatch: missing {missing[:5]}, unexpected {unexpected[:5]}")
    by_file: Dict[str, list] = {}
    for k, path in keys.items():
        if k in state:
            by_file.setdefault(path, []).append(k)
    with torch.no_grad():
        for path, ks in by_file.items():
            with safe_open(path, framework="pt", device="cpu") as fh:
                for k in ks:
                    t = fh.get_tensor(k)
                    if t.shape != state[k].shape:
                        raise ValueError(f"{k}: checkpoint shape {tuple(t.shape)} != model shape {tuple(state[k].shape)}")
                    state[k].copy_(t.to(state[k].dtype))
    if qcfg.format == FORMAT_GPTQ:
        convert_gptq_v1_to_v2_format(model, qcfg)
        qcfg.format = FORMAT_GPTQ_V2
    model.quantization_method = "gptq"
    model.quantize_config = qcfg
    return model.to(device), qcfg


def save_quantized(model: nn.Module, save_dir: str, quantize_config: QuantizeConfig):
    """Write `model.safetensors` + `quantize_config.json` in `quantize_config.format` (the in-memory
    zero points are v2; a `gptq` file gets them converted back to v1)."""
    from safetensors.torch import save_file  # pylint: disable=import-outside-toplevel

    os.makedirs(save_dir, exist_ok=True)
    state = {k: v.detach().cpu().contiguous().clone() for k, v in model.state_dict().items()}
    if quantize_config.format == FORMAT_GPTQ:
        inc = _V1_TO_V2[quantize_config.bits]
        for k in state:
            if k.endswith(".qzeros"):
                state[k] -= inc
    save_file(state, os.path.join(save_dir, "model.safetensors"), metadata={"format": "pt"})
    quantize_config.save_pretrained(save_dir)

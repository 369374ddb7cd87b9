"""Namesake of `fms_acceleration_peft`: the quantised base-layer data layouts (GPTQ QuantLinear,
NF4 container), a stand-in LoRA wrapper, and the plugin configuration shells."""
from .framework_plugin_autogptq import AutoGPTQAccelerationPlugin
from .framework_plugin_bnb import BNBAccelerationPlugin
from .lora import LoraLinear, install_lora_adapters
from .qlinear import QuantLinear, QuantLinearFunction
from .nf4 import Linear4bit, Params4bit, QuantState, quantize_4bit, quantize_nf4
from .gptq_checkpoint import QuantizeConfig, convert_gptq_v1_to_v2_format, convert_gptq_v2_to_v1_format, load_quantized, save_quantized

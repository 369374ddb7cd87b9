"""Namesake of `fms_acceleration_foak` restricted to the fused quantised-LoRA operators."""
from .framework_plugin_fast_kernels import FastKernelsAccelerationPlugin

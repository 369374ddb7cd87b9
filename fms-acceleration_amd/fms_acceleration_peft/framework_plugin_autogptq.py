"""Configuration shell of the GPTQ-LoRA plugin (reference:
accelerated-peft/src/fms_acceleration_peft/framework_plugin_autogptq.py:44-395).

Built: registration under `peft.quantization.auto_gptq`, validation of the configuration keys, a
loader for LOCAL GPTQ checkpoint directories (gptq_checkpoint.py), the `quantization_method`
marker that the fast-kernels plugin keys on, and `augmentation`, which installs the LoRA adapters
the `peft_config` describes on the QuantLinear modules (the reference goes through peft's
get_peft_model, :250-330; peft is not importable where this is built, so the in-tree `LoraLinear`,
which carries the attributes the fused operators read from a PEFT layer, stands in).
"""
from fms_acceleration import AccelerationPlugin


class AutoGPTQAccelerationPlugin(AccelerationPlugin):
    require_packages = []

    def __init__(self, configurations):
        super().__init__(configurations)
        self._check_config_equal(key="peft.quantization.auto_gptq.kernel", value="triton_v2")
        self._check_config_equal(key="peft.quantization.auto_gptq.from_quantized", value=True)
        self.use_external_lib = self._check_config_and_maybe_check_values(
            key="peft.quantization.auto_gptq.use_external_lib", values=[True, False], default=False
        )

    @property
    def requires_custom_loading(self):
        return True

    @property
    def requires_augmentation(self):
        return True

    def model_loader(self, model_name: str, **kwargs):
        """Load a GPTQ checkpoint from a LOCAL directory (config.json + quantize_config.json +
        safetensors): the architecture is built from its config with empty weights, the packed
        linears become QuantLinear modules and the tensors are read from the file (reference:
        :108-222, which goes through the hub and accelerate; there is no network here)."""
        import os  # pylint: disable=import-outside-toplevel

        import torch  # pylint: disable=import-outside-toplevel
        from transformers import AutoConfig, AutoModelForCausalLM  # pylint: disable=import-outside-toplevel

        from .gptq_checkpoint import load_quantized  # pylint: disable=import-outside-toplevel

        if not os.path.isdir(model_name):
            raise NotImplementedError(
                f"'{model_name}' is not a local directory: this build loads GPTQ checkpoints from disk only "
                "(no hub access)"
            )
        torch_dtype = kwargs.get("torch_dtype", torch.float16)
        config = AutoConfig.from_pretrained(model_name)
        prev = torch.get_default_dtype()
        torch.set_default_dtype(torch_dtype)
        try:
            model = AutoModelForCausalLM.from_config(config)
        finally:
            torch.set_default_dtype(prev)
        device = kwargs.get("device", "cuda" if torch.cuda.is_available() else "cpu")
        model, _ = load_quantized(model, model_name, device=device)
        return model

    def augmentation(self, model, train_args, modifiable_args):
        """Installs the adapters of `peft_config` (a peft LoraConfig, or any object / dict with `r`,
        `lora_alpha`, `lora_dropout`, `target_modules`) on the matching QuantLinear modules, freezes
        everything else and returns `(None,)` in place of the config, so that the trainer does not
        wrap the model again (reference :269-330).  `target_modules` follows peft: a list matches by name
        or dotted suffix, a string is a regular expression ("all-linear" aside), None takes the default of
        the model type."""
        from .lora import install_lora_adapters  # pylint: disable=import-outside-toplevel
        from .qlinear import QuantLinear  # pylint: disable=import-outside-toplevel

        (peft_config,) = modifiable_args
        assert peft_config is not None, "need peft_config to install PEFT adapters"
        installed = install_lora_adapters(model, peft_config, QuantLinear)  # raises before anything is modified
        # the marker FastKernelsAccelerationPlugin.augmentation looks for (:235-236 of the reference)
        setattr(model, "quantization_method", "gptq")
        setattr(model, "is_loaded_in_4bit", True)
        if getattr(train_args, "gradient_checkpointing", False) and hasattr(model, "enable_input_require_grads"):
            model.enable_input_require_grads()  # what prepare_model_for_kbit_training does for checkpointed models
        model._fmsa_lora_modules = installed
        return model, (None,)


AccelerationPlugin.register_plugin(AutoGPTQAccelerationPlugin, configuration_and_paths=["peft.quantization.auto_gptq"])

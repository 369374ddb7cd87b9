"""The bitsandbytes-LoRA plugin (reference:
accelerated-peft/src/fms_acceleration_peft/framework_plugin_bnb.py:95-268).

Built: registration under `peft.quantization.bitsandbytes`, validation of `quant_type` (`nf4` or `fp4`:
the kernels take the 16-entry code book as an input) and `no_peft_model`, a loader for LOCAL checkpoint
directories that quantises the model's linears on load the way transformers' BitsAndBytesConfig(load_in_4bit,
double quant) does, and `augmentation`, which installs the LoRA adapters the `peft_config` describes on the
4-bit linears and returns `(None,)` in place of the config (reference :192-218, through peft's
get_peft_model; peft and bitsandbytes are not importable where this is built, so the in-tree `Linear4bit` /
`LoraLinear`, which carry the attributes the fused operators read, stand in).
"""
import warnings

from fms_acceleration import AccelerationPlugin


class BNBAccelerationPlugin(AccelerationPlugin):
    require_packages = []

    def __init__(self, configurations):
        super().__init__(configurations)
        self._quant_type = self._check_config_and_maybe_check_values(
            key="peft.quantization.bitsandbytes.quant_type", values=["fp4", "nf4"]
        )
        self._no_peft_model = self._check_config_and_maybe_check_values(
            key="peft.quantization.bitsandbytes.no_peft_model", values=[True, False]
        )

    @property
    def requires_custom_loading(self):
        return True

    @property
    def requires_augmentation(self):
        return not self._no_peft_model  # with no_peft_model the trainer prepares the PEFT model itself (:186-189)

    def model_loader(self, model_name: str, **kwargs):
        """Load a dense checkpoint from a LOCAL directory and quantise every linear but the output embedding to
        4 bits with double-quantised statistics, as `BitsAndBytesConfig(load_in_4bit=True,
        bnb_4bit_use_double_quant=True, bnb_4bit_quant_type=quant_type, bnb_4bit_compute_dtype=torch_dtype)`
        does on load in the reference (:142-157, through the hub; there is no network here)."""
        import os  # pylint: disable=import-outside-toplevel

        import torch  # pylint: disable=import-outside-toplevel
        from transformers import AutoModelForCausalLM  # pylint: disable=import-outside-toplevel

        from .nf4 import Linear4bit  # pylint: disable=import-outside-toplevel

        if not os.path.isdir(model_name):
            raise NotImplementedError(
                f"'{model_name}' is not a local directory: this build loads checkpoints from disk only (no hub access)")
        torch_dtype = kwargs.get("torch_dtype", torch.float32)
        if self._no_peft_model is True:
            warnings.warn("plugin config `no_peft_model: True` on a single device: PEFT preparation is left to the "
                          "trainer, whose extra dtype casts slow training down")
        model = AutoModelForCausalLM.from_pretrained(model_name, torch_dtype=torch_dtype,
                                                     attn_implementation=kwargs.get("attn_implementation"))
        device = kwargs.get("device", "cuda" if torch.cuda.is_available() else "cpu")
        compute_dtype = torch_dtype if torch_dtype in (torch.float16, torch.bfloat16) else torch.bfloat16
        skip = model.get_output_embeddings()
        for parent in list(model.modules()):
            for name, child in list(parent.named_children()):
                if isinstance(child, torch.nn.Linear) and child is not skip and child.in_features % 64 == 0:
                    q = Linear4bit.from_dense(child.weight.data.to(device), None if child.bias is None else child.bias.data,
                                              compute_dtype=compute_dtype, quant_type=self._quant_type)
                    setattr(parent, name, q.to(device))
        model = model.to(device)
        setattr(model, "is_loaded_in_4bit", True)
        setattr(model, "quantization_method", "bitsandbytes")
        return model

    def augmentation(self, model, train_args, modifiable_args):
        """Freezes the base model and wraps the 4-bit linears named by `peft_config.target_modules` in LoRA layers
        (reference :192-218: the plugin's own prepare_model_for_kbit_training, which freezes and, under gradient
        checkpointing, makes the inputs require gradients, then get_peft_model)."""
        from .lora import install_lora_adapters  # pylint: disable=import-outside-toplevel
        from .nf4 import Linear4bit  # pylint: disable=import-outside-toplevel

        assert (
            getattr(train_args, "bf16", False) is True or getattr(train_args, "fp16", False) is True
        ), f"{self.__class__} requires mixed precision argument `--fp16` or `--bf16`"
        (peft_config,) = modifiable_args
        assert peft_config is not None, "need peft_config to install PEFT adapters"
        installed = install_lora_adapters(model, peft_config, Linear4bit)  # raises before anything is modified
        setattr(model, "quantization_method", "bitsandbytes")
        setattr(model, "is_loaded_in_4bit", True)
        if getattr(train_args, "gradient_checkpointing", False) and hasattr(model, "enable_input_require_grads"):
            model.enable_input_require_grads()
        model._fmsa_lora_modules = installed
        return model, (None,)


AccelerationPlugin.register_plugin(BNBAccelerationPlugin, configuration_and_paths=["peft.quantization.bitsandbytes"])

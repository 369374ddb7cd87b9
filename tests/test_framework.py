"""Plugin registry / framework behaviours (mirrors plugins/framework/tests/test_framework.py of
the reference): AND / OR configuration paths, activation order, errors."""
import os

import pytest
import torch

from fms_acceleration import AccelerationPlugin, AccelerationPluginConfigError
from fms_acceleration.framework_plugin import get_relevant_configuration_sections
from fms_acceleration.utils.test_utils import instantiate_framework, register_plugins_and_configure


def make_plugin(name, loading=False, augment=False, archs=None, packages=None):
    class _P(AccelerationPlugin):
        restricted_model_archs = archs
        require_packages = packages

        @property
        def requires_custom_loading(self):
            return loading

        @property
        def requires_augmentation(self):
            return augment

        def model_loader(self, model_name, **kw):
            return f"loaded:{model_name}"

        def augmentation(self, model, train_args, modifiable_args):
            model.augmented_by = getattr(model, "augmented_by", []) + [name]
            return model, modifiable_args

    _P.__name__ = name
    return _P


class _Model(torch.nn.Module):
    def __init__(self, archs):
        super().__init__()
        self.config = type("C", (), {"architectures": archs})()


def test_register_needs_a_path():
    with pytest.raises(AssertionError):
        AccelerationPlugin.register_plugin(make_plugin("X"))


def test_and_or_path_selection():
    A, B, C = make_plugin("A"), make_plugin("B"), make_plugin("C")
    regs = [
        (A, {"configuration_and_paths": ["x.a", "x.b"]}),
        (B, {"configuration_or_paths": ["y.a", "y.b"]}),
        (C, {"configuration_and_paths": ["z.a"]}),
    ]
    with register_plugins_and_configure(regs):
        cfg = {"x": {"a": {"v": 1}}, "y": {"b": {"w": 2}}}
        got = get_relevant_configuration_sections(cfg)
        # A needs both x.a and x.b -> rejected; B is rescued by y.b; C absent
        assert [(c.__name__, s) for s, c in got] == [("B", {"y": {"b": {"w": 2}}})]
        cfg["x"]["b"] = {"u": 3}
        got = get_relevant_configuration_sections(cfg)
        assert [c.__name__ for _, c in got] == ["A", "B"]
        assert got[0][0] == {"x": {"a": {"v": 1}, "b": {"u": 3}}}


def test_activation_follows_registration_order_and_dedups():
    A, B = make_plugin("A", augment=True), make_plugin("B", augment=True)
    regs = [(B, {"configuration_and_paths": ["p.b"]}), (A, {"configuration_and_paths": ["p.a"]}),
            (B, {"configuration_and_paths": ["p.b2"]})]
    with register_plugins_and_configure(regs):
        with instantiate_framework({"p": {"a": {"k": 1}, "b": {"k": 1}, "b2": {"k": 1}}}) as fw:
            assert [n for n, _ in fw.active_plugins] == ["B", "A"]
            assert fw.requires_augmentation and not fw.requires_custom_loading
            model, _ = fw.augmentation(_Model(["LlamaForCausalLM"]), None, ())
            assert model.augmented_by == ["B", "A"]


def test_errors():
    A = make_plugin("A", loading=True)
    B = make_plugin("B", loading=True)
    with register_plugins_and_configure([(A, {"configuration_and_paths": ["p.a"]})]):
        with pytest.raises(ValueError, match="No plugins could be configured"):
            with instantiate_framework({"q": {"k": 1}}):
                pass
    with register_plugins_and_configure([(A, {"configuration_and_paths": ["p.a"]}),
                                         (B, {"configuration_and_paths": ["p.b"]})]):
        with pytest.raises(AssertionError, match="at most 1 plugin with custom model loading"):
            with instantiate_framework({"p": {"a": {"k": 1}, "b": {"k": 1}}}):
                pass
    C = make_plugin("C", augment=True, archs={"OnlyThisArch"})
    with register_plugins_and_configure([(C, {"configuration_and_paths": ["p.c"]})]):
        with instantiate_framework({"p": {"c": {"k": 1}}}) as fw:
            with pytest.raises(ValueError, match="are not supported"):
                fw.augmentation(_Model(["LlamaForCausalLM"]), None, ())
            with pytest.raises(NotImplementedError):
                fw.model_loader("m")
    D = make_plugin("D", packages={"a_package_that_does_not_exist_xyz"})
    with register_plugins_and_configure([(D, {"configuration_and_paths": ["p.d"]})]):
        with pytest.raises(ValueError, match="is missing"):
            with instantiate_framework({"p": {"d": {"k": 1}}}):
                pass
        with instantiate_framework({"p": {"d": {"k": 1}}}, require_packages_check=False) as fw:
            assert [n for n, _ in fw.active_plugins] == ["D"]


def test_model_loader_dispatch():
    A = make_plugin("A", loading=True)
    with register_plugins_and_configure([(A, {"configuration_and_paths": ["p.a"]})]):
        with instantiate_framework({"p": {"a": {"k": 1}}}) as fw:
            assert fw.model_loader("m") == "loaded:m"


def test_config_value_checks():
    P = make_plugin("P")
    p = P({"a": {"b": "x", "d": {"only": {"z": 1}}, "multi": {"u": 1, "v": 2}}})
    assert p._check_config_and_maybe_check_values("a.b", ["x", "y"]) == "x"
    assert p._check_config_and_maybe_check_values("a.d", ["only"]) == "only"  # dict node named by its key
    assert p._check_config_and_maybe_check_values("a.missing", ["x"], default="x") == "x"
    with pytest.raises(AccelerationPluginConfigError, match="P: Value at 'a.b' was 'x'"):
        p._check_config_and_maybe_check_values("a.b", ["q"])
    with pytest.raises(AccelerationPluginConfigError):
        p._check_config_and_maybe_check_values("a.missing", ["x"])
    with pytest.raises(AccelerationPluginConfigError):
        p._check_config_and_maybe_check_values("a.multi", ["u"])
    with pytest.raises(AccelerationPluginConfigError):
        p._check_config_and_maybe_check_values("nope")
    assert p._check_config_equal("a.b", "x") == "x"


def test_shipped_plugins_are_registered_and_configurable():
    """The two plugins of this build register under the reference's configuration paths and accept
    the reference's sample configuration keys."""
    cfg = {
        "peft": {"quantization": {
            "auto_gptq": {"kernel": "triton_v2", "from_quantized": True},
            "fused_ops_and_kernels": {"base_layer": "auto_gptq", "fused_lora": True, "fast_loss": True,
                                      "fast_rms_layernorm": True, "fast_rope_embeddings": True},
        }}
    }
    with instantiate_framework(cfg, require_packages_check=False) as fw:
        assert [n for n, _ in fw.active_plugins] == ["AutoGPTQAccelerationPlugin", "FastKernelsAccelerationPlugin"]
        assert fw.requires_custom_loading and fw.requires_augmentation
    bad = {"peft": {"quantization": {"fused_ops_and_kernels": {"base_layer": "something_else"}}}}
    with pytest.raises(AccelerationPluginConfigError, match="FastKernelsAccelerationPlugin: Value at 'base_layer'"):
        with instantiate_framework(bad):
            pass
    alt = {"training": {"fused_ops_and_kernels": {"fused_lora": True}}}
    with instantiate_framework(alt) as fw:
        plugin = fw.active_plugins[0][1]
        assert plugin.configurations["base_layer"] == "auto_gptq" and plugin.configurations["fast_loss"] is False


def test_shipped_sample_configurations(monkeypatch):
    """The YAML files under fms-acceleration_amd/configs (the reference's plugin configuration keys under
    the framework's `plugins:` body, cf. plugins/accelerated-peft/tests/test_peft_plugins.py:47-120 and
    plugins/fused-ops-and-kernels/tests/test_foak_plugins.py:39-85): read from the path and through the
    ACCELERATION_FRAMEWORK_CONFIG_FILE route, each activates the plugins it names with the values it sets."""
    import glob

    import yaml

    from fms_acceleration.constants import KEY_PLUGINS
    from fms_acceleration.framework import AccelerationFramework, read_configuration_file

    cfg_dir = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fms-acceleration_amd", "configs")
    expected = {
        "accelerated-peft-autogptq-foak.yaml": (["AutoGPTQAccelerationPlugin", "FastKernelsAccelerationPlugin"], "auto_gptq", True),
        "accelerated-peft-autogptq-foak-liger.yaml": (["AutoGPTQAccelerationPlugin", "FastKernelsAccelerationPlugin"], "auto_gptq", "fused_ce_liger"),
        "accelerated-peft-bnb-nf4-foak.yaml": (["BNBAccelerationPlugin", "FastKernelsAccelerationPlugin"], "bitsandbytes", True),
        "foak-fast-kernels.yaml": (["FastKernelsAccelerationPlugin"], "auto_gptq", True),
    }
    files = sorted(glob.glob(os.path.join(cfg_dir, "*.yaml")))
    assert sorted(os.path.basename(f) for f in files) == sorted(expected)
    for path in files:
        names, base_layer, fast_loss = expected[os.path.basename(path)]
        body = read_configuration_file(path)
        for via_env in (False, True):
            # the framework keeps its activation lists on the class: a fresh pair per instantiation
            monkeypatch.setattr(AccelerationFramework, "active_plugins", [])
            monkeypatch.setattr(AccelerationFramework, "plugins_require_custom_loading", [])
            if via_env:
                monkeypatch.setenv("ACCELERATION_FRAMEWORK_CONFIG_FILE", path)
                fw = AccelerationFramework(None, require_packages_check=False)
            else:
                monkeypatch.delenv("ACCELERATION_FRAMEWORK_CONFIG_FILE", raising=False)
                fw = AccelerationFramework(path, require_packages_check=False)
            assert [n for n, _ in fw.active_plugins] == names
            foak = dict(fw.active_plugins)["FastKernelsAccelerationPlugin"]
            assert foak.configurations["base_layer"] == base_layer and foak.configurations["fast_loss"] == fast_loss
            assert fw.requires_augmentation and fw.requires_custom_loading == (len(names) == 2)
        monkeypatch.delenv("ACCELERATION_FRAMEWORK_CONFIG_FILE", raising=False)
        # a value outside the allowed set is refused with the plugin's name in the message
        section = body["peft"]["quantization"] if "peft" in body else body["training"]
        section["fused_ops_and_kernels"]["fast_loss"] = "something_else"
        with pytest.raises(AccelerationPluginConfigError, match="FastKernelsAccelerationPlugin"):
            with instantiate_framework(body, require_packages_check=False):
                pass
    assert yaml.safe_load(open(files[0], encoding="utf-8"))[KEY_PLUGINS]

"""AccelerationFramework: YAML -> active plugins -> loader / augmentation / patching.

Mirrors plugins/framework/src/fms_acceleration/framework.py:96-261 (activation in registration
order, de-duplicated by class name; errors for no plugin, >1 custom loader, unsupported
architecture, missing packages).  The accelerator (dataloader) patcher of the reference is not
on the fused-LoRA path and is not built.
"""
from __future__ import annotations

import importlib.util
import logging
import os
from typing import List, Optional, Tuple

import yaml

from .constants import ACCELERATION_FRAMEWORK_ENV_KEY, KEY_PLUGINS
from .framework_plugin import PLUGIN_REGISTRATIONS, AccelerationPlugin, get_relevant_configuration_sections

logger = logging.getLogger(__name__)


def _is_package_available(name: str) -> bool:
    return importlib.util.find_spec(name) is not None


def check_plugin_packages(plugin: AccelerationPlugin):
    if plugin.require_packages is None:
        return True, []
    missing = [p for p in plugin.require_packages if not _is_package_available(p)]
    return len(missing) == 0, missing


def read_configuration_file(configuration_file: str):
    with open(configuration_file, "r", encoding="utf-8") as f:
        contents = yaml.safe_load(f)
    if not contents or contents.get(KEY_PLUGINS) is None:
        raise ValueError(f"Configuration file must contain a '{KEY_PLUGINS}' body")
    return dict(contents[KEY_PLUGINS].items())


class AccelerationFramework:
    active_plugins: List[Tuple[str, AccelerationPlugin]] = []
    plugins_require_custom_loading: List = []

    def __init__(self, configuration_file: Optional[str] = None, require_packages_check: bool = True):
        env_file = os.environ.get(ACCELERATION_FRAMEWORK_ENV_KEY)
        if configuration_file is None and env_file is None:
            raise ValueError(
                "configuration_file is not passed into configuration_file but "
                f"{ACCELERATION_FRAMEWORK_ENV_KEY} is not set. Please choose one "
                "of the means to initialize the framework."
            )
        plugin_configs = {}
        if configuration_file is not None:
            plugin_configs = read_configuration_file(configuration_file)
        if env_file is not None and len(plugin_configs) == 0:
            plugin_configs = read_configuration_file(env_file)

        for section, cls in get_relevant_configuration_sections(plugin_configs):
            name = str(cls.__name__)
            plugin = cls(section)
            ok, missing = check_plugin_packages(plugin)
            if not ok and require_packages_check:
                raise ValueError(
                    f"Packages '{', '.join(missing)}' required by activated plugin '{name}' "
                    "is missing. Please install it."
                )
            if any(n == name for n, _ in self.active_plugins):
                continue  # one activation per plugin class name
            self.active_plugins.append((name, plugin))
            if plugin.requires_custom_loading:
                self.plugins_require_custom_loading.append(name)

        if len(self.active_plugins) == 0:
            raise ValueError(
                "No plugins could be configured. Please check the acceleration framework configuration file."
            )
        assert len(self.plugins_require_custom_loading) <= 1, (
            "Can load at most 1 plugin with custom model loading, "
            f"but tried to '{self.plugins_require_custom_loading}'."
        )

    def model_loader(self, model_name: str, **kwargs):
        if not self.plugins_require_custom_loading:
            raise NotImplementedError(
                f"Attempted model loading, but none of activated plugins '{list(self.active_plugins)}' "
                "require custom loading."
            )
        wanted = self.plugins_require_custom_loading[0]
        plugin = next(p for n, p in self.active_plugins if n == wanted)
        return plugin.model_loader(model_name, **kwargs)

    def augmentation(self, model, train_args, modifiable_args: Tuple):
        archs = set(getattr(model.config, "architectures", None) or [])
        for name, plugin in self.active_plugins:
            allowed = plugin.restricted_model_archs
            if allowed and not any(a in archs for a in allowed):
                raise ValueError(f"Model architectures in '{archs}' are not supported for '{name}'.")
            if plugin.requires_augmentation:
                model, modifiable_args = plugin.augmentation(model, train_args, modifiable_args=modifiable_args)
        return model, modifiable_args

    @property
    def requires_custom_loading(self):
        return len(self.plugins_require_custom_loading) > 0

    @property
    def requires_augmentation(self):
        return any(p.requires_augmentation for _, p in self.active_plugins)

    def get_callbacks_and_ready_for_train(self, model=None, accelerator=None):
        from .model_patcher import ModelPatcher  # late import, as in the reference (:224-227)

        if model is not None:
            ModelPatcher.patch(model)
        if accelerator is None or getattr(accelerator, "is_main_process", True):
            active = {n for n, _ in self.active_plugins}
            logger.info("***** FMS AccelerationFramework *****")
            for reg in PLUGIN_REGISTRATIONS:
                if reg.plugin.__name__ in active:
                    logger.info("Active Plugin: %s. Python package: %s. Version: %s.",
                                reg.plugin.__name__, reg.package_name, reg.package_version)
            for line in ModelPatcher.summary(raw=False).split("\n"):
                logger.info(line)
        callbacks = []
        for _, plugin in self.active_plugins:
            callbacks.extend(plugin.get_callbacks_and_ready_for_train(model, accelerator))
        return callbacks

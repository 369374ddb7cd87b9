"""Isolation helpers for tests of the registry and the patcher
(reference: plugins/framework/src/fms_acceleration/utils/test_utils.py:146-212)."""
from __future__ import annotations

import os
import tempfile
from contextlib import contextmanager
from typing import Any, Dict, List, Tuple

import yaml

from ..constants import KEY_PLUGINS


@contextmanager
def instantiate_model_patcher():
    """Run a block against an empty ModelPatcher (rules and history), restoring the previous
    singleton state afterwards."""
    from ..model_patcher import ModelPatcher

    saved = (ModelPatcher.rules, ModelPatcher.history)
    ModelPatcher.rules, ModelPatcher.history = {}, []
    try:
        yield
    finally:
        ModelPatcher.rules, ModelPatcher.history = saved


@contextmanager
def instantiate_framework(plugins_config: Dict, require_packages_check: bool = True, instantiate: bool = True):
    """Write {plugins: plugins_config} to a temporary YAML and build an AccelerationFramework
    from it, with the class-level activation lists reset around the block."""
    from ..framework import AccelerationFramework

    saved = (AccelerationFramework.active_plugins, AccelerationFramework.plugins_require_custom_loading)
    AccelerationFramework.active_plugins = []
    AccelerationFramework.plugins_require_custom_loading = []
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "accel.yaml")
        with open(path, "w", encoding="utf-8") as f:
            yaml.safe_dump({KEY_PLUGINS: plugins_config}, f)
        try:
            yield AccelerationFramework(path, require_packages_check=require_packages_check) if instantiate else path
        finally:
            AccelerationFramework.active_plugins, AccelerationFramework.plugins_require_custom_loading = saved


@contextmanager
def register_plugins_and_configure(registrations: List[Tuple[type, Dict[str, Any]]]):
    """Temporarily replace the global registration list with `registrations`, given as
    (plugin_class, {"configuration_and_paths": [...]} or {"configuration_or_paths": [...]})."""
    from .. import framework_plugin as fp

    saved = list(fp.PLUGIN_REGISTRATIONS)
    fp.PLUGIN_REGISTRATIONS.clear()
    try:
        for cls, paths in registrations:
            fp.AccelerationPlugin.register_plugin(cls, **paths)
        yield
    finally:
        fp.PLUGIN_REGISTRATIONS.clear()
        fp.PLUGIN_REGISTRATIONS.extend(saved)

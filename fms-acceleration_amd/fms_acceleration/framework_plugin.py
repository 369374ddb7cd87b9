"""Plugin base class and registry.

Mirrors plugins/framework/src/fms_acceleration/framework_plugin.py: `register_plugin` with AND / OR
dotted configuration paths (:124-159), selection of the configuration sub-tree handed to each
plugin (:53-118), the plugin surface (:161-191) and `_check_config_and_maybe_check_values`
(:193-226).  peft / accelerate / transformers types appear in the reference signatures only as
annotations, so nothing here imports them.
"""
from __future__ import annotations

import importlib.metadata
import sys
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Set, Tuple


@dataclass
class PluginRegistration:
    plugin: type
    AND: Optional[List[str]] = None
    OR: Optional[List[str]] = None
    package_name: Optional[str] = None
    package_version: Optional[str] = None


PLUGIN_REGISTRATIONS: List[PluginRegistration] = []

_MISSING = object()


def _trace_key_path(configuration: Dict, key: str):
    """Value at dotted path `key`, or None when any component is absent."""
    node = configuration
    for part in key.split("."):
        if not isinstance(node, dict) or part not in node:
            return None
        node = node[part]
    return node


def _graft(tree: Dict, key: str, content: Any) -> None:
    parts = key.split(".")
    for part in parts[:-1]:
        tree = tree.setdefault(part, {})
    tree[parts[-1]] = content


def get_relevant_configuration_sections(configuration: Dict) -> List[Tuple[Dict, type]]:
    """For every registration, in registration order: the union of the sub-trees found at its
    paths.  All AND paths must be present (non-None); any present OR path rescues the
    registration and contributes its content."""
    selected = []
    for reg in PLUGIN_REGISTRATIONS:
        and_hits = [(k, _trace_key_path(configuration, k)) for k in (reg.AND or [])]
        or_hits = [(k, _trace_key_path(configuration, k)) for k in (reg.OR or [])]
        and_ok = all(v is not None for _, v in and_hits)
        or_present = [(k, v) for k, v in or_hits if v is not None]
        if not and_ok and not or_present:
            continue
        section: Dict = {}
        if and_ok:
            for k, v in and_hits:
                _graft(section, k, v)
        for k, v in or_present:
            _graft(section, k, v)
        if section:
            selected.append((section, reg.plugin))
    return selected


class AccelerationPluginConfigError(Exception):
    pass


class AccelerationPlugin:
    restricted_model_archs: Optional[Set] = None
    require_packages: Optional[Set] = None

    @staticmethod
    def register_plugin(plugin: type, configuration_and_paths: List[str] = None,
                        configuration_or_paths: List[str] = None, **kwargs):
        assert (configuration_and_paths and len(configuration_and_paths) > 0) or (
            configuration_or_paths and len(configuration_or_paths) > 0
        ), "Specify at least one AND or OR path"
        pkg = getattr(sys.modules.get(plugin.__module__), "__package__", None)
        try:
            version = importlib.metadata.version(pkg) if pkg else None
        except importlib.metadata.PackageNotFoundError:
            version = None
        PLUGIN_REGISTRATIONS.append(
            PluginRegistration(plugin, configuration_and_paths, configuration_or_paths, pkg, version)
        )

    def __init__(self, configurations: Dict[str, Dict]):
        self.configurations = configurations

    @property
    def requires_custom_loading(self):
        return False

    @property
    def requires_augmentation(self):
        return False

    def model_loader(self, model_name: str, **kwargs):
        raise NotImplementedError

    def augmentation(self, model, train_args, modifiable_args):
        raise NotImplementedError

    def get_callbacks_and_ready_for_train(self, model=None, accelerator=None):
        return []

    def _check_config_and_maybe_check_values(self, key: str, values: List[Any] = None, default: Any = None):
        found = _trace_key_path(self.configurations, key)
        name = self.__class__.__name__
        if values is None:
            if found is None:
                if default is None:
                    raise AccelerationPluginConfigError(f"{name}: '{key}' was not a valid configuration config")
                return default
            return found
        if isinstance(found, dict):
            # a dict-valued node is identified by its single key
            if len(found) > 1:
                raise AccelerationPluginConfigError(
                    f"{name}: '{key}' found but amongst multiple '{list(found)}' exist. "
                    f"Ambiguous check in expected set '{values}'."
                )
            found = next(iter(found))
        if found in values:
            return found
        if found is None and default is not None:
            return default
        raise AccelerationPluginConfigError(
            f"{name}: Value at '{key}' was '{found}'. Not found in expected set '{values}'."
        )

    def _check_config_equal(self, key: str, value: Any, **kwargs):
        return self._check_config_and_maybe_check_values(key, [value], **kwargs)

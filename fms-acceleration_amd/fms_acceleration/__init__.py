"""Plugin host of the fused quantised-LoRA path (namesake of the reference's `fms_acceleration`).

Importing this package imports every `fms_acceleration_<postfix>` package that can be found, in
the precedence order of constants.PLUGINS, which is what registers their plugins
(reference: plugins/framework/src/fms_acceleration/__init__.py:28-31).
"""
import importlib
import importlib.util

from .constants import PLUGIN_PREFIX, PLUGINS
from .framework import AccelerationFramework
from .framework_plugin import (
    AccelerationPlugin,
    AccelerationPluginConfigError,
    get_relevant_configuration_sections,
)

for _postfix in PLUGINS:
    _name = f"{PLUGIN_PREFIX}{_postfix}"
    if importlib.util.find_spec(_name):
        importlib.import_module(_name)

"""Names shared by the plugin host (reference: plugins/framework/src/fms_acceleration/constants.py:15-24)."""

KEY_PLUGINS = "plugins"  # top-level key of the acceleration YAML
PLUGIN_PREFIX = "fms_acceleration_"
ACCELERATION_FRAMEWORK_ENV_KEY = "ACCELERATION_FRAMEWORK_CONFIG_FILE"

# Import (= registration = activation) order of the plugin packages.  Only the two packages that
# carry the fused quantised-LoRA path exist in this build; the other postfixes of the reference
# ("aadp", "moe", "odm", "mcp") are simply not found and skipped, as they would be when not installed.
PLUGINS = ["peft", "foak", "aadp", "moe", "odm", "mcp"]

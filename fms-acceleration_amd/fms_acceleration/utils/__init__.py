from .test_utils import instantiate_framework, instantiate_model_patcher, register_plugins_and_configure  # noqa: F401

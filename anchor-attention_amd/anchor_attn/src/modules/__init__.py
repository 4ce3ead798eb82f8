from .patch import get_config_example, patch_model  # noqa: F401

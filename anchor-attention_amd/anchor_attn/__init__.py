"""AnchorAttention for MI355X.  ``from anchor_attn import patch_model`` works as in the reference
(anchor_attn/__init__.py:1); the import of transformers is deferred until it is called."""


def patch_model(model, pattern: str, config: dict = None):
    from .src.modules.patch import patch_model as _patch_model
    return _patch_model(model, pattern, config)


def get_config_example(pattern: str = None):
    from .src.modules.patch import get_config_example as _get
    return _get(pattern)

"""``patch_model``: switch a Hugging Face causal LM to AnchorAttention prefill.

Counterpart of the reference's anchor_attn/src/modules/patch.py:116-164,290-327 for the patterns on the
AnchorAttention path: "default", "flash" (the framework's library attention), "dense" (plain causal attention
on this package's own MFMA kernel - the baseline "built on the same kernels"), "anchor_attn" and
"anchor_attn_lite" (in the reference the two names select the same forward with the same defaults,
patch.py:36-45,142-144); the competitor patterns of the reference are not part of this package and raise
``ValueError``.  In transformers 5 the attention product is selected by
name through ``AttentionInterface``, so patching is: register the plug once, point the model's config at it,
and copy the pattern's parameters onto the config (patch.py:106-109 does the same ``setattr`` loop).  Like the
reference (patch.py:146-157), every pattern but "default" also makes the model return logits for the last position
only and evaluates the MLPs in chunks of 32768 positions (``model_forward.py``).
"""
import copy
import json

from my_utils import Logger

from anchor_attn.src.modules.model_forward import MLP_CHUNK_TOKENS, chunk_mlp_over_tokens, keep_last_token_logits

ATTENTION_CONFIG_EXAMPLE = {
    "default": {},
    "flash": {},
    "dense": {},
    "anchor_attn": {"block_size_M": 128, "theta": 12, "step": 16},
    "anchor_attn_lite": {"block_size_M": 128, "theta": 12, "step": 16},
}

_SUPPORTED_MODELS = ("llama", "qwen2")
SUPPORTED_BLOCK_SIZES = (16, 32, 64, 128, 256)


def get_config_example(pattern: str = None):
    if pattern is None:
        return copy.deepcopy(ATTENTION_CONFIG_EXAMPLE)
    return copy.deepcopy(ATTENTION_CONFIG_EXAMPLE[pattern])


def _register():
    from transformers import AttentionInterface, AttentionMaskInterface
    from transformers.masking_utils import sdpa_mask

    from anchor_attn.src.modules.llama.anchor_attention import (ATTN_NAME, DENSE_ATTN_NAME, anchor_attention_forward,
                                                                dense_attention_forward)
    for name, fn in ((ATTN_NAME, anchor_attention_forward), (DENSE_ATTN_NAME, dense_attention_forward)):
        if name not in AttentionInterface().valid_keys():
            AttentionInterface.register(name, fn)
            # same mask convention as SDPA: None when the mask is purely causal, a boolean mask otherwise
            AttentionMaskInterface.register(name, sdpa_mask)
    return ATTN_NAME, DENSE_ATTN_NAME


def _config_dict(config):
    """``config`` as the reference's callers pass it: None, a dict, or the JSON text of one (test_hf.py hands its
    ``--config`` string straight through; patch.py:62-74 parses it and reports bad JSON as ``ValueError``)."""
    if config is None:
        return {}
    if isinstance(config, str):
        try:
            config = json.loads(config)
        except json.JSONDecodeError as e:
            raise ValueError(f"Configuration string is not valid JSON: {e}")
    if not isinstance(config, dict):
        raise ValueError(f"config must be a dict or the JSON text of one, got {type(config).__name__}")
    return config


def patch_model(model, pattern: str, config=None):
    """Patch ``model`` (a transformers ``PreTrainedModel`` of the Llama or Qwen2 family) in place.

    pattern: "default" (leave as is), "flash" (the framework's library attention), "dense" (causal attention on this
             package's own kernel), "anchor_attn" or "anchor_attn_lite" (same operator, same defaults).
    config : None, a dict or a JSON string; for the anchor patterns ``{"block_size_M": 128, "theta": 12, "step": 16}``
             (the defaults; keys left out keep them).  Two optional keys with no counterpart in the reference steer
             the model-level patches the reference applies unconditionally: ``"last_token_logits"`` (default True) and
             ``"mlp_chunk_tokens"`` (default 32768; 0 leaves the MLPs alone).
    """
    from transformers import PreTrainedModel
    if not isinstance(model, PreTrainedModel):
        raise ValueError("Only Hugging Face transformers models are supported")
    if pattern not in ATTENTION_CONFIG_EXAMPLE:
        raise ValueError(f"Unknown attention pattern {pattern}")
    name = type(model).__name__.lower()
    if not any(m in name for m in _SUPPORTED_MODELS):
        raise ValueError(f"Unsupported model type: {type(model).__name__}")
    if pattern == "default":
        return model
    cfg = get_config_example(pattern)
    cfg.update(_config_dict(config))
    last_token_logits = bool(cfg.pop("last_token_logits", True))
    mlp_chunk_tokens = int(cfg.pop("mlp_chunk_tokens", MLP_CHUNK_TOKENS))
    if pattern == "flash":
        model.set_attn_implementation("sdpa")
    elif pattern == "dense":
        model.set_attn_implementation(_register()[1])
    else:
        if cfg["step"] not in (16, 32) or cfg["block_size_M"] not in SUPPORTED_BLOCK_SIZES:
            raise ValueError(f"{pattern} supports block_size_M in {SUPPORTED_BLOCK_SIZES} and step in (16, 32)")
        model.set_attn_implementation(_register()[0])
        for k, v in cfg.items():
            setattr(model.config, k, v)
    if last_token_logits:
        keep_last_token_logits(model)
    chunk_mlp_over_tokens(model, mlp_chunk_tokens)
    Logger.log(f"replace attention with {pattern}: {cfg}")
    return model

"""``patch_model``: switch a Hugging Face causal LM to AnchorAttention prefill.

Counterpart of the reference's anchor_attn/src/modules/patch.py:116-164,290-327 for the patterns on the
AnchorAttention path ("default", "flash", "anchor_attn"); the competitor patterns of the reference are not
part of this package and raise ``ValueError``.  In transformers 5 the attention product is selected by
name through ``AttentionInterface``, so patching is: register the plug once, point the model's config at it,
and copy the pattern's parameters onto the config (patch.py:106-109 does the same ``setattr`` loop).
"""
import copy

from my_utils import Logger

ATTENTION_CONFIG_EXAMPLE = {
    "default": {},
    "flash": {},
    "anchor_attn": {"block_size_M": 128, "theta": 12, "step": 16},
}

_SUPPORTED_MODELS = ("llama", "qwen2")


def get_config_example(pattern: str = None):
    if pattern is None:
        return copy.deepcopy(ATTENTION_CONFIG_EXAMPLE)
    return copy.deepcopy(ATTENTION_CONFIG_EXAMPLE[pattern])


def _register():
    from transformers import AttentionInterface, AttentionMaskInterface
    from transformers.masking_utils import sdpa_mask

    from anchor_attn.src.modules.llama.anchor_attention import ATTN_NAME, anchor_attention_forward
    if ATTN_NAME not in AttentionInterface().valid_keys():
        AttentionInterface.register(ATTN_NAME, anchor_attention_forward)
        # same mask convention as SDPA: None when the mask is purely causal, a boolean mask otherwise
        AttentionMaskInterface.register(ATTN_NAME, sdpa_mask)
    return ATTN_NAME


def patch_model(model, pattern: str, config: dict = None):
    """Patch ``model`` (a transformers ``PreTrainedModel`` of the Llama or Qwen2 family) in place.

    pattern: "default" (leave as is), "flash" (library dense attention) or "anchor_attn".
    config : for "anchor_attn" ``{"block_size_M": 128, "theta": 12, "step": 16}`` (the defaults).
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
    cfg.update(config or {})
    if pattern == "flash":
        model.set_attn_implementation("sdpa")
    else:
        if cfg["step"] not in (16, 32) or cfg["block_size_M"] != 128:
            raise ValueError("anchor_attn supports block_size_M = 128 and step in (16, 32)")
        model.set_attn_implementation(_register())
        for k, v in cfg.items():
            setattr(model.config, k, v)
    Logger.log(f"replace attention with {pattern}: {cfg}")
    return model

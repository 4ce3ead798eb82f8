"""Qwen2 uses the same attention plug as Llama in transformers 5 (the reference keeps a separate copy of the
forward, modules/qwen2/anchor_attention.py:126-157, whose only functional difference - the ``q_len >= 2048``
guard - is part of the shared implementation here)."""
from anchor_attn.src.modules.llama.anchor_attention import ATTN_NAME, anchor_attention_forward  # noqa: F401

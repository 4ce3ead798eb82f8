"""The Hugging Face attention hook that runs prefill through the AnchorAttention operator.

Counterpart of ``llama_flash_attn2_forward_anchorattn`` (reference
anchor_attn/src/modules/llama/anchor_attention.py:17-118).  The reference replaces the whole
``forward`` of ``LlamaFlashAttention2``; that class no longer exists in transformers 5, where the
projections, RoPE and the KV cache stay in ``LlamaAttention.forward`` and only the attention product is
pluggable (``AttentionInterface``).  This function is that plug: it receives ``query [B,Hq,N,D]`` and
un-repeated ``key``/``value [B,Hkv,Nkv,D]`` and returns ``[B,N,Hq,D]``.

What it keeps from the reference: prefill rows ``[0, N - pad)`` with ``pad = N % (block_size_M*step)``
go through ``anchor_attn``; the ``pad`` tail rows and single-token decode steps use dense attention.
What it changes: K/V are passed with their native KV heads (no ``repeat_kv`` copies), q/k/v/out are
consumed in the layout transformers hands over (no ``clone().contiguous()``), and ``pad == 0`` works (the
reference's ``[:-0]`` slices are empty there).  Sequences shorter than one big block are dense, which is
what the Qwen2 variant of the reference guards for (modules/qwen2/anchor_attention.py:147).
"""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from anchor_attn.src.ops.anchor_attn_v4 import LOG2E, _anchor_attn, anchor_attn, dense_causal_attention

ATTN_NAME = "anchor_attn"
DENSE_ATTN_NAME = "anchor_attn_dense"

# Measurement scripts set ``record_ratio``; the plug then also asks the operator for the per-big-block counts and
# leaves the sparsity ratio of the most recent prefill call in ``last_ratio`` as a 0-dim DEVICE tensor (nothing is
# copied to the host and nothing is logged, so the model stays free of host synchronisation either way).  By default
# the operator is called with ``return_computational_ratio=False`` as the reference's caller does
# (modules/llama/anchor_attention.py:92-100).
record_ratio: bool = False
last_ratio: Optional[torch.Tensor] = None


def _dense(query, key, value, attention_mask, scaling, causal_offset: Optional[int]):
    """Dense attention for the parts the sparse operator does not cover (tail rows, decode, padded batches).
    ``causal_offset``: query row i may see keys ``<= causal_offset + i`` (None: use ``attention_mask`` as is)."""
    groups = query.shape[1] // key.shape[1]
    mask = attention_mask
    if causal_offset is not None and mask is None and query.shape[2] > 1:
        rows = torch.arange(query.shape[2], device=query.device)[:, None] + causal_offset
        mask = torch.arange(key.shape[2], device=query.device)[None, :] <= rows
    return F.scaled_dot_product_attention(query, key, value, attn_mask=mask, scale=scaling, enable_gqa=groups > 1)


def anchor_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                             attention_mask: Optional[torch.Tensor], dropout: float = 0.0,
                             scaling: Optional[float] = None, **kwargs) -> Tuple[torch.Tensor, None]:
    global last_ratio
    cfg = module.config
    block_size, step, theta = int(cfg.block_size_M), int(cfg.step), float(cfg.theta)
    big = block_size * step
    B, Hq, N, D = query.shape
    n_kv = key.shape[2]
    out = torch.empty(B, N, Hq, D, dtype=query.dtype, device=query.device)  # the layout the caller reshapes
    out_bhnd = out.transpose(1, 2)
    # Prefill of a fresh sequence without padding is the case the operator is defined for.
    sparse_ok = N > 1 and n_kv == N and attention_mask is None and N >= big and query.dtype in (torch.bfloat16, torch.float16)
    if not sparse_ok:
        out_bhnd.copy_(_dense(query, key, value, attention_mask, scaling, n_kv - N if attention_mask is None else None))
        return out, None
    pad = N % big
    main = N - pad
    if record_ratio:
        sm_scale = scaling if scaling else 1.0 / (D ** 0.5)
        _, last_ratio = _anchor_attn(query[:, :, :main], key[:, :, :main], value[:, :, :main], sm_scale, block_size, step,
                                     theta * LOG2E, True, out=out_bhnd[:, :, :main])
    else:
        anchor_attn(query[:, :, :main], key[:, :, :main], value[:, :, :main], sm_scale=scaling,
                    block_size=block_size, step=step, difference=theta,
                    return_computational_ratio=False, out=out_bhnd[:, :, :main])
    if pad:
        out_bhnd[:, :, main:].copy_(_dense(query[:, :, main:], key, value, None, scaling, main))
    return out, None


def dense_attention_forward(module, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor,
                            attention_mask: Optional[torch.Tensor], dropout: float = 0.0,
                            scaling: Optional[float] = None, **kwargs) -> Tuple[torch.Tensor, None]:
    """Plain causal attention on the library's own MFMA core (``aa_dense_causal_fwd``): the dense baseline "built on
    the same kernels" that the sparse operator is compared with.  Counterpart of the reference's ``"flash"`` pattern
    (modules/patch.py:128-130 -> modules/llama/flash_attention.py, ops/flash_attn_triton.py:641-657), with the same
    division of labour as the sparse plug: a fresh unpadded bf16/fp16 prefill goes through the kernel in multiples of
    128 rows, the remaining tail rows, decode steps and padded batches through the framework's dense attention."""
    B, Hq, N, D = query.shape
    n_kv = key.shape[2]
    out = torch.empty(B, N, Hq, D, dtype=query.dtype, device=query.device)
    out_bhnd = out.transpose(1, 2)
    kernel_ok = N >= 128 and n_kv == N and attention_mask is None and query.dtype in (torch.bfloat16, torch.float16) and query.is_cuda
    if not kernel_ok:
        out_bhnd.copy_(_dense(query, key, value, attention_mask, scaling, n_kv - N if attention_mask is None else None))
        return out, None
    main = N - N % 128
    dense_causal_attention(query[:, :, :main], key[:, :, :main], value[:, :, :main], sm_scale=scaling, out=out_bhnd[:, :, :main])
    if main < N:
        out_bhnd[:, :, main:].copy_(_dense(query[:, :, main:], key, value, None, scaling, main))
    return out, None

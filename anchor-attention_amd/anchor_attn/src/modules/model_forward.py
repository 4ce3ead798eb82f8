"""The two model-level patches that the reference applies next to the attention forward, for every pattern but
"default" (anchor_attn/src/modules/patch.py:146-157): logits for the last position only, and the MLP evaluated in
chunks of the sequence.  Both exist to keep a 128k-token prefill small in memory - full logits are
131072 x 128256 values (33 GB in bf16 before the float32 copy), the MLP's intermediate 131072 x 14336 x 3.

The reference replaces ``LlamaForCausalLM.forward`` and ``LlamaMLP.forward`` wholesale with edited copies of the
transformers 4.45 sources (modules/llama/causal_model_forward.py:100-126, modules/llama/llama_mlp_forward.py:46-58).
Here both are thin wrappers around whatever forward the installed transformers has, so nothing is tied to one
release: the causal-LM wrapper asks the model's own ``logits_to_keep`` mechanism for one position, the MLP wrapper
calls the module's own forward on slices.
"""
import functools

import torch

MLP_CHUNK_TOKENS = 32768  # the reference's chunk (llama_mlp_forward.py:52)


def keep_last_token_logits(model) -> None:
    """After this, ``model(input_ids)`` returns float32 logits of the last position only, ``[B, 1, vocab]`` - what the
    reference's patched forward returns (causal_model_forward.py:124-125: ``lm_head(hidden_states[:, -1:, :])``, then
    ``.float()``).  A caller that passes ``logits_to_keep`` itself, or ``labels`` (a loss needs every position), gets
    what it asked for."""
    inner = model.forward
    if getattr(inner, "_keeps_last_token_logits", False):
        return

    @functools.wraps(inner)
    def forward(*args, **kwargs):
        if "logits_to_keep" not in kwargs and kwargs.get("labels") is None:
            kwargs["logits_to_keep"] = 1
        out = inner(*args, **kwargs)
        logits = out.get("logits") if isinstance(out, dict) else None
        if logits is not None and logits.dtype != torch.float32:
            out["logits"] = logits.float()
        return out

    forward._keeps_last_token_logits = True
    model.forward = forward


def chunk_mlp_over_tokens(model, chunk_tokens: int = MLP_CHUNK_TOKENS) -> int:
    """Every MLP of the model (a module named ``mlp`` with gate/up/down projections) is evaluated ``chunk_tokens``
    positions at a time per batch element, into a preallocated output, as llama_mlp_forward.py:46-58 does.  Rows of
    a linear layer do not interact, so the result is that of the unchunked forward.  Returns how many modules were
    wrapped; calling it again only updates the chunk size."""
    n = 0
    for _, m in model.named_modules():
        if not all(hasattr(m, a) for a in ("gate_proj", "up_proj", "down_proj")):
            continue
        n += 1
        m._mlp_chunk_tokens = int(chunk_tokens)
        if getattr(m.forward, "_chunks_tokens", False):
            continue
        inner = m.forward

        def forward(x, _inner=inner, _m=m):
            chunk = _m._mlp_chunk_tokens
            if chunk <= 0 or x.dim() != 3 or x.shape[1] <= chunk:
                return _inner(x)
            out = torch.empty_like(x)
            for b in range(x.shape[0]):
                for i in range(0, x.shape[1], chunk):
                    out[b:b + 1, i:i + chunk] = _inner(x[b:b + 1, i:i + chunk])
            return out

        forward._chunks_tokens = True
        m.forward = forward
    return n

"""Token-level ideal of difference-aware sparse attention, in plain torch (an analysis tool, not a kernel).

Counterpart of ``sparse_attn_with_torch`` (reference anchor_attn/src/ops/sparse_attn_with_pytorch.py:175-241):
every query row keeps exactly the causal keys whose score is within ``diff_anchor`` of the row's own maximum,
``score + diff_anchor >= max``; the returned ratio is kept / causal.  It is the accuracy ceiling that the
block-pooled stage 2 of the operator approximates.  Runs on whatever device the inputs live on, in query
chunks so that the score matrix never exceeds ``chunk x n_keys``.  K/V may have fewer (KV) heads than Q.
"""
import math

import torch


def sparse_attn_with_torch(q, k, v, softmax_scale=None, diff_anchor=12, fullkv: bool = False,
                           return_computational_ratio: bool = False, chunk_size: int = 256):
    B, H, Nq, D = q.shape
    Nk = k.shape[2]
    group = H // k.shape[1]
    scale = softmax_scale if softmax_scale is not None else 1.0 / math.sqrt(D)
    kt = k.float().repeat_interleave(group, 1).transpose(-1, -2) if group > 1 else k.float().transpose(-1, -2)
    vf = v.float().repeat_interleave(group, 1) if group > 1 else v.float()
    out = torch.empty(B, H, Nq, D, dtype=q.dtype, device=q.device)
    cols = torch.arange(Nk, device=q.device)[None, :]
    kept = torch.zeros((), dtype=torch.float64, device=q.device)
    causal = torch.zeros((), dtype=torch.float64, device=q.device)
    for r0 in range(0, Nq, chunk_size):
        r1 = min(r0 + chunk_size, Nq)
        s = torch.matmul(q[:, :, r0:r1].float(), kt) * scale
        visible = cols <= (torch.arange(r0, r1, device=q.device)[:, None] + (Nk - Nq))
        s = s.masked_fill(~visible, float("-inf"))
        if not fullkv:
            keep = (s + diff_anchor) >= s.amax(dim=-1, keepdim=True)
            kept += keep.sum()
            causal += visible.sum() * (B * H)
            s = s.masked_fill(~keep, float("-inf"))
        out[:, :, r0:r1] = torch.matmul(torch.softmax(s, dim=-1), vf).to(q.dtype)
    if return_computational_ratio:
        return out, (float(kept / causal) if float(causal) > 0 else 1.0)
    return out

"""``get_q_mask`` with the reference's signature and return layout (``anchor_attn/src/ops/get_mask_test.py:127-159``),
backed by the gfx950 stage-2 kernels, and ``get_mask_block``, the framework-tensor restatement of the same stage that
the reference keeps next to it (``:162-232``)."""
from __future__ import annotations

from .anchor_step_1_2_v2 import expand_coords, select_stripes_packed


def get_q_mask(Q, K, anchors, block_size, step, diff, B, H, seq, h_dim, qk_scale):
    assert Q.is_contiguous(), "Q should be contiguous"
    assert K.is_contiguous(), "K should be contiguous"
    assert block_size in [16, 32, 64, 128, 256], "BLOCK_SIZE must be a power of 2 and ≥16"
    assert step in [16, 32], "step must be ≥16"
    assert seq % (block_size * step) == 0
    coords, counts = select_stripes_packed(Q, K, anchors.reshape(B, H, seq), block_size, step, diff, B, H, seq, h_dim, qk_scale)
    return expand_coords(coords, counts, seq, block_size, step), counts


def get_mask_block(Q, K, anchors, block_size_N, block_size_M, step, diff, B, H, seq, h_dim, sm_scale, device,
                   return_sparsity_ratio: bool = False):
    """Stage 2 restated with framework tensor operations, the counterpart of the reference's ``get_mask_block``
    (get_mask_test.py:162-232): an analysis helper, not part of the operator.  Everything is evaluated in the tensors'
    own precision without the kernels' rounding points: queries and anchors are mean-pooled over ``block_size_N`` rows,
    key ``j`` is kept for big block ``i`` iff ``mean_q . k_j * sm_scale + diff >= mean_anchor`` for one of the block's
    ``step`` pooled rows, and the kept keys of ``[block_size_N, i*block_size_N*step - block_size_N)`` become an
    ascending list.  ``anchors`` is ``[B,H,seq]``; ``sm_scale`` and ``diff`` must be in the anchors' domain (the
    operator's anchors are base-2 logarithms of scores scaled by ``sm_scale * 1.44269504``).  ``K`` must carry ``H``
    heads.  Returns ``(true_coords [B,H,c_n,seq] int32, true_counts [B,H,c_n,1] int32[, selected / candidates])`` in
    the layout of :func:`get_q_mask`.  ``block_size_M`` is accepted for the reference's signature and not used, as there.
    """
    import torch
    c_n = (seq // block_size_N + step - 1) // step
    pad_rows = (step - (seq // block_size_N) % step) % step
    mean_q = Q.to(device).reshape(B, H, -1, block_size_N, h_dim).mean(dim=-2)
    mean_a = anchors.to(device).reshape(B, H, -1, block_size_N, 1).mean(dim=-2)
    keep = (torch.matmul(mean_q, K.to(device).transpose(-1, -2) * sm_scale) + diff) >= mean_a  # [B,H,seq/bs,seq]
    if pad_rows:
        keep = torch.nn.functional.pad(keep, (0, 0, 0, pad_rows))
    keep = keep.reshape(B, H, c_n, step, seq).any(dim=-2)
    # candidate range of big block i: [block_size_N, i*S - block_size_N)
    key = torch.arange(seq, device=keep.device)
    hi = torch.arange(c_n, device=keep.device) * (block_size_N * step) - block_size_N
    keep &= (key[None, :] >= block_size_N) & (key[None, :] < hi[:, None])
    counts = keep.sum(dim=-1, dtype=torch.int32)
    # ascending indices first (stable sort of "not kept"), zeros past the count as in the reference's buffer
    order = torch.sort((~keep).to(torch.uint8), dim=-1, stable=True).indices.to(torch.int32)
    coords = torch.where(key[None, None, None, :] < counts[..., None], order, torch.zeros_like(order))
    true_counts = counts.reshape(B, H, c_n, 1)
    if return_sparsity_ratio:
        candidates = int(hi.clamp(min=block_size_N).sub(block_size_N).sum()) * B * H
        return coords, true_counts, (float(counts.sum()) / candidates if candidates else 0.0)
    return coords, true_counts

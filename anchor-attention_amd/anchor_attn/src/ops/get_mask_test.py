"""``get_q_mask`` with the reference's signature and return layout
(``anchor_attn/src/ops/get_mask_test.py:127-159``), backed by the gfx950 stage-2 kernels."""
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

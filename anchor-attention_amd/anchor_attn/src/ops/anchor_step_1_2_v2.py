"""Stage 1 (anchor computation) and stage 2 (stripe identification) entry points, named after the
reference's ``anchor_attn/src/ops/anchor_step_1_2_v2.py`` (``anchor_attn_step_1`` :164-196,
``anchor_attn_step_2`` :199-210) and backed by the gfx950 kernels.

Differences a caller can see:

* K/V may carry fewer heads than Q (native GQA); pre-repeated K/V works too.
* ``Acc_buffer`` is returned in the kernels' MFMA fragment order (it is scratch between stage 1
  and stage 3); :func:`acc_rows` gives the ``[B,H,N,D]`` view the reference stores.
* index lists are packed (no ``[B,H,N/S,N]`` buffer); :func:`expand_coords` rebuilds the
  reference layout when it is wanted.
"""
from __future__ import annotations

import torch

from . import _hip


def _row_major(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _check_inputs(Q, K, V=None):
    assert Q.is_cuda and K.is_cuda, "anchor_attn runs on the GPU only (there is no CPU path)"
    assert Q.dtype in (torch.bfloat16, torch.float16) and K.dtype == Q.dtype, "anchor_attn kernels take bf16 or fp16 inputs (one type per call)"
    assert Q.shape[1] % K.shape[1] == 0, "number of KV heads must divide the number of query heads"
    if V is not None:
        assert V.dtype == Q.dtype and V.shape == K.shape


def anchor_attn_step_1(Q, K, V, init_cnt, local_cnt, block_size, step, B, H, N, D, sm_scale,
                       BLOCK_SZ_M=128, BLOCK_SZ_N=128, scale_mode=_hip.AA_SCALE_BF16_CHAIN):
    """Windowed flash attention over ``[0,S) U [bb*S, r]``; returns ``(L_buffer, M_buffer,
    Acc_buffer)`` float32.  ``init_cnt`` and ``local_cnt`` must be 1, the only values the
    operator uses (anchor_attn_v4.py:237-241)."""
    assert init_cnt == 1 and local_cnt == 1, "only init_cnt = local_cnt = 1 is implemented"
    _check_inputs(Q, K, V)
    Q, K, V = _row_major(Q), _row_major(K), _row_major(V)
    L = torch.empty((B, H, N), dtype=torch.float32, device=Q.device)
    M = torch.empty((B, H, N), dtype=torch.float32, device=Q.device)
    Acc = torch.empty((B, H, N, D), dtype=torch.float32, device=Q.device)
    _hip.check(_hip.lib().aa_stage1_anchor_fwd(
        *_hip.t3(Q), *_hip.t3(K), *_hip.t3(V), M.data_ptr(), L.data_ptr(), Acc.data_ptr(),
        B, H, K.shape[1], N, D, block_size, step, float(sm_scale), scale_mode, _hip.dtype_code(Q), _stream()))
    return L, M, Acc


def acc_rows(Acc_frag: torch.Tensor) -> torch.Tensor:
    """Fragment-ordered accumulator -> ``[B,H,N,D]`` rows.  Element (row, d) of a head sits at
    32-row block ``row//32``, d-block ``d//32``, register group ``(d%32)//8``, wave half
    ``(d%8)//4``, lane column ``row%32``, component ``d%4``."""
    B, H, N, D = Acc_frag.shape
    v = Acc_frag.view(B, H, N // 32, D // 32, 4, 2, 32, 4)  # rb, db, rg, half, q, c
    return v.permute(0, 1, 2, 6, 3, 4, 5, 7).reshape(B, H, N, D)


def pool_q_anchor(Q, M_buffer, block_size):
    """Mean-pooled queries ``[B,H,N/bs,D]`` and anchors ``[B,H,N/bs]`` in the queries' 16-bit type (get_mask_test.py:75-84)."""
    Q = _row_major(Q)
    B, H, N, D = Q.shape
    qbar = torch.empty((B, H, N // block_size, D), dtype=Q.dtype, device=Q.device)
    abar = torch.empty((B, H, N // block_size), dtype=Q.dtype, device=Q.device)
    M_buffer = M_buffer.reshape(B, H, N).contiguous()
    _hip.check(_hip.lib().aa_pool_q_anchor(*_hip.t3(Q), M_buffer.data_ptr(), qbar.data_ptr(), abar.data_ptr(),
                                           B, H, N, D, block_size, _hip.dtype_code(Q), _stream()))
    return qbar, abar


def select_stripes_packed(Q, K, M_buffer, block_size, step, theta, B, H, N, D, sm_scale, geometry=_hip.AA_GEOMETRY_AS_RUN):
    """Stage 2 with packed outputs: ``(coords int32 [B,H,entries_per_head], counts int32
    [B,H,N/S,1])``; ``theta`` is already in the log2 domain, as the reference passes it."""
    _check_inputs(Q, K)
    K = _row_major(K)
    lib = _hip.lib()
    qbar, abar = pool_q_anchor(Q, M_buffer, block_size)
    n_bb = N // (block_size * step)
    per_head = lib.aa_coords_entries_per_head(N, block_size, step)
    mask = torch.empty((lib.aa_mask_words(B, H, N, block_size, step),), dtype=torch.int32, device=Q.device)
    coords = torch.empty((B, H, max(per_head, 1)), dtype=torch.int32, device=Q.device)
    counts = torch.empty((B, H, n_bb, 1), dtype=torch.int32, device=Q.device)
    _hip.check(lib.aa_stage2_select(qbar.data_ptr(), abar.data_ptr(), *_hip.t3(K), mask.data_ptr(), coords.data_ptr(),
                                    counts.data_ptr(), B, H, K.shape[1], N, D, block_size, step,
                                    float(sm_scale), float(theta), int(geometry), _hip.dtype_code(Q), _stream()))
    return coords, counts


def expand_coords(coords, counts, N, block_size, step):
    """Packed index lists -> the reference's ``true_coords [B,H,N/S,N]`` (zeros past the count)."""
    B, H = coords.shape[:2]
    n_bb = N // (block_size * step)
    lib = _hip.lib()
    out = torch.zeros((B, H, n_bb, N), dtype=torch.int32, device=coords.device)
    cnt = counts.reshape(B, H, n_bb)
    for bb in range(1, n_bb):
        cap = bb * block_size * step - 2 * block_size
        off = lib.aa_coords_offset(bb, block_size, step)
        seg = coords[:, :, off:off + cap]
        keep = torch.arange(cap, device=coords.device)[None, None, :] < cnt[:, :, bb, None]
        out[:, :, bb, :cap] = torch.where(keep, seg, torch.zeros_like(seg))
    return out


def anchor_attn_step_2(Q, K, M_buffer, block_size, step, theta, B, H, N, D, sm_scale):
    """Reference-shaped stage 2: ``(true_coords [B,H,N/S,N], true_counts [B,H,N/S,1])``.  The
    operator itself uses :func:`select_stripes_packed`; this wrapper exists for callers that
    want the reference's buffers."""
    from .get_mask_test import get_q_mask
    return get_q_mask(Q, K, M_buffer.unsqueeze(-1), block_size, step, theta, B, H, N, D, sm_scale)

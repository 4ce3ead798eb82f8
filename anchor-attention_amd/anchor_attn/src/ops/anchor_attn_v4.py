"""The AnchorAttention prefill operator on MI355X.

Same entry points, argument meaning, assertions and return arity as the reference's
``anchor_attn/src/ops/anchor_attn_v4.py`` (``anchor_attn`` :291-324, ``anchor_attn_test_time``
:328-354, ``anchor_attn_without_anchor`` :275-289); the three stages underneath are hand-written
gfx950 kernels reached through the C ABI in ``include/anchor_attn_hip.h``.

Beyond the reference: K and V may be passed with their native (un-repeated) KV heads, any
``[B,H,N,D]`` view with unit last stride is taken without a copy, and ``out`` may be supplied.
There is no CPU or eager fallback - tensors must be bf16 (or fp16, which the reference's kernels also take) on the GPU.
"""
from __future__ import annotations

import time

import torch

from . import _hip
from .anchor_step_1_2_v2 import (_check_inputs, _row_major, _stream, anchor_attn_step_1,
                                 select_stripes_packed)

LOG2E = 1.44269504


def _ratio(true_counts, B, H, N, block_size, step):
    # same expression as the reference (anchor_attn_v4.py:271); stays a 0-dim device tensor
    return true_counts.sum() / (B * H * N * N / (block_size * step) // 2)


def _log_ratio(sparse_ratio):
    """The reference logs the ratio on every call (anchor_attn_v4.py:321-323).  Formatting the 0-dim device tensor
    copies it to the host, i.e. waits for the whole operator; that is only paid when the logger is switched on."""
    from my_utils import Logger
    if Logger.enabled:
        Logger.log(f"anchor sparse_ratio:{sparse_ratio}")


def _workspace(B, H, N, D, block_size, step, device):
    nbytes = _hip.lib().aa_workspace_bytes(B, H, N, D, block_size, step)
    if nbytes == 0:
        raise _hip.AnchorAttnHipError(f"unsupported problem shape B={B} H={H} N={N} D={D} block_size={block_size} step={step}")
    return torch.empty((nbytes,), dtype=torch.uint8, device=device)


def _anchor_attn(Q, K, V, sm_scale=None, block_size=64, step=16, difference=100, return_sparsity_ratio=False,
                 BLOCK_SIZE_M=128, BLOCK_SIZE_N=128, out=None, scale_mode=_hip.AA_SCALE_BF16_CHAIN,
                 geometry=_hip.AA_GEOMETRY_AS_RUN):
    """All three stages on the current stream, one C call (``difference`` is in the log2 domain
    here, as in the reference's private function, anchor_attn_v4.py:226-273)."""
    B, H, N, D = Q.shape
    assert N % block_size == 0
    assert block_size in [16, 32, 64, 128, 256], "BLOCK_SIZE must be a power of 2 and ≥16"  # get_mask_test.py:133
    _check_inputs(Q, K, V)
    output = torch.empty_like(Q) if out is None else out
    assert output.shape == Q.shape and output.dtype == Q.dtype and output.stride(-1) == 1
    ws = _workspace(B, H, N, D, block_size, step, Q.device)
    n_bb = N // (block_size * step)
    counts = torch.empty((B, H, n_bb, 1), dtype=torch.int32, device=Q.device) if return_sparsity_ratio else None
    _hip.check(_hip.lib().aa_anchor_attn_fwd(
        *_hip.t3(Q), *_hip.t3(K), *_hip.t3(V), *_hip.t3(output),
        ws.data_ptr(), ws.numel(), counts.data_ptr() if counts is not None else None,
        B, H, K.shape[1], N, D, block_size, step, float(sm_scale), float(difference), scale_mode, int(geometry),
        _hip.dtype_code(Q), _stream()))
    if return_sparsity_ratio:
        return output, _ratio(counts, B, H, N, block_size, step)
    return output, 1.0


def _stage3(Q, K, V, coords, counts, L, M, Acc, sm_scale, block_size, step, out=None):
    B, H, N, D = Q.shape
    output = torch.empty_like(Q) if out is None else out
    _hip.check(_hip.lib().aa_stage3_sparse_fwd(
        *_hip.t3(Q), *_hip.t3(K), *_hip.t3(V), coords.data_ptr(), counts.data_ptr(),
        M.data_ptr(), L.data_ptr(), Acc.data_ptr(), *_hip.t3(output),
        B, H, K.shape[1], N, D, block_size, step, float(sm_scale), _hip.dtype_code(Q), _stream()))
    return output


def _anchor_attn_staged(Q, K, V, sm_scale, block_size, step, difference, timed):
    B, H, N, D = Q.shape
    assert N % block_size == 0
    _check_inputs(Q, K, V)
    if timed:
        torch.cuda.synchronize()
        t0 = time.time()
    L, M, Acc = anchor_attn_step_1(Q, K, V, 1, 1, block_size, step, B, H, N, D, sm_scale)
    coords, counts = select_stripes_packed(Q, K, M, block_size, step, difference, B, H, N, D, sm_scale)
    if timed:
        torch.cuda.synchronize()
        t1 = time.time()
    output = _stage3(Q, K, V, coords, counts, L, M, Acc, sm_scale, block_size, step)
    if timed:
        torch.cuda.synchronize()
        t2 = time.time()
        return output, counts, (t1 - t0) * 1000, (t2 - t1) * 1000
    return output, counts, None, None


def _prepare(Q, K, V):
    return _row_major(Q), _row_major(K), _row_major(V)


def anchor_attn_without_anchor(Q, K, V, sm_scale: float = None, block_size: int = 128, step: int = 16,
                               difference: float = 12):
    difference *= LOG2E
    Q, K, V = _prepare(Q, K, V)
    assert Q.size(-2) % block_size == 0
    B, H, N, D = Q.shape
    sm_scale = sm_scale if sm_scale else 1.0 / (D ** 0.5)
    output, counts, _, _ = _anchor_attn_staged(Q, K, V, sm_scale, block_size, step, difference, timed=False)
    return output, _ratio(counts, B, H, N, block_size, step)


def anchor_attn(Q, K, V, sm_scale: float = None, block_size: int = 128, step: int = 16, difference: float = 12,
                return_computational_ratio: bool = True, out: torch.Tensor = None, strict_reference: bool = True):
    """Sparse prefill attention.  ``Q`` ``[B,H,N,D]`` bf16 or fp16; ``K``/``V`` ``[B,H or H_kv,N,D]`` of the same type;
    returns ``out`` or ``(out, ratio)`` exactly like the reference.

    ``strict_reference=False`` (analysis only, never the default) lets stage 2 choose from ``[S, bb*S)``
    - the range of the reference's fused variant, anchor_fuse_step_1_2_v2.py:152 - instead of the as-run
    ``[block_size, bb*S - block_size)``: no key is attended twice and none is left out."""
    difference *= LOG2E
    Q, K, V = _prepare(Q, K, V)
    assert Q.stride(-1) == 1 and K.stride(-1) == 1 and V.stride(-1) == 1, \
        "Q, K, V must be contiguous. Please call .contiguous() before passing."

    assert step in [16, 32], \
        f"Invalid step size: {step}. Only step sizes 16 or 32 are supported."

    assert Q.size(-2) % (block_size * step) == 0, \
        f"Sequence length {Q.size(-2)} must be divisible by (block_size * step = {block_size * step})."

    B, H, N, D = Q.shape
    sm_scale = sm_scale if sm_scale else 1.0 / (D ** 0.5)
    sparse_output, sparse_ratio = _anchor_attn(Q, K, V, sm_scale, block_size, step, difference,
                                               return_computational_ratio, out=out,
                                               geometry=_hip.AA_GEOMETRY_AS_RUN if strict_reference else _hip.AA_GEOMETRY_INTENDED)
    if return_computational_ratio:
        _log_ratio(sparse_ratio)
        return sparse_output, sparse_ratio
    return sparse_output


def anchor_attn_test_time(Q, K, V, sm_scale: float = None, block_size: int = 128, step: int = 16,
                          difference: float = 12, return_computational_ratio: bool = True):
    """Same result as :func:`anchor_attn` plus the wall-clock of (stage 1 + stage 2) and of stage 3
    in milliseconds, each bracketed by device synchronisation (anchor_attn_v4.py:107-169)."""
    difference *= LOG2E
    Q, K, V = _prepare(Q, K, V)
    assert Q.size(-2) % block_size == 0
    B, H, N, D = Q.shape
    sm_scale = sm_scale if sm_scale else 1.0 / (D ** 0.5)
    output, counts, search_time, compute_time = _anchor_attn_staged(Q, K, V, sm_scale, block_size, step, difference, timed=True)
    if return_computational_ratio:
        sparse_ratio = _ratio(counts, B, H, N, block_size, step)
        _log_ratio(sparse_ratio)
        return output, sparse_ratio, search_time, compute_time
    return output, search_time, compute_time


def dense_causal_attention(Q, K, V, sm_scale: float = None, out: torch.Tensor = None):
    """Plain causal attention on the same MFMA core (the dense baseline the sparse operator is
    compared with; GQA-aware like the reference's flash_attn_triton.py:129-132)."""
    Q, K, V = _prepare(Q, K, V)
    _check_inputs(Q, K, V)
    B, H, N, D = Q.shape
    sm_scale = sm_scale if sm_scale else 1.0 / (D ** 0.5)
    output = torch.empty_like(Q) if out is None else out
    _hip.check(_hip.lib().aa_dense_causal_fwd(*_hip.t3(Q), *_hip.t3(K), *_hip.t3(V), *_hip.t3(output),
                                              B, H, K.shape[1], N, D, float(sm_scale), _hip.dtype_code(Q), _stream()))
    return output

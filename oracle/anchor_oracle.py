"""CPU oracle for the AnchorAttention prefill operator (numpy, float32 + emulated bf16 rounding).

TEST INFRASTRUCTURE ONLY.  This module restates, on the CPU, the arithmetic that the
reference's three GPU kernels perform *as they run* (window geometry, candidate range,
rounding points, double-counted keys, the never-attended 128-key gap).  It exists so that
tests, the smoke check and the benchmark's CPU-baseline leg have something to compare the
HIP kernels with.  Nothing in the product path imports it, and it is never a fallback.

Reference files restated here (paths relative to the reference checkout):

* stage 1  ``anchor_attn/src/ops/anchor_step_1_2_v2.py:8-161``  (kernel ``get_mask_fused_anchor_triton``)
* stage 2  ``anchor_attn/src/ops/get_mask_test.py:7-124``        (kernel ``get_q_mask_triton``)
* stage 3  ``anchor_attn/src/ops/anchor_attn_v4.py:7-105``       (kernel ``_triton_stripe_sparse_attn_fwd_kernel_step3``)
* driver   ``anchor_attn/src/ops/anchor_attn_v4.py:226-273,291-324`` (``_anchor_attn`` / ``anchor_attn``)

Parity status: the reference ships no golden vectors for this path, so every function below
is pinned by mathematics instead (tests/test_oracle_*.py): float64 brute force over the
explicit key sets, library softmax attention where the key set is the full causal prefix,
closed forms for theta -> +/- infinity, an independent bf16 rounding (torch's cast) and the
multiplicity formula for double-counted keys.  The two query pre-scaling chains
(``q1_scale_chain``: bf16 products for stage 1, whose kernel takes ``sm_scale`` as a constexpr;
``q3_scale_chain``: float32 products for stage 3, whose kernel takes it at run time) are pinned
bit for bit against the Triton toolchain itself: tests/triton_promotion_probe.py compiles the two
forms of the reference's expression as micro-kernels of its own, and its outputs on an MI355X are
the fixture tests/golden/triton_scale_chain_probe.npz (made with Triton 3.6.0; the reference's
requirements.txt pins 3.2.0, which is not installed here).  ``stage1_scale_mode`` remains a switch.
Nothing here depends on the head dimension (the reference's kernels take ``D`` from the tensors); besides 128 the
pins run at 64 (tests/test_oracle_pins.py::test_head_dim_64_by_independent_closed_form).

Conventions: ``Q`` is ``[B, Hq, N, D]``, ``K``/``V`` are ``[B, Hkv, N, D]`` with ``Hkv | Hq``
(query head ``h`` reads KV head ``h // (Hq // Hkv)``, the order ``repeat_kv`` produces);
all arrays are float32 holding values representable in the tensors' 16-bit type: bf16, the type every caller of
the reference uses and the default of every function here, or fp16 (``dtype="fp16"``), which its kernels also take.  ``S = block_size * step`` is the
"big block"; ``LOG2E`` is the literal 1.44269504 the reference multiplies by.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Dict, List, Optional, Tuple

import numpy as np

LOG2E = 1.44269504  # literal used throughout the reference (anchor_attn_v4.py:66,298)
MASK_ADD = np.float32(-1.0e6)  # additive causal mask (anchor_step_1_2_v2.py:129,146)


# --------------------------------------------------------------------------------------
# bf16 rounding
# --------------------------------------------------------------------------------------
def rn16(x: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest bf16 (ties to even) and return it as float32.

    This is what a ``.to(tl.bfloat16)`` does on the reference's hardware path
    (e.g. get_mask_test.py:78,84,97).  NaN stays NaN, +/-inf stay as they are.
    """
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    lsb = (bits >> np.uint32(16)) & np.uint32(1)
    rounded = bits + np.uint32(0x7FFF) + lsb
    rounded &= np.uint32(0xFFFF0000)
    out = rounded.view(np.float32)
    nan = np.isnan(x)
    if nan.any():
        out = np.where(nan, x, out)
    return out


def f32(x) -> np.float32:
    return np.float32(x)


def rnd16(x: np.ndarray, dtype: str = "bf16") -> np.ndarray:
    """Round float32 to the tensors' 16-bit type and back: what a ``.to(dtype)`` of the reference's kernels does,
    where ``dtype`` is ``tl.bfloat16`` for bf16 inputs and ``tl.float16`` otherwise (anchor_step_1_2_v2.py:193,
    get_mask_test.py:157, anchor_attn_v4.py:265).  ``"fp16"``: IEEE half, ties to even, overflow to infinity."""
    if dtype == "bf16":
        return rn16(x)
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)
    raise ValueError(dtype)


# --------------------------------------------------------------------------------------
# query scaling chains
# --------------------------------------------------------------------------------------
def q1_scale_chain(q: np.ndarray, sm_scale: float, mode: str = "bf16_chain", dtype: str = "bf16") -> np.ndarray:
    """Stage-1 query pre-scaling (anchor_step_1_2_v2.py:115-116).

    ``sm_scale`` is a compile-time constant there, so ``q * sm_scale * 1.44269504`` is
    evaluated on a bf16 tensor with both constants materialised as bf16 and a bf16 rounding
    after each multiply (``mode="bf16_chain"``; with fp16 tensors the same chain runs in fp16).
    ``mode="fp32"`` is the alternative reading (float32 products, one rounding) kept as a switch.
    """
    q = np.asarray(q, dtype=np.float32)
    if mode == "bf16_chain":
        s = rnd16(np.array([sm_scale], dtype=np.float32), dtype)[0]
        c = rnd16(np.array([LOG2E], dtype=np.float32), dtype)[0]
        return rnd16(rnd16(q * s, dtype) * c, dtype)
    if mode == "fp32":
        return q3_scale_chain(q, sm_scale, dtype)
    raise ValueError(mode)


def q3_scale_chain(q: np.ndarray, sm_scale: float, dtype: str = "bf16") -> np.ndarray:
    """Stage-3 query pre-scaling (anchor_attn_v4.py:65-66): ``sm_scale`` is a run-time float32
    argument, so both multiplies are float32 and there is a single rounding to bf16."""
    q = np.asarray(q, dtype=np.float32)
    return rnd16((q * np.float32(sm_scale)) * np.float32(LOG2E), dtype)


# --------------------------------------------------------------------------------------
# stage 1: anchor / window flash attention
# --------------------------------------------------------------------------------------
def _online_tile(m, l, acc, s, v, dtype="bf16"):
    """One online-softmax tile update in the exp2 domain (anchor_step_1_2_v2.py:130-137 and
    anchor_attn_v4.py:91-101): float32 row sum of the unrounded ``p``, bf16 ``p`` into PV."""
    m_new = np.maximum(m, s.max(axis=1))
    p = np.exp2(s - m_new[:, None]).astype(np.float32)
    alpha = np.exp2(m - m_new).astype(np.float32)
    l = l * alpha + p.sum(axis=1, dtype=np.float32)
    acc = acc * alpha[:, None]
    acc = acc + rnd16(p, dtype) @ v
    return m_new, l, acc


def stage1_anchor(
    Q: np.ndarray,
    K: np.ndarray,
    V: np.ndarray,
    sm_scale: float,
    block_size: int = 128,
    step: int = 16,
    scale_mode: str = "bf16_chain",
    tile_n: int = 128,
    dtype: str = "bf16",
) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Windowed flash attention that yields the anchors.

    Restates ``get_mask_fused_anchor_triton`` as launched with ``init_cnt=1, local_cnt=1``
    (anchor_attn_v4.py:237-241).  For query row ``r`` in big block ``bb = r // S`` the key set
    is ``[0, min(S, (m+1)*128))`` followed by ``[max(bb*S, init_end), (bb+1)*S)``, both under
    the additive causal mask, i.e. effectively ``[0, S) U [bb*S, r]`` for ``bb >= 1`` and
    ``[0, r]`` for ``bb == 0``.  Tiles that lie wholly above the diagonal add exactly zero
    (``p`` underflows to 0, ``alpha`` is 1), so all rows of a big block can walk the same tile
    list.

    Returns ``(M, L, Acc)``: running max in the log2 / stage-1-scaled domain ``[B,Hq,N]``,
    row sums ``[B,Hq,N]`` and the unnormalised PV accumulator ``[B,Hq,N,D]``, all float32.
    """
    B, Hq, N, D = Q.shape
    Hkv = K.shape[1]
    group = Hq // Hkv
    S = block_size * step
    assert N % S == 0
    M = np.empty((B, Hq, N), np.float32)
    L = np.empty((B, Hq, N), np.float32)
    Acc = np.empty((B, Hq, N, D), np.float32)
    n_bb = N // S
    for b in range(B):
        for h in range(Hq):
            k = K[b, h // group]
            v = V[b, h // group]
            for bb in range(n_bb):
                r0 = bb * S
                rows = np.arange(r0, r0 + S)
                q1 = q1_scale_chain(Q[b, h, r0 : r0 + S], sm_scale, scale_mode, dtype)
                m = np.full(S, -np.inf, np.float32)
                l = np.zeros(S, np.float32)
                acc = np.zeros((S, D), np.float32)
                tiles = list(range(0, S, tile_n))
                if bb >= 1:
                    tiles += list(range(r0, r0 + S, tile_n))
                for j in tiles:
                    s = q1 @ k[j : j + tile_n].T
                    keys = np.arange(j, j + tile_n)
                    s = s + np.where(keys[None, :] <= rows[:, None], np.float32(0), MASK_ADD)
                    m, l, acc = _online_tile(m, l, acc, s.astype(np.float32), v[j : j + tile_n], dtype)
                M[b, h, r0 : r0 + S] = m
                L[b, h, r0 : r0 + S] = l
                Acc[b, h, r0 : r0 + S] = acc
    return M, L, Acc


# --------------------------------------------------------------------------------------
# stage 2: stripe identification
# --------------------------------------------------------------------------------------
def pool_rows_f32_sequential(x: np.ndarray, block: int) -> np.ndarray:
    """Sum groups of ``block`` consecutive rows in float32, strictly in ascending row order.

    The reference writes ``tl.sum(q, axis=1) / BLOCK_SZ`` on the loaded tile (get_mask_test.py:76-77,82-83)
    and fixes neither the order nor, for the bf16 query tile, the accumulator type: that is a property
    of the Triton release (releases up to 3.1 widened bf16 to float32 inside ``tl.sum``; 3.6.0 reduces
    the bf16 tile in bf16; the reference pins 3.2.0, which is not available to check).  The anchors are
    float32 and are summed in float32 by every release.  This oracle takes the float32 sum - the
    closer of the two readings to the exact mean - in a sequential order, so that a kernel can
    reproduce it bit for bit; what the other reading changes was measured (38 of 855 140 selected
    indices and at most one bf16 step in the output at 128k tokens, tests/test_gpu_parity.py)."""
    n, c = x.shape
    xr = x.reshape(n // block, block, c)
    acc = np.zeros((n // block, c), np.float32)
    for t in range(block):
        acc = acc + xr[:, t, :]
    return acc


def pooled_queries(Qh: np.ndarray, block_size: int, dtype: str = "bf16") -> np.ndarray:
    """``rn16(mean over each 128-row block)`` of the raw (unscaled) queries of one head
    (get_mask_test.py:75-78).  ``Qh`` is ``[N, D]``; returns ``[N/block, D]``."""
    s = pool_rows_f32_sequential(Qh.astype(np.float32), block_size)
    return rnd16(s / np.float32(block_size), dtype)


def pooled_anchors(Mh: np.ndarray, block_size: int, dtype: str = "bf16") -> Tuple[np.ndarray, np.ndarray]:
    """``rn16(mean over each 128-row block)`` of the anchors (get_mask_test.py:81-84).
    Returns ``(rounded, unrounded float32 mean)``; the second is only used to classify
    near-boundary disagreements in tests."""
    s = pool_rows_f32_sequential(Mh.astype(np.float32)[:, None], block_size)[:, 0]
    mean = (s / np.float32(block_size)).astype(np.float32)
    return rnd16(mean, dtype), mean


def stage2_scores(qbar: np.ndarray, k_rows: np.ndarray, sm_scale: float, dtype: str = "bf16") -> Tuple[np.ndarray, np.ndarray]:
    """Pooled-query x key scores of get_mask_test.py:86,96-97: float32 dot, multiplied by
    ``sm_scale * 1.44269504`` (a double-precision product turned into a float32 constant) and cast to the 16-bit
    type.  Returns ``(rounded, pre_rounding)`` as float32 ``[rows, keys]``.

    bf16: a float32 product, then the rounding (two roundings; pinned bit for bit by the Triton probe).
    fp16: the Triton tool chain compiles ``(dot * scale).to(tl.float16)`` into one mixed-precision instruction that
    rounds the exact product once (pinned bit for bit by the same probe, tests/golden/triton_scale_chain_probe_fp16.npz);
    that is what is restated here.  It differs from two roundings only where the float32 product is exactly half-way
    between two fp16 values."""
    scale2 = np.float32(sm_scale * LOG2E)
    dot = (qbar @ k_rows.T).astype(np.float32)
    raw = (dot * scale2).astype(np.float32)
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            once = (dot.astype(np.float64) * np.float64(scale2)).astype(np.float16).astype(np.float32)
        return once, raw
    return rnd16(raw, dtype), raw


def stage2_select(
    Q: np.ndarray,
    K: np.ndarray,
    M: np.ndarray,
    sm_scale: float,
    theta: float,
    block_size: int = 128,
    step: int = 16,
    strict_reference: bool = True,
    dtype: str = "bf16",
) -> Tuple[List[List[List[np.ndarray]]], np.ndarray]:
    """Difference-aware stripe identification (``get_q_mask_triton``).

    ``strict_reference=False`` replaces the as-run candidate range by ``[S, bb*S)``, the range the
    reference's fused variant walks (anchor_fuse_step_1_2_v2.py:152); everything else is unchanged.

    For big block ``bb`` the candidate keys are ``[block_size, bb*S - block_size)``
    (get_mask_test.py:93-94); key ``j`` is selected iff for some pooled row ``i`` of the big
    block ``float(rn16(score_ij)) + diff >= float(anchor_i)`` with ``diff = float32(theta *
    1.44269504)`` (anchor_attn_v4.py:298, get_mask_test.py:100-101).

    Returns ``(coords, counts)``: ``coords[b][h][bb]`` is the ascending int32 index array and
    ``counts`` is ``[B, Hq, nBB]`` int32.
    """
    B, Hq, N, D = Q.shape
    Hkv = K.shape[1]
    group = Hq // Hkv
    S = block_size * step
    n_bb = N // S
    diff = np.float32(theta * LOG2E)
    counts = np.zeros((B, Hq, n_bb), np.int32)
    coords: List[List[List[np.ndarray]]] = []
    for b in range(B):
        per_b = []
        for h in range(Hq):
            k = K[b, h // group]
            qbar = pooled_queries(Q[b, h], block_size, dtype)
            abar, _ = pooled_anchors(M[b, h], block_size, dtype)
            per_h = []
            for bb in range(n_bb):
                lo, hi = (block_size, bb * S - block_size) if strict_reference else (S, bb * S)
                if hi <= lo:
                    per_h.append(np.zeros(0, np.int32))
                    continue
                sc, _ = stage2_scores(qbar[bb * step : (bb + 1) * step], k[lo:hi], sm_scale, dtype)
                hit = (sc + diff) >= abar[bb * step : (bb + 1) * step, None]
                idx = (np.nonzero(hit.any(axis=0))[0] + lo).astype(np.int32)
                per_h.append(idx)
                counts[b, h, bb] = idx.size
            per_b.append(per_h)
        coords.append(per_b)
    return coords, counts


def coords_to_reference_layout(coords, counts, N: int) -> np.ndarray:
    """Pack index lists into the reference's ``true_coords [B,H,nBB,N]`` (zero beyond count)."""
    B, Hq, n_bb = counts.shape
    out = np.zeros((B, Hq, n_bb, N), np.int32)
    for b in range(B):
        for h in range(Hq):
            for bb in range(n_bb):
                c = coords[b][h][bb]
                out[b, h, bb, : c.size] = c
    return out


# --------------------------------------------------------------------------------------
# stage 3: gathered sparse flash attention
# --------------------------------------------------------------------------------------
def stage3_sparse(
    Q: np.ndarray,
    K: np.ndarray,
    V: np.ndarray,
    coords,
    counts: np.ndarray,
    M: np.ndarray,
    L: np.ndarray,
    Acc: np.ndarray,
    sm_scale: float,
    block_size: int = 128,
    step: int = 16,
    num_indices: int = 128,
    dtype: str = "bf16",
) -> np.ndarray:
    """Resume the online softmax of stage 1 over the selected keys of the row's big block
    (``_triton_stripe_sparse_attn_fwd_kernel_step3``): chunks of 128 indices, lanes beyond the
    count at ``-inf``, no causal mask, then ``out = rn16(acc / l)``.  A selected key that
    already lies in the stage-1 window is simply counted a second time, as in the reference."""
    B, Hq, N, D = Q.shape
    Hkv = K.shape[1]
    group = Hq // Hkv
    S = block_size * step
    n_bb = N // S
    out = np.empty((B, Hq, N, D), np.float32)
    for b in range(B):
        for h in range(Hq):
            k = K[b, h // group]
            v = V[b, h // group]
            for bb in range(n_bb):
                r0 = bb * S
                q3 = q3_scale_chain(Q[b, h, r0 : r0 + S], sm_scale, dtype)
                m = M[b, h, r0 : r0 + S].copy()
                l = L[b, h, r0 : r0 + S].copy()
                acc = Acc[b, h, r0 : r0 + S].copy()
                idx = coords[b][h][bb]
                cnt = int(counts[b, h, bb])
                for c0 in range(0, cnt, num_indices):
                    ids = idx[c0 : min(c0 + num_indices, cnt)]
                    pad = num_indices - ids.size
                    s = (q3 @ k[ids].T).astype(np.float32)
                    vv = v[ids]
                    if pad:
                        s = np.concatenate([s, np.full((S, pad), -np.inf, np.float32)], axis=1)
                        vv = np.concatenate([vv, np.zeros((pad, D), np.float32)], axis=0)
                    m, l, acc = _online_tile(m, l, acc, s, vv, dtype)
                out[b, h, r0 : r0 + S] = rnd16(acc / l[:, None], dtype)
    return out


# --------------------------------------------------------------------------------------
# whole operator
# --------------------------------------------------------------------------------------
@dataclasses.dataclass
class OracleResult:
    out: np.ndarray  # [B,Hq,N,D] float32 holding bf16 values
    M: np.ndarray
    L: np.ndarray
    Acc: np.ndarray
    coords: list
    counts: np.ndarray  # [B,Hq,nBB] int32
    ratio: float


def sparsity_ratio(counts: np.ndarray, B: int, H: int, N: int, block_size: int, step: int) -> float:
    """``true_counts.sum() / (B*H*N*N / (block_size*step) // 2)`` (anchor_attn_v4.py:270-272);
    the ``//`` applies to the already divided float."""
    return float(counts.sum()) / ((B * H * N * N / (block_size * step)) // 2)


def anchor_attn_reference(
    Q: np.ndarray,
    K: np.ndarray,
    V: np.ndarray,
    sm_scale: Optional[float] = None,
    block_size: int = 128,
    step: int = 16,
    difference: float = 12.0,
    stage1_scale_mode: str = "bf16_chain",
    strict_reference: bool = True,
    dtype: str = "bf16",
) -> OracleResult:
    """The operator end to end, as ``anchor_attn`` runs it (anchor_attn_v4.py:291-324)."""
    B, Hq, N, D = Q.shape
    assert step in (16, 32)
    assert N % (block_size * step) == 0
    if not sm_scale:
        sm_scale = 1.0 / math.sqrt(D)
    M, L, Acc = stage1_anchor(Q, K, V, sm_scale, block_size, step, stage1_scale_mode, dtype=dtype)
    coords, counts = stage2_select(Q, K, M, sm_scale, difference, block_size, step, strict_reference, dtype=dtype)
    out = stage3_sparse(Q, K, V, coords, counts, M, L, Acc, sm_scale, block_size, step, dtype=dtype)
    ratio = sparsity_ratio(counts, B, Hq, N, block_size, step)
    return OracleResult(out, M, L, Acc, coords, counts, ratio)


# --------------------------------------------------------------------------------------
# helpers for the index-parity rule
# --------------------------------------------------------------------------------------
def _bf16_step(b: float, up: bool, dtype: str = "bf16") -> float:
    """Next value of the 16-bit type above (``up``) or below a number representable in it."""
    if dtype == "fp16":
        return float(np.nextafter(np.float16(b), np.float16(np.inf if up else -np.inf)))
    b = np.float32(b)
    if b == 0:
        tiny = np.array([0x00010000], np.uint32).view(np.float32)[0]
        return float(tiny if up else -tiny)
    bits = np.array([b], np.float32).view(np.uint32)[0]
    away = (b > 0) == up  # moving away from zero increases the magnitude bits
    bits = bits + np.uint32(0x10000) if away else bits - np.uint32(0x10000)
    return float(np.array([bits], np.uint32).view(np.float32)[0])


def stage2_decision_boundary(abar: float, theta: float, dtype: str = "bf16") -> float:
    """The pre-rounding score at which one pooled row's stage-2 decision flips.

    The decision ``float32(rn16(raw) + diff) >= abar`` is monotone in ``raw``: it becomes true
    at the smallest bf16 value ``b`` with ``float32(b + diff) >= abar``, and ``rn16(raw)`` reaches
    ``b`` when ``raw`` crosses the midpoint between ``b`` and the bf16 value below it."""
    diff = np.float32(theta * LOG2E)
    abar = np.float32(abar)
    b = float(rnd16(np.array([np.float32(abar - diff)], np.float32), dtype)[0])
    passes = lambda c: bool(np.float32(np.float32(c) + diff) >= abar)
    while passes(b):
        b = _bf16_step(b, False, dtype)
    while not passes(b):
        b = _bf16_step(b, True, dtype)
    return 0.5 * (b + _bf16_step(b, False, dtype))


def stage2_flip_distance(
    qbar_rows: np.ndarray,
    abar_rows: np.ndarray,
    abar_mean_rows: np.ndarray,
    k_row: np.ndarray,
    sm_scale: float,
    theta: float,
    dtype: str = "bf16",
) -> float:
    """Distance (in pre-rounding score units) of one key from the nearest point at which its
    stage-2 decision would flip: the minimum over the big block's pooled rows of
    ``|raw - stage2_decision_boundary|``.  A disagreement between two implementations on this key
    is excusable when the distance is below the parity band (1e-3).  If a pooled anchor's
    unrounded mean lies within 1e-4 of a bf16 rounding boundary the threshold itself is ambiguous
    at float32 accuracy and 0 is returned."""
    _, raw = stage2_scores(qbar_rows, k_row[None, :], sm_scale, dtype)
    raw = raw[:, 0].astype(np.float64)
    best = np.inf
    for i in range(raw.size):
        a = float(abar_rows[i])
        mean = float(abar_mean_rows[i])
        for nb in (_bf16_step(a, True, dtype), _bf16_step(a, False, dtype)):
            if abs(mean - 0.5 * (a + nb)) < 1e-4:
                return 0.0
        best = min(best, abs(raw[i] - stage2_decision_boundary(a, theta, dtype)))
    return float(best)

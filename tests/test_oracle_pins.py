"""Pins the CPU oracle (oracle/anchor_oracle.py) with checks that do not retype its formulas:
float64 brute force over explicit key sets, a literal walk of the reference's two tile loops,
library softmax attention, closed forms at theta -> +/-inf, torch's own bf16 cast."""
import math

import numpy as np
import pytest
import torch

from anchor_attn.synthetic import make_qkv
from oracle import anchor_oracle as ao

D = 128
S = 2048
SM = 1.0 / math.sqrt(D)


def _np(*ts):
    return [t.float().numpy() for t in ts]


@pytest.fixture(scope="module")
def small():
    """N = 3 big blocks, GQA 2:1, 96 stripes: bb = 0, 1 and 2 are all exercised."""
    q, k, v, pos = make_qkv(3 * S, 2, 1, n_stripes=96, seed=11)
    Q, K, V = _np(q, k, v)
    res = ao.anchor_attn_reference(Q, K, V, difference=12.0)
    return Q, K, V, pos.numpy(), res


# ---------------------------------------------------------------- bf16 rounding and scale chains
def test_rn16_matches_torch_cast():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(200000, generator=g) * torch.logspace(-30, 30, 200000)
    bits = torch.randint(0, 2**31 - 1, (200000,), generator=g, dtype=torch.int64).to(torch.int32)
    y = bits.view(torch.float32)
    ties = (torch.arange(1, 4097, dtype=torch.int32) << 16 | 0x8000).view(torch.float32)  # exact ties
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 1e-40, -1e-40, 3.3895e38])
    for t in (x, y[torch.isfinite(y)], ties, special):
        want = t.to(torch.bfloat16).float().numpy()
        got = ao.rn16(t.numpy())
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    assert np.isnan(ao.rn16(np.array([np.nan], np.float32))[0])


def test_scale_chain_constants_and_torch_bf16_arithmetic():
    # constants the stage-1 chain rounds to for D=128
    assert float(ao.rn16(np.array([SM], np.float32))[0]) == 0.08837890625
    assert float(ao.rn16(np.array([ao.LOG2E], np.float32))[0]) == 1.4453125
    q = torch.randn(4096, D, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    # torch evaluates bf16*bf16 as a float32 product rounded once to bf16
    t1 = (q * torch.tensor(SM, dtype=torch.bfloat16)) * torch.tensor(ao.LOG2E, dtype=torch.bfloat16)
    assert t1.dtype == torch.bfloat16
    assert np.array_equal(t1.float().numpy(), ao.q1_scale_chain(q.float().numpy(), SM))
    t3 = ((q.float() * torch.tensor(SM, dtype=torch.float32)) * torch.tensor(ao.LOG2E, dtype=torch.float32)).to(torch.bfloat16)
    assert np.array_equal(t3.float().numpy(), ao.q3_scale_chain(q.float().numpy(), SM))
    # the two chains really differ (that is why both exist): ratio ~1.0017
    r = ao.q1_scale_chain(np.full(1, 64.0, np.float32), SM)[0] / (64.0 * SM * ao.LOG2E)
    assert abs(r - 1.0017) < 2e-3 and r != 1.0


# ---------------------------------------------------------------- stage 1
def _literal_stage1_block(Qh, Kh, Vh, m_idx, sm_scale, block=128, step=16):
    """Walk the two loops of the reference's stage-1 program for ONE 128-query block exactly as
    written (loop bounds, pointer start/advance, additive mask) in float64; returns (M, L, Acc).
    anchor_step_1_2_v2.py:42-44 (offsets), :97-112 (local pointers), :125-156 (loops)."""
    big = (m_idx * block) // (block * step)
    init_offset = min(1 * block * step, (m_idx + 1) * block)
    local_offset = max((big - 1 + 1) * block * step, 0)
    rows = np.arange(m_idx * block, (m_idx + 1) * block)
    q = ao.q1_scale_chain(Qh[rows], sm_scale).astype(np.float64)
    m = np.full(block, -np.inf)
    l = np.zeros(block)
    acc = np.zeros((block, Qh.shape[1]))

    def tile(kptr, j, m, l, acc):
        s = q @ Kh[kptr : kptr + block].astype(np.float64).T
        s = s + np.where((np.arange(block)[None, :] + j) <= rows[:, None], 0.0, -1e6)
        m_new = np.maximum(m, s.max(1))
        p = np.exp2(s - m_new[:, None])
        a = np.exp2(m - m_new)
        return m_new, l * a + p.sum(1), acc * a[:, None] + p @ Vh[kptr : kptr + block].astype(np.float64)

    kptr = 0
    for j in range(0, init_offset, block):
        m, l, acc = tile(kptr, j, m, l, acc)
        kptr += block
    kptr = local_offset
    for j in range(max(local_offset, init_offset), (big + 1) * block * step, block):
        m, l, acc = tile(kptr, j, m, l, acc)
        kptr += block
    return m, l, acc


def _window_mask(N):
    """W(r) = [0,S) U [bb*S, r] for bb>=1, [0,r] for bb=0, built straight from that sentence."""
    r = np.arange(N)[:, None]
    j = np.arange(N)[None, :]
    bb = r // S
    return (j <= r) & ((j < S) | (j >= bb * S))


def test_stage1_literal_walk_equals_window_closed_form(small):
    Q, K, V, _, res = small
    N = Q.shape[2]
    mask = _window_mask(N)
    for h in range(2):
        q1 = ao.q1_scale_chain(Q[0, h], SM).astype(np.float64)
        s = q1 @ K[0, 0].astype(np.float64).T
        s[~mask] = -np.inf
        M = s.max(1)
        P = np.exp2(s - M[:, None])
        L = P.sum(1)
        A = P @ V[0, 0].astype(np.float64)
        # (a) the literal loop walk gives the closed-form key set (checks my reading of the loops)
        for m_idx in (0, 1, 7, 15, 16, 17, 31, 32, 40, 47):
            lm, ll, la = _literal_stage1_block(Q[0, h], K[0, 0], V[0, 0], m_idx, SM)
            rows = slice(m_idx * 128, (m_idx + 1) * 128)
            np.testing.assert_allclose(lm, M[rows], atol=1e-9)
            np.testing.assert_allclose(ll, L[rows], rtol=1e-9)
            np.testing.assert_allclose(la, A[rows], rtol=1e-7, atol=1e-9)
        # (b) the oracle agrees with the closed form: M to float32 dot accuracy, L/Acc to the
        # bf16 rounding of p (relative 2^-9 per term)
        np.testing.assert_allclose(res.M[0, h], M, atol=2e-5 * np.abs(M).max())
        np.testing.assert_allclose(res.L[0, h], L, rtol=1e-5)
        np.testing.assert_allclose(res.Acc[0, h] / res.L[0, h][:, None], A / L[:, None], atol=6e-3)


def test_stage1_is_library_causal_attention_for_first_two_big_blocks():
    q, k, v, _ = make_qkv(2 * S, 4, 2, n_stripes=32, seed=3)
    Q, K, V = _np(q, k, v)
    M, L, Acc = ao.stage1_anchor(Q, K, V, SM)
    q1 = torch.from_numpy(ao.q1_scale_chain(Q, SM)) * math.log(2.0)
    kk = torch.from_numpy(K).repeat_interleave(2, dim=1)
    vv = torch.from_numpy(V).repeat_interleave(2, dim=1)
    ref = torch.nn.functional.scaled_dot_product_attention(q1.double(), kk.double(), vv.double(), is_causal=True, scale=1.0)
    got = Acc / L[..., None]
    np.testing.assert_allclose(got, ref.numpy(), atol=6e-3)
    assert np.abs(got - ref.numpy()).mean() < 3e-4
    # the anchor is the row max of the scaled logits in the log2 domain
    s = torch.einsum("bhnd,bhmd->bhnm", q1.double() / math.log(2.0), kk.double())
    s = s.masked_fill(~torch.ones(2 * S, 2 * S, dtype=torch.bool).tril(), -float("inf"))
    np.testing.assert_allclose(M, s.amax(-1).numpy(), atol=1e-3)


def test_stage1_tile_width_only_changes_rounding(small):
    Q, K, V, _, res = small
    M2, L2, A2 = ao.stage1_anchor(Q[:, :1], K, V, SM, tile_n=64)
    assert np.array_equal(M2[0, 0], res.M[0, 0])  # a max does not depend on tiling
    np.testing.assert_allclose(L2[0, 0], res.L[0, 0], rtol=1e-5)
    np.testing.assert_allclose(A2[0, 0] / L2[0, 0][:, None], res.Acc[0, 0] / res.L[0, 0][:, None], atol=4e-3)


# ---------------------------------------------------------------- stage 2
def test_stage2_structure_and_closed_forms(small):
    Q, K, V, pos, res = small
    n_bb = Q.shape[2] // S
    for h in range(2):
        assert res.counts[0, h, 0] == 0 and res.coords[0][h][0].size == 0
        for bb in range(1, n_bb):
            c = res.coords[0][h][bb]
            assert c.dtype == np.int32 and c.size == res.counts[0, h, bb]
            assert np.all(np.diff(c) > 0)
            if c.size:
                assert c[0] >= 128 and c[-1] < bb * S - 128
    # theta -> +inf: every candidate; theta -> -inf: none; monotone in theta
    allc, alln = ao.stage2_select(Q, K, res.M, SM, 1e4)
    for bb in range(n_bb):
        want = np.arange(128, bb * S - 128, dtype=np.int32) if bb else np.zeros(0, np.int32)
        assert np.array_equal(allc[0][1][bb], want)
        assert alln[0, 1, bb] == max(bb * S - 256, 0)
    _, none = ao.stage2_select(Q, K, res.M, SM, -1e4)
    assert none.sum() == 0
    prev = None
    for theta in (8.0, 10.0, 12.0, 14.0, 16.0):
        c, _ = ao.stage2_select(Q, K, res.M, SM, theta)
        cur = [set(c[0][0][bb].tolist()) for bb in range(n_bb)]
        if prev is not None:
            assert all(a <= b for a, b in zip(prev, cur))
        prev = cur
    # on this input the stripes (and only keys carrying the stripe bias) are what gets picked
    picked = set(np.concatenate(res.coords[0][0]).tolist())
    assert picked and picked <= set(pos.tolist())


def test_stage2_independent_bruteforce(small):
    """Same decisions from an independent route: torch bf16 casts, float64 dots, dense boolean
    matrix, then the candidate slice - in the style of the reference's own torch restatement
    get_mask_block (get_mask_test.py:162-232) plus the kernel's rounding points."""
    Q, K, V, pos, res = small
    N = Q.shape[2]
    theta = 12.0
    diff = torch.tensor(theta * ao.LOG2E, dtype=torch.float32)
    for h in range(2):
        q = torch.from_numpy(Q[0, h])
        qbar = (q.view(N // 128, 128, D).double().sum(1) / 128).float().to(torch.bfloat16)
        abar = (torch.from_numpy(res.M[0, h]).view(N // 128, 128).double().sum(1) / 128).float().to(torch.bfloat16)
        raw = (qbar.double() @ torch.from_numpy(K[0, 0]).double().T) * (SM * ao.LOG2E)
        sc = raw.float().to(torch.bfloat16)
        hit = (sc.float() + diff) >= abar.float()[:, None]  # [N/128, N]
        big = hit.view(N // S, 16, N).any(1)
        for bb in range(N // S):
            want = torch.nonzero(big[bb, 128 : max(bb * S - 128, 128)])[:, 0] + 128
            got = res.coords[0][h][bb]
            sym = set(want.tolist()) ^ set(got.tolist())
            # float64-vs-float32 dots may only disagree right at a decision boundary
            for j in sym:
                rows = slice(bb * 16, bb * 16 + 16)
                ab, mean = ao.pooled_anchors(res.M[0, h], 128)
                d = ao.stage2_flip_distance(ao.pooled_queries(Q[0, h], 128)[rows], ab[rows], mean[rows], K[0, 0, j], SM, theta)
                assert d < 1e-3
            assert len(sym) <= 2


def test_stage2_decision_boundary_is_where_the_decision_flips():
    rng = np.random.default_rng(0)
    for _ in range(200):
        abar = float(ao.rn16(np.array([rng.uniform(5, 40)], np.float32))[0])
        theta = float(rng.uniform(6, 18))
        diff = np.float32(theta * ao.LOG2E)
        b = ao.stage2_decision_boundary(abar, theta)
        for eps, want in ((+1e-4, True), (-1e-4, False)):
            sc = ao.rn16(np.array([b + eps], np.float32))[0]
            assert bool(np.float32(sc + diff) >= np.float32(abar)) is want


# ---------------------------------------------------------------- stage 3 and the whole operator
def test_stage3_multiplicity_closed_form(small):
    """out_r = sum_j c_j 2^{s_rj} v_j / sum_j c_j 2^{s_rj}; c_j = [j in W(r)] + [j in Sel(bb)];
    window logits use the stage-1 scaling, stripe logits the stage-3 scaling."""
    Q, K, V, pos, res = small
    N = Q.shape[2]
    wmask = _window_mask(N)
    k64, v64 = K[0, 0].astype(np.float64), V[0, 0].astype(np.float64)
    for h in range(2):
        s1 = ao.q1_scale_chain(Q[0, h], SM).astype(np.float64) @ k64.T
        s3 = ao.q3_scale_chain(Q[0, h], SM).astype(np.float64) @ k64.T
        sel = np.zeros((N, N), bool)
        for bb in range(N // S):
            sel[bb * S : (bb + 1) * S, res.coords[0][h][bb]] = True
        s1 = np.where(wmask, s1, -np.inf)
        s3 = np.where(sel, s3, -np.inf)
        mx = np.maximum(s1.max(1), s3.max(1))
        w = np.exp2(s1 - mx[:, None]) + np.exp2(s3 - mx[:, None])
        want = (w @ v64) / w.sum(1)[:, None]
        err = np.abs(res.out[0, h] - want)
        assert err.max() < 2e-2 and err.mean() < 1.5e-3
        # the double count matters: leaving it out must break the tolerance on this input
        sel_nodup = sel & ~wmask
        w2 = np.exp2(s1 - mx[:, None]) + np.exp2(np.where(sel_nodup, s3, -np.inf) - mx[:, None])
        assert np.abs((w2 @ v64) / w2.sum(1)[:, None] - res.out[0, h]).max() > 5e-2
    assert (sel & wmask).any()


def _closed_form_check(bs, step, n_bb, dtype, head_dim=D):
    """The whole operator against an independent route: float64 window/selection masks and the multiplicity closed form
    for the output, torch casts to the 16-bit type and float64 dots for the selection - none of it shares code with the
    oracle's tile loops."""
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float16
    S_ = bs * step
    N = n_bb * S_
    sm = SM if head_dim == D else 1.0 / np.sqrt(head_dim)
    q, k, v, _ = make_qkv(N, 2, 1, head_dim=head_dim, n_stripes=max(8, N // 64), seed=300 + bs, dtype=tdt)
    Q, K, V = _np(q, k, v)
    theta = 12.0
    res = ao.anchor_attn_reference(Q, K, V, block_size=bs, step=step, difference=theta, dtype=dtype)
    assert res.counts[:, :, 0].sum() == 0 and res.counts.sum() > 0
    r = np.arange(N)[:, None]
    j = np.arange(N)[None, :]
    bb_r = r // S_
    wmask = (j <= r) & ((j < S_) | (j >= bb_r * S_))
    k64, v64 = K[0, 0].astype(np.float64), V[0, 0].astype(np.float64)
    diff = torch.tensor(theta * ao.LOG2E, dtype=torch.float32)
    for h in range(2):
        # ---- selection, independently
        qt = torch.from_numpy(Q[0, h])
        qbar = (qt.view(N // bs, bs, head_dim).double().sum(1) / bs).float().to(tdt)
        s1 = ao.q1_scale_chain(Q[0, h], sm, dtype=dtype).astype(np.float64) @ k64.T
        m_rows = np.where(wmask, s1, -np.inf).max(1)                       # the anchors are the windowed row maxima
        np.testing.assert_allclose(res.M[0, h], m_rows, atol=2e-4)
        abar = (torch.from_numpy(res.M[0, h]).view(N // bs, bs).double().sum(1) / bs).float().to(tdt)
        sc = ((qbar.double() @ torch.from_numpy(K[0, 0]).double().T) * (sm * ao.LOG2E)).float().to(tdt)
        hit = ((sc.float() + diff) >= abar.float()[:, None]).view(n_bb, step, N).any(1)
        sel = np.zeros((N, N), bool)
        for bb in range(n_bb):
            lo, hi = bs, bb * S_ - bs
            want = (torch.nonzero(hit[bb, lo:hi])[:, 0] + lo).numpy() if hi > lo else np.zeros(0, np.int64)
            got = res.coords[0][h][bb]
            assert got.size == 0 or (got[0] >= lo and got[-1] < hi)
            assert len(set(want.tolist()) ^ set(got.tolist())) <= 2          # float64 vs float32 dots at a boundary
            sel[bb * S_:(bb + 1) * S_, got] = True
        # ---- output: multiplicity closed form
        s3 = ao.q3_scale_chain(Q[0, h], sm, dtype=dtype).astype(np.float64) @ k64.T
        a = np.where(wmask, s1, -np.inf)
        b = np.where(sel, s3, -np.inf)
        mx = np.maximum(a.max(1), b.max(1))
        w = np.exp2(a - mx[:, None]) + np.exp2(b - mx[:, None])
        err = np.abs(res.out[0, h] - (w @ v64) / w.sum(1)[:, None])
        assert err.max() < 2e-2 and err.mean() < 1.5e-3
    return res


@pytest.mark.parametrize("bs,step,n_bb", [(16, 16, 5), (32, 32, 3), (64, 16, 4), (256, 16, 2)])
def test_other_block_sizes_by_independent_closed_form(bs, step, n_bb):
    """block_size is a parameter of all three stages (pooling width, candidate range [bs, bb*S - bs), big block
    S = bs*step, window [0,S) U [bb*S, r]): every block size the reference's assert admits."""
    _closed_form_check(bs, step, n_bb, "bf16")


@pytest.mark.parametrize("bs,step,n_bb,dtype", [(128, 16, 3, "bf16"), (64, 16, 4, "bf16"), (128, 16, 2, "fp16")])
def test_head_dim_64_by_independent_closed_form(bs, step, n_bb, dtype):
    """The reference's kernels take the head dimension from the tensors (anchor_attn_v4.py:263, anchor_step_1_2_v2.py:21);
    the default softmax scale is then 1/sqrt(64) = 0.125, which both scale chains represent exactly."""
    res = _closed_form_check(bs, step, n_bb, dtype, head_dim=64)
    assert res.out.shape[-1] == 64


# ---------------------------------------------------------------- fp16 tensors
def test_fp16_rounding_matches_torch_cast():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(200000, generator=g) * torch.logspace(-9, 5, 200000)
    ties = torch.arange(1, 2049, dtype=torch.float32) * 2.0 ** -11 + 1.0          # 1 + k/2048: every second one is a tie
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 1e-8, -3e-8, 65504.0, 65519.9, 65520.0, 1e6, 6.1e-5, 5.9e-8])
    for t in (x, ties, special):
        want = t.to(torch.float16).float().numpy()
        got = ao.rnd16(t.numpy(), "fp16")
        assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    assert np.array_equal(ao.rnd16(x.numpy(), "bf16"), ao.rn16(x.numpy()))
    with pytest.raises(ValueError):
        ao.rnd16(x.numpy(), "fp8")


def test_fp16_scale_chains_are_torch_half_arithmetic():
    """With fp16 tensors the stage-1 chain rounds both constants and both products to fp16 (torch evaluates a
    half*half product as a float32 product rounded once), the stage-3 chain rounds once."""
    q = torch.randn(4096, D, generator=torch.Generator().manual_seed(2)).to(torch.float16)
    t1 = (q * torch.tensor(SM, dtype=torch.float16)) * torch.tensor(ao.LOG2E, dtype=torch.float16)
    assert t1.dtype == torch.float16
    assert np.array_equal(t1.float().numpy(), ao.q1_scale_chain(q.float().numpy(), SM, dtype="fp16"))
    t3 = ((q.float() * torch.tensor(SM, dtype=torch.float32)) * torch.tensor(ao.LOG2E, dtype=torch.float32)).to(torch.float16)
    assert np.array_equal(t3.float().numpy(), ao.q3_scale_chain(q.float().numpy(), SM, dtype="fp16"))
    # fp16 keeps three more bits than bf16: the chain stays within 1e-3 of the exact scale (bf16: 1.0017)
    r = ao.q1_scale_chain(np.full(1, 64.0, np.float32), SM, dtype="fp16")[0] / (64.0 * SM * ao.LOG2E)
    assert abs(r - 1.0) < 1e-3 and (ao.q1_scale_chain(q.float().numpy(), SM, dtype="fp16") != ao.q1_scale_chain(q.float().numpy(), SM)).any()


@pytest.mark.parametrize("bs,step,n_bb", [(128, 16, 3), (64, 16, 4)])
def test_fp16_operator_by_independent_closed_form(bs, step, n_bb):
    res = _closed_form_check(bs, step, n_bb, "fp16")
    # the decision-boundary helper works in fp16 steps too
    b = ao.stage2_decision_boundary(24.5, 12.0, "fp16")
    for eps, want in ((+1e-4, True), (-1e-4, False)):
        sc = ao.rnd16(np.array([b + eps], np.float32), "fp16")[0]
        assert bool(np.float32(sc + np.float32(12.0 * ao.LOG2E)) >= np.float32(24.5)) is want
    assert res.counts.sum() > 0


def test_stage3_constant_values_give_that_value(small):
    Q, K, V, pos, res = small
    row = ao.rn16(np.linspace(-2, 2, D).astype(np.float32))
    Vc = np.broadcast_to(row, V.shape).copy()
    out = ao.anchor_attn_reference(Q, K, Vc, difference=12.0).out
    np.testing.assert_allclose(out, np.broadcast_to(row, out.shape), atol=2e-2, rtol=1e-2)


def test_theta_minus_inf_at_two_big_blocks_is_dense_causal_attention():
    q, k, v, _ = make_qkv(2 * S, 2, 2, n_stripes=32, seed=5)
    Q, K, V = _np(q, k, v)
    res = ao.anchor_attn_reference(Q, K, V, difference=-1e4)
    assert res.counts.sum() == 0 and res.ratio == 0.0
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(Q).double(), torch.from_numpy(K).double(), torch.from_numpy(V).double(), is_causal=True
    ).numpy()
    err = np.abs(res.out - ref)
    # stage-1 scale chain inflates logits by 1.0017: allow for it
    assert err.max() < 3e-2 and err.mean() < 2e-3


def test_ratio_formula_and_gap(small):
    Q, K, V, pos, res = small
    B, H, N, _ = Q.shape
    assert res.ratio == res.counts.sum() / math.floor(B * H * N * N / 2048 / 2)
    assert ao.sparsity_ratio(np.array([[[0, 1792]]]), 1, 1, 4096, 128, 16) == 1792 / 4096.0
    # keys in [bb*S-128, bb*S) are never candidates for bb >= 2
    allc, _ = ao.stage2_select(Q, K, res.M, SM, 1e4)
    assert allc[0][0][2].max() == 2 * S - 129


def test_reference_layout_packing(small):
    Q, K, V, pos, res = small
    tc = ao.coords_to_reference_layout(res.coords, res.counts, Q.shape[2])
    assert tc.shape == (1, 2, 3, Q.shape[2]) and tc.dtype == np.int32
    c = res.coords[0][1][2]
    assert np.array_equal(tc[0, 1, 2, : c.size], c) and not tc[0, 1, 2, c.size :].any()


def test_intended_geometry_candidate_range_and_dense_limit():
    """strict_reference=False: candidates are exactly [S, bb*S) (theta -> +inf selects all of them), and then the
    operator has no double-counted key and no gap, so it equals plain causal attention - which the as-run
    geometry does not (keys below S counted twice, the last 128 keys before each big block missing)."""
    rng = np.random.default_rng(11)
    N, H = 3 * 2048, 1
    Q = ao.rn16(rng.standard_normal((1, H, N, 128)).astype(np.float32))
    K = ao.rn16(rng.standard_normal((1, H, N, 128)).astype(np.float32))
    V = ao.rn16(rng.standard_normal((1, H, N, 128)).astype(np.float32))
    res = ao.anchor_attn_reference(Q, K, V, difference=1e4, strict_reference=False)
    for bb in range(3):
        want = np.arange(2048, bb * 2048, dtype=np.int32) if bb >= 2 else np.zeros(0, np.int32)
        assert np.array_equal(res.coords[0][0][bb], want)
    q = torch.from_numpy(Q).double(); k = torch.from_numpy(K).double(); v = torch.from_numpy(V).double()
    dense = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True).numpy()
    assert np.abs(res.out - dense).max() < 2e-2 and np.abs(res.out - dense).mean() < 2e-3
    as_run = ao.anchor_attn_reference(Q, K, V, difference=1e4)
    assert np.abs(as_run.out[0, 0, 2 * 2048:] - dense[0, 0, 2 * 2048:]).max() > 5e-2


def test_oracle_regression_fixture():
    """The committed fixture (tests/golden/, written by this repository's oracle, see the script there) still
    matches: index lists exactly, floating-point results to BLAS-rounding tolerance."""
    import importlib.util
    import os
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    spec = importlib.util.spec_from_file_location("make_oracle_fixture", os.path.join(here, "make_oracle_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    got = mod.run_case()
    want = np.load(os.path.join(here, "oracle_small_case.npz"))
    assert np.array_equal(got["stripe_positions"], want["stripe_positions"])
    assert np.array_equal(got["counts"], want["counts"]) and np.array_equal(got["coords"], want["coords"])
    assert float(got["ratio"]) == float(want["ratio"])
    np.testing.assert_allclose(got["M"], want["M"], atol=1e-5)
    np.testing.assert_allclose(got["L"], want["L"], rtol=1e-5)
    np.testing.assert_allclose(got["out"], want["out"], atol=1e-5)


def test_scale_chains_match_triton_compiled_outputs():
    """Pins the two query pre-scaling chains against the Triton toolchain itself.  tests/golden/
    triton_scale_chain_probe.npz holds what tests/triton_promotion_probe.py (own micro-kernels with the two forms
    of the reference's expression, compiled by Triton 3.6.0 for gfx950 and run on an MI355X) returned for every
    bf16 value with 2^-8 <= |x| < 2^8 and for zero: a constexpr sm_scale keeps the products in bf16 (stage 1), a
    run-time sm_scale promotes them to float32 (stage 3).  Bit-exact, three scales."""
    import os
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "triton_scale_chain_probe.npz"))
    unbits = lambda b: (b.astype(np.uint32) << 16).view(np.float32)
    x = unbits(fx["x_bf16_bits"])
    assert x.size > 4000
    for name in ("d128", "d64", "odd"):
        sm = float(fx[f"sm_{name}"])
        want1, want3 = unbits(fx[f"constexpr_{name}_bf16_bits"]), unbits(fx[f"runtime_{name}_bf16_bits"])
        assert np.array_equal(ao.q1_scale_chain(x, sm, mode="bf16_chain"), want1)
        assert np.array_equal(ao.q3_scale_chain(x, sm), want3)
        assert np.array_equal(ao.q1_scale_chain(x, sm, mode="fp32"), want3)
        assert (want1 != want3).sum() > 500  # the two chains are different functions, so the pin discriminates
    # element-wise stage-2 test: constexpr qk_scale * literal, bf16 rounding of the score, float32 "+ diff >= anchor"
    dot, anchor = fx["s2_dot"], unbits(fx["s2_anchor_bf16_bits"])
    sm, theta = float(fx["s2_sm"]), float(fx["s2_theta"])
    raw = (dot * np.float32(sm * ao.LOG2E)).astype(np.float32)
    assert np.array_equal(ao.rn16(raw), unbits(fx["s2_qk_bf16_bits"]))
    hit = (ao.rn16(raw) + np.float32(theta * ao.LOG2E)) >= anchor
    assert np.array_equal(hit, fx["s2_hit"].astype(bool)) and 0.2 < hit.mean() < 0.8
    assert ((raw + np.float32(theta * ao.LOG2E) >= anchor) != hit).sum() > 300       # un-rounded score: a different test
    # the oracle's own boundary helper agrees with the compiled decisions
    for i in range(0, dot.size, 97):
        xb = ao.stage2_decision_boundary(float(anchor[i]), theta)
        if float(raw[i]) != xb:  # (exactly on the midpoint the bf16 tie rule decides)
            assert (float(raw[i]) > xb) == bool(fx["s2_hit"][i])


def test_fp16_chains_match_triton_compiled_outputs():
    """The fp16 half of the same probe (tests/golden/triton_scale_chain_probe_fp16.npz): on fp16 tensors the constexpr
    form keeps both products in fp16, the run-time form rounds once; the stage-2 score is one rounding of the exact
    product (the multiply and the cast compile into one mixed-precision instruction)."""
    import os
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "triton_scale_chain_probe_fp16.npz"))
    unbits = lambda b: b.view(np.float16).astype(np.float32)
    x = unbits(fx["x_f16_bits"])
    assert x.size > 4000
    for name in ("d128", "d64", "odd"):
        sm = float(fx[f"sm_{name}"])
        want1, want3 = unbits(fx[f"constexpr_{name}_f16_bits"]), unbits(fx[f"runtime_{name}_f16_bits"])
        assert np.array_equal(ao.q1_scale_chain(x, sm, mode="bf16_chain", dtype="fp16"), want1)
        assert np.array_equal(ao.q3_scale_chain(x, sm, dtype="fp16"), want3)
        assert (want1 != want3).sum() > 500
        assert (want1 != ao.q1_scale_chain(x, sm, mode="bf16_chain", dtype="bf16")).sum() > 500  # and not the bf16 chain
    dot, anchor, qk = fx["s2_dot"], unbits(fx["s2_anchor_f16_bits"]), unbits(fx["s2_qk_f16_bits"])
    sm, theta = float(fx["s2_sm"]), float(fx["s2_theta"])
    # the compiled stage-2 score: one rounding of the exact product (the oracle's fp16 reading), which differs from the
    # two roundings of the source text on exact ties only
    sc, raw = ao.stage2_scores(dot[:, None].astype(np.float32), np.ones((1, 1), np.float32), sm, "fp16")  # dot * 1 = dot
    sc, raw = sc[:, 0], raw[:, 0]
    assert np.array_equal(sc, qk)
    two = ao.rnd16(raw, "fp16")
    odd = np.nonzero(two != qk)[0]
    assert 0 < odd.size <= 8
    for i in odd:
        assert abs(float(raw[i]) - float(two[i])) == abs(float(raw[i]) - float(qk[i]))  # exact ties only
    hit = (sc + np.float32(theta * ao.LOG2E)) >= anchor
    assert np.array_equal(hit, fx["s2_hit"].astype(bool)) and 0.2 < hit.mean() < 0.8

"""Head dimension 64 (the reference's kernels are generic in D: anchor_attn_v4.py:263 ``BLOCK_DMODEL=D``,
anchor_step_1_2_v2.py:21 ``D: tl.constexpr``): the gfx950 kernels instantiated for 64 against the CPU oracle, stage by
stage and end to end, at the tolerances of the 128-wide tests (index sets identical except keys whose pre-rounding
score lies within 1e-3 of a decision flip; outputs max |err| <= 2e-2 and mean |err| <= 2e-3)."""
import math

import numpy as np
import pytest
import torch

from test_gpu_parity import LOG2E, _assert_index_parity, _assert_outputs_close, _np, _packed_lists, mods  # noqa: F401

pytestmark = pytest.mark.gpu

D = 64
SM = 1.0 / math.sqrt(D)


def _case64(n_ctx, hq, hkv, n_stripes, seed, **kw):
    from anchor_attn.synthetic import make_qkv
    return make_qkv(n_ctx, hq, hkv, head_dim=D, n_stripes=n_stripes, seed=seed, **kw)[:3]


@pytest.mark.parametrize("n_bb,hq,hkv,bs,step,theta,seed,base,dtype", [
    (3, 8, 2, 128, 16, 12.0, 601, 5e5, torch.bfloat16),   # Llama-3.2-1B grouping (4:1)
    (4, 7, 1, 128, 16, 12.0, 602, 1e6, torch.bfloat16),   # Qwen2.5-0.5B grouping (7:1)
    (3, 4, 4, 128, 16, 13.0, 603, 5e5, torch.float16),    # fp16 tensors, pre-repeated K/V
    (2, 2, 1, 128, 32, 11.0, 604, 5e5, torch.bfloat16),   # step 32
    (5, 4, 2, 64, 16, 12.0, 605, 5e5, torch.bfloat16),    # block size 64
    (3, 4, 2, 256, 16, 12.0, 606, 5e5, torch.bfloat16),   # block size 256: the stand-alone pooling kernel
    (1, 4, 2, 128, 16, 12.0, 607, 5e5, torch.bfloat16),   # a single big block: nothing to select
    (6, 2, 1, 16, 16, 12.0, 608, 5e5, torch.bfloat16),    # block size 16: eight pooled rows per 128-row work-group
    (3, 2, 2, 32, 32, 12.0, 609, 5e5, torch.bfloat16),    # block size 32, step 32
    (3, 2, 1, 128, 16, 1e4, 610, 5e5, torch.bfloat16),    # every candidate selected: lists of 1792 and 3840 entries (the
                                                          # sparse kernel refills its 1024-entry index window)
])
def test_end_to_end(mods, n_bb, hq, hkv, bs, step, theta, seed, base, dtype):
    hip, v4, st, ao = mods
    q, k, v = _case64(n_bb * bs * step, hq, hkv, 32 * n_bb, seed, rope_base=base, dtype=dtype)
    Q, K, V = _np(q, k, v)
    name = "fp16" if dtype == torch.float16 else "bf16"
    res = ao.anchor_attn_reference(Q, K, V, block_size=bs, step=step, difference=theta, dtype=name)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, ratio = v4.anchor_attn(qd, kd, vd, block_size=bs, step=step, difference=theta)
    B, H, N, _ = q.shape
    L, M, Acc = st.anchor_attn_step_1(qd, kd, vd, 1, 1, bs, step, B, H, N, D, SM)
    np.testing.assert_allclose(M.cpu().numpy(), res.M, atol=3e-4)
    np.testing.assert_allclose(L.cpu().numpy(), res.L, rtol=5e-4)
    err = np.abs(st.acc_rows(Acc).cpu().numpy() / L.cpu().numpy()[..., None] - res.Acc / res.L[..., None])
    assert err.max() < 6e-3 and err.mean() < 3e-4
    coords, counts = st.select_stripes_packed(qd, kd, M, bs, step, theta * LOG2E, B, H, N, D, SM)
    got, got_counts = _packed_lists(hip, coords, counts, N, step, bs)
    _assert_index_parity(ao, got, got_counts, res.coords, Q, K, res.M, theta, 8, step, bs, name, sm=SM)
    assert (res.counts.sum() > 0 or n_bb == 1) and out.dtype == dtype
    _assert_outputs_close(out.float().cpu().numpy(), res.out, name)
    assert abs(float(ratio) - got_counts.sum() / ((B * H * N * N / (bs * step)) // 2)) < 1e-6
    # the one-call entry point (pooling fused into stage 1 for block sizes up to 128) against the staged ones
    staged, ratio2 = v4.anchor_attn_without_anchor(qd, kd, vd, block_size=bs, step=step, difference=theta)
    assert torch.equal(out, staged) and float(ratio) == float(ratio2)


def test_batch_of_two(mods):
    """Two batch elements with different contents: each equals its own single-batch run bit for bit."""
    hip, v4, st, ao = mods
    a = _case64(3 * 2048, 4, 2, 64, 631)
    b = _case64(3 * 2048, 4, 2, 64, 632)
    q, k, v = (torch.cat([x, y], 0).cuda() for x, y in zip(a, b))
    out, ratio = v4.anchor_attn(q, k, v, difference=12.0)
    for i, one in enumerate((a, b)):
        o1 = v4.anchor_attn(*(t.cuda() for t in one), difference=12.0, return_computational_ratio=False)
        assert torch.equal(out[i:i + 1], o1)
    assert 0.0 < float(ratio) < 0.2


def test_stages_pooling_and_dense_baseline(mods):
    """Pooling bit-exact (stand-alone kernel and the one fused into stage 1), stage 3 given the same state, the dense
    baseline against float64 library attention, strided [B,N,H,D] storage, and a repeat that is bit-identical."""
    hip, v4, st, ao = mods
    bs, step = 128, 16
    q, k, v = _case64(3 * 2048, 4, 2, 96, 611)
    Q, K, V = _np(q, k, v)
    res = ao.anchor_attn_reference(Q, K, V, difference=12.0)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    B, H, N, _ = q.shape
    qbar, abar = st.pool_q_anchor(qd, torch.from_numpy(res.M).cuda(), bs)
    assert qbar.shape == (B, H, N // bs, D)
    for h in range(H):
        assert np.array_equal(qbar[0, h].float().cpu().numpy(), ao.pooled_queries(Q[0, h], bs))
        assert np.array_equal(abar[0, h].float().cpu().numpy(), ao.pooled_anchors(res.M[0, h], bs)[0])
    L, M, Acc = st.anchor_attn_step_1(qd, kd, vd, 1, 1, bs, step, B, H, N, D, SM)
    coords, counts = st.select_stripes_packed(qd, kd, M, bs, step, 12.0 * LOG2E, B, H, N, D, SM)
    out = v4._stage3(qd, kd, vd, coords, counts, L, M, Acc, SM, bs, step)
    lists, cnts = _packed_lists(hip, coords, counts, N)
    want = ao.stage3_sparse(Q, K, V, lists, cnts, M.cpu().numpy(), L.cpu().numpy(), st.acc_rows(Acc).cpu().numpy(), SM)
    _assert_outputs_close(out.float().cpu().numpy(), want)
    dense = v4.dense_causal_attention(qd, kd, vd)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.double(), k.double().repeat_interleave(2, 1), v.double().repeat_interleave(2, 1), is_causal=True)
    e = (dense.cpu().double() - ref).abs()
    assert e.max() < 2e-2 and e.mean() < 1e-3
    # the layout transformers hands over: [B,H,N,D] views of [B,N,H,D] storage, and an output view of the same kind
    qh, kh, vh = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (qd, kd, vd))
    plain = v4.anchor_attn(qd, kd, vd, return_computational_ratio=False)
    out_store = torch.empty(B, N, H, D, dtype=q.dtype, device="cuda")
    v4.anchor_attn(qh, kh, vh, return_computational_ratio=False, out=out_store.transpose(1, 2))
    assert torch.equal(out_store.transpose(1, 2), plain)
    assert torch.equal(v4.anchor_attn(qd, kd, vd, return_computational_ratio=False), plain)
    # theta -> -inf with two big blocks is plain causal attention
    o2, r2 = v4.anchor_attn(qd[:, :, :4096].contiguous(), kd[:, :, :4096].contiguous(), vd[:, :, :4096].contiguous(), difference=-1e4)
    assert float(r2) == 0.0
    e2 = (o2.cpu().double() - ref[:, :, :4096]).abs()
    assert e2.max() < 3e-2 and e2.mean() < 2e-3


def test_llama_1b_shape_at_32k_sampled_rows(mods):
    """The Llama-3.2-1B layer shape (32 q / 8 KV heads, head dimension 64) at 32768 tokens: staged == one-call bit for
    bit, finite, and sampled rows of the output against a float64 recomputation of stages 1 and 3 with the kernel's
    own index lists."""
    hip, v4, st, ao = mods
    from anchor_attn.synthetic import make_qkv
    from test_gpu_parity import _check_sampled_rows
    N, hq, hkv, bs, step = 32768, 32, 8, 128, 16
    q, k, v, _ = make_qkv(N, hq, hkv, head_dim=D, n_stripes=256, seed=621)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    out, ratio = v4.anchor_attn(qd, kd, vd, difference=12.0)
    staged, ratio2 = v4.anchor_attn_without_anchor(qd, kd, vd, difference=12.0)
    assert torch.equal(out, staged) and float(ratio) == float(ratio2) and 0.0005 < float(ratio) < 0.2
    assert torch.isfinite(out.float()).all()
    L, M, Acc = st.anchor_attn_step_1(qd, kd, vd, 1, 1, bs, step, 1, hq, N, D, SM)
    coords, counts = st.select_stripes_packed(qd, kd, M, bs, step, 12.0 * LOG2E, 1, hq, N, D, SM)
    lib = hip.lib()
    cnt = counts.reshape(hq, -1).cpu().numpy()
    cds = coords[0].cpu().numpy()

    def index_list(h, bb):
        off = lib.aa_coords_offset(bb, bs, step)
        return cds[h, off:off + cnt[h, bb]]

    _check_sampled_rows(ao, q, k, v, M.cpu().numpy(), L.cpu().numpy(), out, index_list,
                        [(0, N - 1), (5, 2047), (9, 2048), (17, 20000), (31, N - 2048), (22, 12345)], sm=SM)

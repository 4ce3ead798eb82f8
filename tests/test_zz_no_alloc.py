"""The entry point that allocates nothing: aa_stage2_select_static keeps the stage-2 bitmask and thresholds in a
static device array inside the library.  It must give exactly what aa_stage2_select gives with a caller-provided
buffer (integer work: bit-exact), on two calls in a row that share the array, the second on a smaller problem."""
import math

import pytest
import torch

D, BS, STEP, S = 128, 128, 16, 2048
SM = 1.0 / math.sqrt(D)
LOG2E = 1.44269504


def _select_both_ways(n_ctx, hq, hkv, n_stripes, seed, theta):
    from anchor_attn.src.ops import _hip, anchor_step_1_2_v2 as st
    from anchor_attn.synthetic import make_qkv
    lib = _hip.lib()
    q, k, v, _ = make_qkv(n_ctx, hq, hkv, n_stripes=n_stripes, seed=seed)
    q, k, v = q.cuda(), k.cuda(), v.cuda()
    B, H, N, _ = q.shape
    L, M, Acc = st.anchor_attn_step_1(q, k, v, 1, 1, BS, STEP, B, H, N, D, SM)
    qbar, abar = st.pool_q_anchor(q, M, BS)
    n_bb = N // S
    per_head = lib.aa_coords_entries_per_head(N, BS, STEP)
    stream = torch.cuda.current_stream().cuda_stream

    def outputs():
        # poisoned, so that an entry the kernels do not write cannot agree by accident
        return (torch.full((B, H, max(per_head, 1)), -1, dtype=torch.int32, device="cuda"),
                torch.full((B, H, n_bb), -1, dtype=torch.int32, device="cuda"))

    coords_a, counts_a = outputs()
    mask = torch.empty((lib.aa_mask_words(B, H, N, BS, STEP),), dtype=torch.int32, device="cuda")
    _hip.check(lib.aa_stage2_select(qbar.data_ptr(), abar.data_ptr(), *_hip.t3(k), mask.data_ptr(), coords_a.data_ptr(),
                                    counts_a.data_ptr(), B, H, hkv, N, D, BS, STEP, SM, theta * LOG2E, 0, _hip.AA_DTYPE_BF16, stream))
    coords_b, counts_b = outputs()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    _hip.check(lib.aa_stage2_select_static(qbar.data_ptr(), abar.data_ptr(), *_hip.t3(k), coords_b.data_ptr(),
                                           counts_b.data_ptr(), B, H, hkv, N, D, BS, STEP, SM, theta * LOG2E, 0, _hip.AA_DTYPE_BF16, stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # nothing came from torch's allocator either
    return coords_a, counts_a, coords_b, counts_b


@pytest.mark.gpu
def test_static_scratch_entry_point_equals_the_allocating_one_twice_in_a_row():
    from anchor_attn.src.ops import _hip
    lib = _hip.lib()
    total = 0
    # the second problem is smaller in every dimension: it reuses the front of the array the first one filled
    for n_ctx, hq, hkv, n_stripes, seed, theta in [(5 * S, 8, 2, 200, 11, 12.0), (2 * S, 2, 1, 48, 12, 13.0)]:
        coords_a, counts_a, coords_b, counts_b = _select_both_ways(n_ctx, hq, hkv, n_stripes, seed, theta)
        assert torch.equal(counts_a, counts_b) and int(counts_a.min()) >= 0
        assert torch.equal(coords_a, coords_b)  # written entries identical, unwritten entries still poisoned in both
        total += int(counts_a.sum())
        assert int(counts_a[:, :, 0].sum()) == 0 and int(counts_a.sum()) > 0
    assert total > 0
    # a problem beyond the static capacity is refused before anything is launched
    need = lib.aa_mask_words(1, 64, 131072, BS, STEP) * 4
    assert need > _hip.AA_STATIC_SCRATCH_BYTES
    rc = lib.aa_stage2_select_static(1, 1, 1, 0, 0, 128, 1, 1, 1, 64, 8, 131072, D, BS, STEP, SM, 17.0, 0, 0, None)
    assert rc == 2 and b"static scratch" in lib.aa_last_error()
    # the headline layer shape fits
    assert lib.aa_mask_words(1, 32, 131072, BS, STEP) * 4 <= _hip.AA_STATIC_SCRATCH_BYTES

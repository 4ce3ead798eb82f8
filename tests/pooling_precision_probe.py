"""How much the selection depends on the precision in which the pooled queries are accumulated.

The reference pools with ``tl.sum(q, axis=1) / BLOCK_SZ`` on a bf16 tile (get_mask_test.py:75-78).  What that
means depends on the Triton release: up to 3.1 ``tl.sum`` promoted bf16 inputs to float32 before reducing; the
3.6.0 in this image reduces in the input type (every partial sum of the reduction tree is rounded to bf16), and
the tree's order is a property of the backend's register layout.  The library and its oracle accumulate in
float32 (ascending row order).  This script measures, on one workload, what the other reading would change:
it pools with an own Triton micro-kernel written like the reference's lines, feeds those pooled queries to the
library's stage 2 (the C ABI takes them as an input) and compares index lists and final outputs.

    python tests/pooling_precision_probe.py [--workload config2_llama8b_128k]      (needs a GPU and Triton)

One JSON line comes out; tests/test_gpu_parity.py::test_pooling_precision_reading_is_immaterial runs this file in a
process of its own and asserts on that line.
"""
import argparse
import json
import math
import os
import sys

import torch
import triton
import triton.language as tl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path[:0] = [ROOT, os.path.join(ROOT, "anchor-attention_amd")]


@triton.jit
def _pool_big_block(q_ptr, qbar_ptr, q_sh, q_sn, step: tl.constexpr, BLOCK_SZ: tl.constexpr, D: tl.constexpr):
    bb = tl.program_id(0)
    h = tl.program_id(1)
    rows = bb * step * BLOCK_SZ + tl.arange(0, step * BLOCK_SZ)
    q = tl.load(q_ptr + h * q_sh + rows[:, None] * q_sn + tl.arange(0, D)[None, :])
    q = tl.reshape(q, (step, BLOCK_SZ, D))
    q = tl.sum(q, axis=1, keep_dims=False) / BLOCK_SZ
    q = q.to(q_ptr.dtype.element_ty)
    out_rows = (h * tl.num_programs(0) + bb) * step + tl.arange(0, step)
    tl.store(qbar_ptr + out_rows[:, None] * D + tl.arange(0, D)[None, :], q)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="config2_llama8b_128k")
    ap.add_argument("--theta", type=float, default=12.0)
    args = ap.parse_args()
    from bench import make_inputs
    from anchor_attn.src.ops import _hip, anchor_attn_v4 as v4, anchor_step_1_2_v2 as st
    q, k, v = make_inputs(args.workload, 0, "shared", "cuda:0")
    B, H, N, D = q.shape
    BS, STEP = 128, 16
    S, sm = BS * STEP, 1.0 / math.sqrt(D)
    lib = _hip.lib()
    L, M, Acc = st.anchor_attn_step_1(q, k, v, 1, 1, BS, STEP, B, H, N, D, sm)
    qbar, abar = st.pool_q_anchor(q, M, BS)
    qbar_t = torch.empty_like(qbar)
    _pool_big_block[(N // S, H)](q, qbar_t, q.stride(1), q.stride(2), STEP, BS, D)

    def select(qb):
        mask = torch.empty((lib.aa_mask_words(B, H, N, BS, STEP),), dtype=torch.int32, device=q.device)
        coords = torch.zeros((B, H, lib.aa_coords_entries_per_head(N, BS, STEP)), dtype=torch.int32, device=q.device)
        counts = torch.empty((B, H, N // S, 1), dtype=torch.int32, device=q.device)
        _hip.check(lib.aa_stage2_select(qb.data_ptr(), abar.data_ptr(), *_hip.t3(k), mask.data_ptr(), coords.data_ptr(),
                                        counts.data_ptr(), B, H, k.shape[1], N, D, BS, STEP, sm, args.theta * v4.LOG2E,
                                        _hip.AA_GEOMETRY_AS_RUN, _hip.AA_DTYPE_BF16, torch.cuda.current_stream().cuda_stream))
        return coords, counts

    c0, n0 = select(qbar)
    c1, n1 = select(qbar_t)
    out0 = v4._stage3(q, k, v, c0, n0, L, M, Acc, sm, BS, STEP)
    out1 = v4._stage3(q, k, v, c1, n1, L, M, Acc, sm, BS, STEP)
    # symmetric difference of the index sets, per (head, big block), via one-hot rows built on the GPU
    changed = 0
    for h in range(H):
        for bb in range(1, N // S):
            off = lib.aa_coords_offset(bb, BS, STEP)
            a = c0[0, h, off:off + int(n0[0, h, bb, 0])].long()
            b = c1[0, h, off:off + int(n1[0, h, bb, 0])].long()
            hot = torch.zeros(bb * S, dtype=torch.int8, device=q.device)
            hot[a] += 1
            hot[b] -= 1
            changed += int((hot != 0).sum())
    d = (qbar.float() - qbar_t.float()).abs()
    err = (out0.float() - out1.float()).abs()
    big = torch.maximum(out0.float().abs().max(), out1.float().abs().max())
    print(json.dumps({
        "workload": args.workload, "theta": args.theta, "triton": triton.__version__,
        "pooled_query_elements_differing": float((d != 0).float().mean()), "pooled_query_max_abs_diff": float(d.max()),
        "selected_float32_pooling": int(n0.sum()), "selected_triton_pooling": int(n1.sum()),
        "indices_in_one_list_only": changed, "fraction_of_selected": changed / max(int(n0.sum()), 1),
        "output_max_abs_diff": float(err.max()), "output_mean_abs_diff": float(err.mean()),
        "output_max_abs": float(big),
    }))


if __name__ == "__main__":
    main()

"""Recall / sparsity sweep of the operator against dense attention.

Counterpart of the recall bookkeeping in the reference's ops_profile_v2.py:514-532 (recall at a threshold =
fraction of output elements whose absolute difference from dense attention is below it, reported next to the
method's sparsity ratio) and of the theta sweep BASELINE config 2 asks for.  Everything runs on the GPU; the
dense reference is the library's own dense causal kernel on the same MFMA core.

    python -m anchor_attn.src.ops.ops_profile_v2 --workload config2_llama8b_128k --thetas 10 11 12 13 14
"""
import argparse
import json
import os
import sys
from typing import Dict, Iterable, List

import torch

from my_utils.ops_util import get_deff

from .anchor_attn_v4 import anchor_attn, dense_causal_attention

RECALL_THRESHOLDS = (0.01, 0.005)


def recall_ratio(out: torch.Tensor, ref: torch.Tensor, threshold: float) -> float:
    """Fraction of elements with |out - ref| < threshold (ops_profile_v2.py:527-530)."""
    return float(((out.float() - ref.float()).abs() < threshold).sum()) / out.numel()


def record_recall_ratios(out: torch.Tensor, ref: torch.Tensor, sparsity_ratio, thresholds: Iterable[float] = RECALL_THRESHOLDS) -> Dict:
    return {"sparsity_ratio": float(sparsity_ratio), **{f"recall@{t}": recall_ratio(out, ref, t) for t in thresholds}}


def theta_sweep(q, k, v, thetas: Iterable[float], block_size: int = 128, step: int = 16, ref: torch.Tensor = None,
                strict_reference: bool = True) -> List[Dict]:
    """One row per theta: sparsity ratio, error against dense attention (max / mean / recall), time per call.
    ``strict_reference=False`` sweeps the intended-geometry mode of the operator (analysis only)."""
    if ref is None:
        ref = dense_causal_attention(q, k, v)
    rows = []
    out = torch.empty_like(q)
    for theta in thetas:
        anchor_attn(q, k, v, block_size=block_size, step=step, difference=theta, out=out, strict_reference=strict_reference)  # warm-up
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        _, ratio = anchor_attn(q, k, v, block_size=block_size, step=step, difference=theta, out=out, strict_reference=strict_reference)
        e1.record()
        torch.cuda.synchronize()
        mean_err, strict, loose, metrics = get_deff(ref, out, verbose=False)
        rows.append({"theta": theta, "ms": e0.elapsed_time(e1), **record_recall_ratios(out, ref, ratio),
                     "max_abs_err": metrics["max_abs_error"], "mean_abs_err": float(mean_err),
                     "cosine_similarity": metrics["cosine_similarity"]})
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="config2_llama8b_128k")
    ap.add_argument("--thetas", type=float, nargs="+", default=[10, 11, 12, 13, 14])
    ap.add_argument("--qbar-mode", default="shared")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--ideal-rows", type=int, default=0,
                    help="also evaluate the token-level ideal on the last this-many query rows of head 0 (slow)")
    args = ap.parse_args(argv)
    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", "..", ".."))
    from bench import make_inputs  # the workload generator lives with the benchmark at the repository root
    q, k, v = make_inputs(args.workload, args.seed, args.qbar_mode, "cuda:0")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ref = dense_causal_attention(q, k, v)
    e0.record()
    ref = dense_causal_attention(q, k, v)
    e1.record()
    torch.cuda.synchronize()
    print(json.dumps({"workload": args.workload, "qbar_mode": args.qbar_mode, "dense_ms": e0.elapsed_time(e1)}))
    for row in theta_sweep(q, k, v, args.thetas, ref=ref):
        print(json.dumps(row), flush=True)
    if args.ideal_rows:
        from .sparse_attn_with_pytorch import sparse_attn_with_torch
        n = args.ideal_rows
        for theta in args.thetas:
            o, r = sparse_attn_with_torch(q[:, :1, -n:], k[:, :1], v[:, :1], diff_anchor=theta, return_computational_ratio=True)
            print(json.dumps({"theta": theta, "token_level_ideal_rows": n, "kept_fraction": r,
                              **{f"recall@{t}": recall_ratio(o, ref[:, :1, -n:], t) for t in RECALL_THRESHOLDS}}), flush=True)


if __name__ == "__main__":
    main()

"""Writes tests/golden/oracle_small_case.npz: a regression fixture of THIS repository's CPU oracle.

The reference holds no golden vectors, known-answer tests or fixtures for its operator (its tests are ad-hoc
comparisons on a GPU), and it is Python + Triton, so nothing of it runs here.  The oracle is therefore pinned
by mathematics (tests/test_oracle_pins.py); this fixture only guards the oracle against accidental changes:
seeded inputs from anchor_attn.synthetic.make_qkv, and what the oracle returned for them when the pins were
green.  Re-run after a deliberate change of the oracle:  python tests/golden/make_oracle_fixture.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path[:0] = [ROOT, os.path.join(ROOT, "anchor-attention_amd")]

CASE = dict(n_ctx=3 * 2048, n_q_heads=2, n_kv_heads=1, n_stripes=48, seed=77)
THETA = 12.0
ROWS = np.array([0, 1, 127, 2047, 2048, 3000, 4095, 4096, 5000, 6143])


def run_case():
    from anchor_attn.synthetic import make_qkv
    from oracle import anchor_oracle as ao
    q, k, v, pos = make_qkv(**CASE)
    res = ao.anchor_attn_reference(q.float().numpy(), k.float().numpy(), v.float().numpy(), difference=THETA)
    lists = [res.coords[0][h][bb] for h in range(CASE["n_q_heads"]) for bb in range(CASE["n_ctx"] // 2048)]
    return dict(M=res.M[0][:, ROWS], L=res.L[0][:, ROWS], out=res.out[0][:, ROWS], counts=res.counts[0],
                coords=np.concatenate(lists).astype(np.int32), ratio=np.float64(res.ratio),
                stripe_positions=pos.numpy().astype(np.int32))


if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_small_case.npz")
    np.savez_compressed(out, **run_case())
    print("wrote", out, os.path.getsize(out), "bytes")

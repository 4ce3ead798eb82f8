"""CPU-side checks: the C-ABI library loads and exports every symbol the public header declares,
its host-only helpers compute the documented geometry, and the Python host logic around the
kernels (layout conversions, argument checks, synthetic inputs) behaves.  No kernel is launched."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

from anchor_attn.src.ops import _hip
from anchor_attn.src.ops import anchor_step_1_2_v2 as st
from anchor_attn.synthetic import make_qkv, rope_rotate_half, stripe_positions


def _declared(repo_root):
    text = open(os.path.join(repo_root, "include", "anchor_attn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(repo_root):
    names = _declared(repo_root)
    assert len(names) >= 12
    handle = ctypes.CDLL(_hip.library_path())
    for n in names:
        assert hasattr(handle, n), f"{n} is declared in the header but not exported"
    assert sorted(_hip.EXPORTS) == names, "ctypes signature table and header disagree"


def test_host_geometry_helpers():
    lib = _hip.lib()
    assert lib.aa_version() >= 1
    S, bs = 2048, 128
    for n_bb in (1, 2, 3, 4, 16, 64):
        want = sum(max(bb * S - 2 * bs, 0) for bb in range(n_bb))
        assert lib.aa_coords_entries_per_head(n_bb * S, bs, 16) == want
        assert lib.aa_coords_offset(n_bb, bs, 16) == want
    assert lib.aa_coords_offset(0, bs, 16) == 0 and lib.aa_coords_offset(1, bs, 16) == 0
    assert lib.aa_mask_words(1, 32, 131072, 128, 16) * 4 == 32 * 2**20 + 32 * 1024 * 4  # bitmask + per-pooled-row thresholds
    # step 32: big block 4096
    assert lib.aa_coords_offset(2, bs, 32) == 4096 - 256
    ws = lib.aa_workspace_bytes(1, 32, 131072, 128, 128, 16)
    acc = 32 * 131072 * 128 * 4
    assert acc < ws < acc + 2**30
    ws64 = lib.aa_workspace_bytes(1, 32, 131072, 64, 128, 16)  # head_dim 64: half the accumulator state and pooled queries
    assert ws - ws64 == acc // 2 + 32 * 1024 * 64 * 2
    assert lib.aa_workspace_bytes(1, 32, 131072, 96, 128, 16) == 0  # other head dimensions are not supported


def test_error_codes_without_touching_the_gpu():
    """Validation runs before any launch, so bad arguments can be exercised on a CPU-only host."""
    lib = _hip.lib()
    buf = ctypes.create_string_buffer(4096 + 64)
    p = (ctypes.addressof(buf) + 63) & ~63
    s = (2048 * 128 * 2, 2048 * 128, 128)
    dense = lambda q, nq, nkv, n, d, qs=s: lib.aa_dense_causal_fwd(q, *qs, p, *s, p, *s, p, *s, 1, nq, nkv, n, d, 0.1, 0, None)
    assert dense(None, 2, 2, 2048, 128) == 1 and b"q is NULL" in lib.aa_last_error()
    assert dense(p, 3, 2, 2048, 128) == 1 and b"divide" in lib.aa_last_error()
    assert dense(p, 2, 2, 2048, 96) == 2 and b"head_dim" in lib.aa_last_error()  # 128 and 64 are the supported sizes
    assert dense(p, 2, 2, 2000, 128) == 2
    assert dense(p + 2, 2, 2, 2048, 128) == 3 and b"aligned" in lib.aa_last_error()
    assert dense(p, 2, 2, 2048, 128, qs=(s[0], s[1], 132)) == 3
    rc = lib.aa_anchor_attn_fwd(p, *s, p, *s, p, *s, p, *s, p, 1024, None, 1, 2, 2, 2048, 128, 128, 16, 0.1, 12.0, 0, 0, 0, None)
    assert rc == 1 and b"workspace" in lib.aa_last_error()
    rc = lib.aa_anchor_attn_fwd(p, *s, p, *s, p, *s, p, *s, p, 1 << 40, None, 1, 2, 2, 2048 + 128, 128, 128, 16, 0.1, 12.0, 0, 0, 1, None)
    assert rc == 2 and b"multiple" in lib.aa_last_error()
    big = (s[0], s[1], 16384)  # 2^20 rows x 32 KiB per row does not fit 32-bit byte offsets
    rc = lib.aa_stage1_anchor_fwd(p, *big, p, *s, p, *s, p, p, p, 1, 2, 2, 1 << 20, 128, 128, 16, 0.1, 0, 0, None)
    assert rc == 2 and b"32-bit" in lib.aa_last_error()
    rc = lib.aa_stage1_anchor_fwd(p, *s, p, *s, p, *s, p, p, p, 1, 2, 2, 2048, 128, 128, 8, 0.1, 0, 0, None)
    assert rc == 2 and b"step" in lib.aa_last_error()
    rc = lib.aa_stage1_anchor_fwd(p, *s, p, *s, p, *s, p, p, p, 1, 2, 2, 2048, 128, 128, 16, 0.1, 7, 0, None)
    assert rc == 1 and b"scale_mode" in lib.aa_last_error()
    rc = lib.aa_stage1_anchor_fwd(p, *s, p, *s, p, *s, p, p, p, 1, 2, 2, 2048, 128, 128, 16, 0.1, 0, 5, None)
    assert rc == 1 and b"dtype" in lib.aa_last_error()
    assert lib.aa_version() == 3


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_hip, "_lib", None)
    monkeypatch.setattr(_hip, "library_path", lambda: str(tmp_path / "nope.so"))
    with pytest.raises(_hip.AnchorAttnHipError, match="no fallback"):
        _hip.lib()


def test_cpu_tensors_are_rejected():
    from anchor_attn.src.ops.anchor_attn_v4 import anchor_attn
    q = torch.zeros(1, 2, 2048, 128, dtype=torch.bfloat16)
    with pytest.raises(AssertionError, match="GPU only"):
        anchor_attn(q, q, q)


def test_acc_fragment_order_matches_the_documented_formula():
    B, H, N, D = 1, 2, 64, 128
    rows = torch.arange(B * H * N * D, dtype=torch.float32).view(B, H, N, D)
    frag = torch.empty(B * H * N * D)
    b, h = np.meshgrid(np.arange(B), np.arange(H), indexing="ij")
    for hh in range(H):
        for row in range(N):
            d = np.arange(D)
            off = ((((0 * H + hh) * (N // 32) + row // 32) * 4 + d // 32) * 4 + (d % 32) // 8) * 256 \
                + (((d % 8) // 4) * 32 + row % 32) * 4 + d % 4
            frag[torch.from_numpy(off)] = rows[0, hh, row]
    assert torch.equal(st.acc_rows(frag.view(B, H, N, D)), rows)


def test_expand_coords_to_reference_layout():
    lib = _hip.lib()
    N, bs, step = 3 * 2048, 128, 16
    per_head = lib.aa_coords_entries_per_head(N, bs, step)
    coords = torch.full((1, 1, per_head), -7, dtype=torch.int32)
    counts = torch.tensor([0, 3, 2], dtype=torch.int32).view(1, 1, 3, 1)
    coords[0, 0, 0:3] = torch.tensor([130, 500, 1900])
    off2 = lib.aa_coords_offset(2, bs, step)
    coords[0, 0, off2:off2 + 2] = torch.tensor([128, 3967])
    tc = st.expand_coords(coords, counts, N, bs, step)
    assert tc.shape == (1, 1, 3, N)
    assert tc[0, 0, 1, :4].tolist() == [130, 500, 1900, 0] and tc[0, 0, 2, :3].tolist() == [128, 3967, 0]
    assert int(tc[0, 0, 0].abs().sum()) == 0 and int((tc < 0).sum()) == 0


def test_synthetic_generator_properties():
    q, k, v, pos = make_qkv(4096, 4, 2, n_stripes=64, seed=9)
    assert q.shape == (1, 4, 4096, 128) and k.shape == (1, 2, 4096, 128) and q.dtype == torch.bfloat16
    assert pos.numel() == 64 and pos.min() >= 1 and pos.unique().numel() == 64
    q2, k2, _, pos2 = make_qkv(4096, 4, 2, n_stripes=64, seed=9)
    assert torch.equal(q, q2) and torch.equal(k, k2) and torch.equal(pos, pos2)
    # sink and stripes score far above ordinary keys (shared qbar): ~16 and ~8 nats
    s = (q[0, 0].float() @ k[0, 0].float().T) / math.sqrt(128)
    ordinary = torch.ones(4096, dtype=torch.bool)
    ordinary[0] = False
    ordinary[pos] = False
    assert 14 < float(s[:, 0].mean() - s[:, ordinary].mean()) < 18
    assert 6.5 < float(s[:, pos].mean() - s[:, ordinary].mean()) < 9.5
    # literal mode: biases vanish
    ql, kl, _, _ = make_qkv(4096, 4, 2, n_stripes=64, seed=9, qbar_mode="literal")
    sl = (ql[0, 0].float() @ kl[0, 0].float().T) / math.sqrt(128)
    assert abs(float(sl[:, 0].mean())) < 0.5
    # RoPE is a rotation: norms are preserved, position 0 is untouched
    x = torch.randn(64, 128)
    y = rope_rotate_half(x, 5e5)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), atol=1e-4) and torch.equal(y[0], x[0])
    # relative-position property: <rope(a)_m, rope(b)_n> depends on m - n only
    a, b = torch.randn(128), torch.randn(128)
    ra, rb = rope_rotate_half(a.expand(16, 128).clone(), 1e4), rope_rotate_half(b.expand(16, 128).clone(), 1e4)
    assert abs(float(ra[5] @ rb[3]) - float(ra[12] @ rb[10])) < 1e-3
    g = torch.Generator().manual_seed(1)
    pw = stripe_positions(131072, 655, "powerlaw", g)
    assert pw.numel() == 655 and pw.unique().numel() == 655 and pw.min() >= 1 and pw.max() < 131072
    assert (pw < 131072 // 4).sum() > 655 * 0.4  # density decays with position (uniform would give 25%)


def test_analysis_tools_on_cpu():
    """get_deff metrics and the token-level ideal (plain torch, no kernel involved)."""
    import torch
    from anchor_attn.src.ops.sparse_attn_with_pytorch import sparse_attn_with_torch
    from my_utils.ops_util import get_deff
    x = torch.tensor([1.0, -2.0, 0.0, 4.0])
    y = torch.tensor([1.0005, -2.5, 0.00005, 10.0])
    mean_err, strict, loose, m = get_deff(x, y, verbose=False)
    assert abs(float(mean_err) - (0.0005 + 0.5 + 0.00005 + 6.0) / 4) < 1e-6
    assert strict == 0.5 and loose == 0.75  # -2.5 is within 30% of -2; 10 is not within 30% of 4
    assert m["abs_error_ratios"]["<= 0.1"] == 0.5 and 0 < m["cosine_similarity"] < 1
    with pytest.raises(ValueError):
        get_deff(x, y[:2])
    # theta large: the ideal keeps every causal key and equals dense attention; GQA heads are expanded
    torch.manual_seed(0)
    q, k, v = torch.randn(1, 4, 70, 16), torch.randn(1, 2, 70, 16), torch.randn(1, 2, 70, 16)
    out, ratio = sparse_attn_with_torch(q, k, v, diff_anchor=1e4, return_computational_ratio=True, chunk_size=32)
    ref = torch.nn.functional.scaled_dot_product_attention(q, k.repeat_interleave(2, 1), v.repeat_interleave(2, 1), is_causal=True)
    assert ratio == 1.0 and torch.allclose(out, ref, atol=1e-5)
    # theta = 0 keeps only each row's maximum: output is the value row of the arg-max key
    out0, r0 = sparse_attn_with_torch(q, k, v, diff_anchor=0.0, return_computational_ratio=True)
    s = (q @ k.repeat_interleave(2, 1).transpose(-1, -2)).masked_fill(torch.triu(torch.ones(70, 70, dtype=torch.bool), 1), float("-inf"))
    want = torch.gather(v.repeat_interleave(2, 1), 2, s.argmax(-1, keepdim=True).expand(-1, -1, -1, 16))
    assert torch.allclose(out0, want, atol=1e-5) and abs(r0 - 70 / (70 * 71 / 2)) < 1e-9


def test_recall_bookkeeping_on_cpu():
    """recall@t = fraction of elements with |out - ref| < t (strict), reported next to the sparsity ratio
    (counterpart of the reference's ops_profile_v2.py:514-532)."""
    from anchor_attn.src.ops.ops_profile_v2 import RECALL_THRESHOLDS, recall_ratio, record_recall_ratios
    ref = torch.zeros(2, 5)
    out = torch.tensor([[0.0, 0.004, 0.005, 0.0099, 0.01], [0.02, -0.004, -0.0051, 1.0, -0.0]])
    assert recall_ratio(out, ref, 0.01) == 7 / 10     # 0.01 and 0.02 and 1.0 are not below 0.01
    assert recall_ratio(out, ref, 0.005) == 4 / 10    # 0, 0.004, -0.004, -0 only (0.005 itself is not below)
    assert recall_ratio(out.to(torch.bfloat16), ref, 1e9) == 1.0 and recall_ratio(out, ref, 0.0) == 0.0
    row = record_recall_ratios(out, ref, torch.tensor(0.25))
    assert RECALL_THRESHOLDS == (0.01, 0.005)
    assert row == {"sparsity_ratio": 0.25, "recall@0.01": 0.7, "recall@0.005": 0.4}
    assert record_recall_ratios(out, out, 0.5, thresholds=(1e-6,)) == {"sparsity_ratio": 0.5, "recall@1e-06": 1.0}


def test_timing_only_builds_are_refused_as_the_operator(monkeypatch):
    """`make ablations` builds variants of the library that leave part of a kernel out; they report
    aa_version() >= 1000 and the loader does not accept them in place of the product build."""
    import glob
    import os

    from anchor_attn.src.ops import _hip
    libs = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "..", "anchor-attention_amd", "csrc", "_ablations", "*.so")))
    if not libs:
        pytest.skip("timing-only builds not present (make -C anchor-attention_amd/csrc ablations)")
    for path in libs:
        handle = _hip.bind(path)
        assert handle.aa_version() >= 1001
    monkeypatch.setenv("ANCHOR_ATTN_HIP_LIB", libs[0])
    monkeypatch.setattr(_hip, "_lib", None)
    with pytest.raises(_hip.AnchorAttnHipError, match="timing-only"):
        _hip.lib()


def test_bench_cli_contract_without_a_gpu():
    """bench.py measures one GPU: a request for more exits with a message that says so (before anything touches a
    device); the FLOP model it reports is the documented closed form."""
    import subprocess
    import sys
    root = os.path.join(os.path.dirname(__file__), "..")
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)
    sys.path.insert(0, root)
    import bench
    f1, f2, f3 = bench.flops(32, 131072, 855140)
    assert f1 == 32 * (136 + 63 * 392) * 4 * 128 * 128 * 128            # 6.67 TFLOP of window tiles
    assert f2 == 32 * 2 * 16 * 128 * sum(bb * 2048 - 256 for bb in range(1, 64))
    assert f3 == 4 * 128 * 2048 * 855140
    assert abs((f1 + f2 + f3) / 1e12 - 8.10) < 0.01
    assert set(bench.WORKLOADS) == {"config0_llama8b_4k", "config1_llama8b_32k", "config2_llama8b_128k", "config3_qwen7b_64k",
                                    "llama1b_128k_headdim64"}
    assert bench.workload_head_dim("config2_llama8b_128k") == 128 and bench.workload_head_dim("llama1b_128k_headdim64") == 64


def test_get_mask_block_restatement_agrees_with_the_oracle():
    """``get_mask_block`` (the framework-tensor restatement of stage 2 that the reference keeps next to its kernel,
    get_mask_test.py:162-232) against the oracle's stage 2 on the oracle's own anchors: the same candidate range
    [bs, i*S - bs), ascending lists in the reference's buffer layout, zero for big block 0; the two differ only by the
    kernels' rounding points, i.e. by keys within rounding of the threshold."""
    from anchor_attn.src.ops.get_mask_test import get_mask_block
    from oracle import anchor_oracle as ao
    n, bs, step = 3 * 2048, 128, 16
    q, k, v, _ = make_qkv(n, 2, 1, n_stripes=96, seed=5)
    res = ao.anchor_attn_reference(q.float().numpy(), k.float().numpy(), v.float().numpy(), difference=12.0)
    sm = 128 ** -0.5
    coords, counts, ratio = get_mask_block(q.float(), k.repeat_interleave(2, 1).float(), torch.from_numpy(res.M), bs, bs, step,
                                           12.0 * ao.LOG2E, 1, 2, n, 128, sm * ao.LOG2E, "cpu", True)
    assert coords.shape == (1, 2, 3, n) and coords.dtype == torch.int32 and counts.shape == (1, 2, 3, 1)
    assert int(counts[0, :, 0].sum()) == 0
    total = 0
    for h in range(2):
        for bb in range(3):
            c = int(counts[0, h, bb, 0])
            got = coords[0, h, bb, :c].numpy()
            assert np.all(np.diff(got) > 0) and (c == 0 or (got[0] >= bs and got[-1] < bb * bs * step - bs))
            assert int(coords[0, h, bb, c:].abs().sum()) == 0
            assert len(set(got.tolist()) ^ set(res.coords[0][h][bb].tolist())) <= 2
            total += c
    assert total > 0 and abs(ratio - total / (2 * ((2048 - 256) + (4096 - 256)))) < 1e-12

"""Probe of the Triton toolchain's type-promotion rule that decides the arithmetic of the operator's query
pre-scaling (own micro-kernels; nothing of the reference is imported or run).

The reference's stage-1 kernel takes ``sm_scale`` as ``tl.constexpr`` and evaluates
``(q * sm_scale * 1.44269504).to(dtype)`` on a bf16 tile (anchor_step_1_2_v2.py:19,115-116); its stage-3 kernel
evaluates the same expression with ``sm_scale`` as a run-time float argument (anchor_attn_v4.py:9,66).  This script
runs both forms on every finite bf16 value, and the element-wise part of the stage-2 selection test
(get_mask_test.py:86,96-101) on 65536 near-threshold cases, and the pooling lines (get_mask_test.py:75-84) on
eight big blocks - each once for bf16 tensors and once for fp16 tensors (keys prefixed ``h_``) - and writes the
results to an ``.npz``:

    python tests/triton_promotion_probe.py OUT.npz [cpu|cuda]

With ``TRITON_INTERPRET=1`` in the environment the kernels run in Triton's CPU interpreter; on ``cuda`` they are
compiled for the GPU.
"""
import sys

import numpy as np
import torch
import triton
import triton.language as tl


@triton.jit
def _scale_constexpr(x_ptr, out_ptr, sm_scale: tl.constexpr, BLOCK: tl.constexpr):
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    q = tl.load(x_ptr + offs)
    q = (q * sm_scale * 1.44269504).to(x_ptr.dtype.element_ty)
    tl.store(out_ptr + offs, q.to(tl.float32))


@triton.jit
def _scale_runtime(x_ptr, out_ptr, sm_scale, BLOCK: tl.constexpr):
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    q = tl.load(x_ptr + offs)
    q = (q * sm_scale * 1.44269504).to(x_ptr.dtype.element_ty)
    tl.store(out_ptr + offs, q.to(tl.float32))


@triton.jit
def _stage2_decision(s_ptr, a_ptr, qk_ptr, hit_ptr, diff, qk_scale: tl.constexpr, dtype: tl.constexpr, BLOCK: tl.constexpr):
    # the element-wise part of the reference's stage-2 test (get_mask_test.py:86,96-101) with the float32 dot
    # product supplied as an input: constexpr qk_scale re-bound inside the kernel, run-time diff, bf16 anchors
    offs = tl.program_id(0) * BLOCK + tl.arange(0, BLOCK)
    dot = tl.load(s_ptr + offs)
    anchors = tl.load(a_ptr + offs)
    qk_scale = qk_scale * 1.44269504
    qk = dot * qk_scale
    qk = qk.to(dtype)
    cur_mask = ((qk + diff) >= anchors).to(tl.int32)
    tl.store(qk_ptr + offs, qk.to(tl.float32))
    tl.store(hit_ptr + offs, cur_mask)


@triton.jit
def _pool(q_ptr, m_ptr, qbar_ptr, abar_ptr, step: tl.constexpr, BLOCK_SZ: tl.constexpr, D: tl.constexpr, dtype: tl.constexpr):
    # the pooling of one big block as the reference writes it (get_mask_test.py:75-84)
    rows = tl.arange(0, step * BLOCK_SZ)
    q = tl.load(q_ptr + rows[:, None] * D + tl.arange(0, D)[None, :])
    q = tl.reshape(q, (step, BLOCK_SZ, D))
    q = tl.sum(q, axis=1, keep_dims=False) / BLOCK_SZ
    q = q.to(dtype)
    tl.store(qbar_ptr + tl.arange(0, step)[:, None] * D + tl.arange(0, D)[None, :], q.to(tl.float32))
    anchors = tl.load(m_ptr + rows[:, None] + tl.arange(0, 1)[None, :])
    anchors = tl.reshape(anchors, (step, BLOCK_SZ, 1))
    anchors = tl.sum(anchors, axis=1, keep_dims=False) / BLOCK_SZ
    anchors = anchors.to(dtype)
    tl.store(abar_ptr + tl.arange(0, step)[:, None] + tl.arange(0, 1)[None, :], anchors.to(tl.float32))


def stage2_cases(device, sm_scale, theta, dtype=torch.bfloat16):
    """65536 (dot, anchor) pairs whose scaled score lies within a few steps of the 16-bit type of the decision boundary."""
    g = torch.Generator().manual_seed(4)
    anchors = (torch.rand(4096, generator=g) * 38 + 2).to(dtype)
    target = anchors.float() - theta * 1.44269504                       # scaled score at the boundary
    step = torch.clamp(target.abs(), min=1e-3) * (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11)  # about one step there
    delta = torch.linspace(-2.5, 2.5, 16)[None, :] * step[:, None]
    dot = ((target[:, None] + delta) / (sm_scale * 1.44269504)).float().reshape(-1)
    return dot.to(device), anchors[:, None].expand(4096, 16).reshape(-1).contiguous().to(device)


def all_finite_bf16(device):
    bits = torch.arange(0, 1 << 16, dtype=torch.int32)
    x = (bits << 16).view(torch.float32)
    x = x[torch.isfinite(x)]
    pad = (-x.numel()) % 256
    x = torch.cat([x, torch.zeros(pad)])
    return x.to(torch.bfloat16).to(device)


def all_finite_fp16(device):
    x = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16).view(torch.float16)
    x = x[torch.isfinite(x)]
    pad = (-x.numel()) % 256
    return torch.cat([x, torch.zeros(pad, dtype=torch.float16)]).to(device)


def main(out_path, device):
    x = all_finite_bf16(device)
    res = {"x": x.float().cpu().numpy()}
    for name, sm in (("d128", 128 ** -0.5), ("d64", 0.125), ("odd", 0.1)):
        a = torch.empty(x.numel(), dtype=torch.float32, device=device)
        b = torch.empty_like(a)
        grid = (x.numel() // 256,)
        _scale_constexpr[grid](x, a, sm, 256)
        _scale_runtime[grid](x, b, sm, 256)
        res[f"constexpr_{name}"] = a.cpu().numpy()
        res[f"runtime_{name}"] = b.cpu().numpy()
        res[f"sm_{name}"] = np.float64(sm)
    sm, theta = 128 ** -0.5, 12.0
    dot, anchors = stage2_cases(device, sm, theta)
    qk = torch.empty(dot.numel(), dtype=torch.float32, device=device)
    hit = torch.empty(dot.numel(), dtype=torch.int32, device=device)
    _stage2_decision[(dot.numel() // 256,)](dot, anchors, qk, hit, theta * 1.44269504, sm, tl.bfloat16, 256)
    res.update(s2_dot=dot.cpu().numpy(), s2_anchor=anchors.float().cpu().numpy(), s2_qk=qk.cpu().numpy(),
               s2_hit=hit.cpu().numpy().astype(np.uint8), s2_sm=np.float64(sm), s2_theta=np.float64(theta))
    # pooling of eight big blocks of synthetic queries (a shared component plus N(0,1)) and anchors
    g = torch.Generator().manual_seed(9)
    pq = (torch.randn(8, 2048, 128, generator=g) + torch.randn(128, generator=g) * 0.6).to(torch.bfloat16).to(device)
    pm = (torch.randn(8, 2048, generator=g) * 1.5 + 20).to(device)
    qbar = torch.empty(8, 16, 128, dtype=torch.float32, device=device)
    abar = torch.empty(8, 16, dtype=torch.float32, device=device)
    for i in range(8):
        _pool[(1,)](pq[i], pm[i], qbar[i], abar[i], 16, 128, 128, tl.bfloat16)
    res.update(pool_q=pq.float().cpu().numpy(), pool_m=pm.cpu().numpy(), pool_qbar=qbar.cpu().numpy(), pool_abar=abar.cpu().numpy())
    # ---- the same three probes on fp16 tensors (keys prefixed h_): the reference selects dtype = tl.float16 for them
    hx = all_finite_fp16(device)
    res["h_x"] = hx.float().cpu().numpy()
    for name, sm in (("d128", 128 ** -0.5), ("d64", 0.125), ("odd", 0.1)):
        a = torch.empty(hx.numel(), dtype=torch.float32, device=device)
        b = torch.empty_like(a)
        grid = (hx.numel() // 256,)
        _scale_constexpr[grid](hx, a, sm, 256)
        _scale_runtime[grid](hx, b, sm, 256)
        res[f"h_constexpr_{name}"] = a.cpu().numpy()
        res[f"h_runtime_{name}"] = b.cpu().numpy()
    sm, theta = 128 ** -0.5, 12.0
    dot, anchors = stage2_cases(device, sm, theta, torch.float16)
    qk = torch.empty(dot.numel(), dtype=torch.float32, device=device)
    hit = torch.empty(dot.numel(), dtype=torch.int32, device=device)
    _stage2_decision[(dot.numel() // 256,)](dot, anchors, qk, hit, theta * 1.44269504, sm, tl.float16, 256)
    res.update(h_s2_dot=dot.cpu().numpy(), h_s2_anchor=anchors.float().cpu().numpy(), h_s2_qk=qk.cpu().numpy(),
               h_s2_hit=hit.cpu().numpy().astype(np.uint8))
    hq = pq.to(torch.float16)
    hqbar = torch.empty_like(qbar)
    habar = torch.empty_like(abar)
    for i in range(8):
        _pool[(1,)](hq[i], pm[i], hqbar[i], habar[i], 16, 128, 128, tl.float16)
    res.update(h_pool_q=hq.float().cpu().numpy(), h_pool_qbar=hqbar.cpu().numpy(), h_pool_abar=habar.cpu().numpy())
    np.savez_compressed(out_path, **res)


if __name__ == "__main__":
    main(sys.argv[1], sys.argv[2] if len(sys.argv) > 2 else "cpu")

#!/usr/bin/env python3
"""Benchmark of the AnchorAttention prefill operator on one MI355X.

A step is one full operator call (stage 1 -> pooling -> stage 2 -> stage 3) for one attention layer
on seeded synthetic q/k/v already resident in HBM.  The default workload is the headline one:
Llama-3.1-8B layer shape (32 q heads / 8 KV heads, head_dim 128) at 131072 tokens, theta 12.
Prints ONE JSON line.  `value` is effective TFLOP/s = (F1 + F2 + F3) / time with
  F1 = Hq * T1 * 4*128*128*D,  T1 = 136 + (nBB-1)*392 useful 128x128 tiles of the anchor window pass,
  F2 = Hq * 2*16*D * sum_bb max(bb*S - 256, 0)   (pooled-query x candidate-key scores),
  F3 = 4*D*S * sum(counts)                        (selected keys x the 2048 queries of a big block).
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "anchor-attention_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 FETCH_SIZE/WRITE_SIZE; a counter run cannot be made from inside
# this script, so the figure is carried here for the workload it was taken on, with the file it was copied from
TRAFFIC_SOURCE = "profiles/hbm_traffic_config2_llama8b_128k.md"
MEASURED_TRAFFIC_BYTES = {
    "config2_llama8b_128k": {0: 3.84e9, 3: 4.51e9},  # dominant-kernel index -> bytes (stage 1 as bench.py times it: without pooling; stage 3)
}

WORKLOADS = {
    # name: (n_ctx, hq, hkv, rope_base, n_stripes, stripe_dist[, head_dim = 128])
    "config0_llama8b_4k": (4096, 32, 8, 5e5, 64, "uniform"),
    "config1_llama8b_32k": (32768, 32, 8, 5e5, 512, "uniform"),
    "config2_llama8b_128k": (131072, 32, 8, 5e5, 655, "powerlaw"),
    "config3_qwen7b_64k": (65536, 28, 4, 1e6, 328, "uniform"),
    # not a BASELINE configuration: the Llama-3.2-1B layer shape, for the kernels' head-dimension-64 instantiation
    "llama1b_128k_headdim64": (131072, 32, 8, 5e5, 655, "powerlaw", 64),
}


def workload_head_dim(name):
    w = WORKLOADS[name]
    return w[6] if len(w) > 6 else 128


def flops(hq, n_ctx, sum_counts, D=128, S=2048):
    n_bb = n_ctx // S
    t1 = 136 + (n_bb - 1) * 392
    f1 = hq * t1 * 4 * 128 * 128 * D
    f2 = hq * 2 * 16 * D * sum(max(bb * S - 256, 0) for bb in range(n_bb))
    f3 = 4 * D * S * sum_counts
    return f1, f2, f3


def make_inputs(name, seed, qbar_mode, device):
    """Same construction as anchor_attn.synthetic.make_qkv, but drawn on the GPU (a 128k-token layer
    is 0.5 G random numbers per tensor); stripe positions still come from the CPU generator."""
    import torch
    from anchor_attn.synthetic import stripe_positions
    n_ctx, hq, hkv, base, n_stripes, dist = WORKLOADS[name][:6]
    D = workload_head_dim(name)
    g = torch.Generator(device=device).manual_seed(seed)
    cg = torch.Generator(device="cpu").manual_seed(seed)
    inv = 1.0 / (base ** (torch.arange(0, D, 2, dtype=torch.float64, device=device) / D))
    ang = torch.arange(n_ctx, dtype=torch.float64, device=device)[:, None] * inv[None, :]
    cos = torch.cat([ang.cos(), ang.cos()], -1).float()
    sin = torch.cat([ang.sin(), ang.sin()], -1).float()
    del ang

    def rope(x):
        x1, x2 = x[..., : D // 2], x[..., D // 2:]
        return x * cos + torch.cat([-x2, x1], -1) * sin

    group = hq // hkv
    pos = stripe_positions(n_ctx, n_stripes, dist, cg).to(device)
    u = torch.randn(hkv, D, generator=cg).to(device)
    qbar = u / u.norm(dim=-1, keepdim=True) * math.sqrt(16.0 / (4.0 / math.sqrt(D)))
    q = torch.empty(1, hq, n_ctx, D, dtype=torch.bfloat16, device=device)
    k = torch.empty(1, hkv, n_ctx, D, dtype=torch.bfloat16, device=device)
    v = torch.randn(1, hkv, n_ctx, D, generator=g, device=device).to(torch.bfloat16)
    qsum = torch.zeros(hkv, D, device=device)
    kf = []
    for h in range(hkv):
        kf.append(rope(torch.randn(n_ctx, D, generator=g, device=device)))
    for h in range(hq):
        x = rope(torch.randn(n_ctx, D, generator=g, device=device))
        if qbar_mode == "shared":
            x = x + qbar[h // group]
        else:
            qsum[h // group] += x.mean(0) / group
        q[0, h] = x.to(torch.bfloat16)
    if qbar_mode != "shared":
        qbar = qsum
    for h in range(hkv):
        x = kf[h]
        x[0] += 4.0 * qbar[h]
        x[pos] += 2.0 * qbar[h]
        k[0, h] = x.to(torch.bfloat16)
    return q, k, v


def cpu_baseline():
    """The CPU oracle (our numpy restatement of the reference algorithm - the reference has no CPU
    path of its own) timed on this host on a bounded sample of the workload: one layer of the same head
    configuration at N=16384 (10-30 s of CPU work; the full 128k layer would take tens of minutes)."""
    import numpy as np
    from anchor_attn.synthetic import make_qkv
    from oracle import anchor_oracle as ao
    n_ctx, hq, hkv = 16384, 32, 8
    q, k, v, _ = make_qkv(n_ctx, hq, hkv, n_stripes=256, seed=0)
    Q, K, V = (t.float().numpy() for t in (q, k, v))
    t0 = time.time()
    res = ao.anchor_attn_reference(Q, K, V, difference=12.0)
    dt = time.time() - t0
    f1, f2, f3 = flops(hq, n_ctx, int(res.counts.sum()))
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return {
        "value": (f1 + f2 + f3) / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"numpy oracle, one layer at N={n_ctx}, {hq}q/{hkv}kv heads, theta=12, {dt * 1e3:.0f} ms "
                  f"(BLAS threads={cores})",
        "ms": dt * 1e3,
    }


def gemm_reference(dev):
    """What the vendor GEMM library sustains on this box for bf16 with N(0,1) operands: the published MFMA peak
    assumes the maximum clock, while a matrix-core-bound kernel on real data runs power-limited well below it
    (all-zero operands run ~1.4x faster than random ones).  Two sizes are timed (the larger one runs faster) and the
    better rate is the reference that `roofline.frac_of_gemm_reference` is taken against.  For context only."""
    import torch
    cases = []
    for n, reps in ((8192, 20), (16384, 6)):
        g = torch.Generator(device=dev).manual_seed(1)
        a = torch.randn(n, n, generator=g, device=dev).to(torch.bfloat16)
        b = torch.randn(n, n, generator=g, device=dev).to(torch.bfloat16)
        for _ in range(3):
            c = a @ b
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            c = a @ b
        e1.record()
        torch.cuda.synchronize()
        del a, b, c
        ms = e0.elapsed_time(e1) / reps
        cases.append({"n": n, "ms": ms, "tflops": 2 * n ** 3 / ms / 1e9})
    best = max(cases, key=lambda c: c["tflops"])
    return {"kind": f"torch.matmul bf16 {best['n']}^3, N(0,1) operands (hipBLASLt); the better of 8192^3 and 16384^3",
            "ms": best["ms"], "tflops": best["tflops"], "cases": cases}


def staged_pass(q, k, v, theta, steps, out):
    """The operator's kernels launched stage by stage through their own entry points, with events between them on the
    launch stream.  Returns the mean milliseconds of (stage 1, stand-alone pooling, stage 2, stage 3) and sum(counts)."""
    import torch
    from anchor_attn.src.ops import _hip, anchor_attn_v4 as v4, anchor_step_1_2_v2 as st
    _, hq, n_ctx, D = q.shape
    hkv = k.shape[1]
    BS, STEP, S = 128, 16, 2048
    sm = 1.0 / math.sqrt(D)
    dev = q.device
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(steps)]
    theta2 = theta * v4.LOG2E
    counts = None
    lib = _hip.lib()
    for i in range(steps):
        ev[i][0].record()
        L, M, Acc = st.anchor_attn_step_1(q, k, v, 1, 1, BS, STEP, 1, hq, n_ctx, D, sm)
        ev[i][1].record()
        qbar, abar = st.pool_q_anchor(q, M, BS)
        ev[i][2].record()
        if counts is None:
            mask = torch.empty((lib.aa_mask_words(1, hq, n_ctx, BS, STEP),), dtype=torch.int32, device=dev)
            coords = torch.empty((1, hq, lib.aa_coords_entries_per_head(n_ctx, BS, STEP)), dtype=torch.int32, device=dev)
            counts = torch.empty((1, hq, n_ctx // S, 1), dtype=torch.int32, device=dev)
        _hip.check(lib.aa_stage2_select(qbar.data_ptr(), abar.data_ptr(), *_hip.t3(k), mask.data_ptr(), coords.data_ptr(),
                                        counts.data_ptr(), 1, hq, hkv, n_ctx, D, BS, STEP, sm, theta2, _hip.AA_GEOMETRY_AS_RUN,
                                        _hip.dtype_code(q), torch.cuda.current_stream().cuda_stream))
        ev[i][3].record()
        v4._stage3(q, k, v, coords, counts, L, M, Acc, sm, BS, STEP, out=out)
        ev[i][4].record()
        del L, M, Acc
    torch.cuda.synchronize()
    st_ms = [sum(ev[i][j].elapsed_time(ev[i][j + 1]) for i in range(steps)) / steps for j in range(4)]
    return st_ms, int(counts.sum())


def stage1_on_zero_operands(dev, name, dtype):
    """Stage 1 of the workload's shape on all-zero q, k, v: the same instruction stream (the kernel's control flow does not
    depend on the data), but operands that do not toggle, so the power management lets the chip hold its nominal clock.
    What this leg reports is therefore the kernel's efficiency per cycle; the headline figures are what the same kernel
    gets at the clock the chip grants for real data.  The vendor GEMM is timed on all-zero operands next to it."""
    import torch
    from anchor_attn.src.ops import anchor_step_1_2_v2 as st
    n_ctx, hq, hkv = WORKLOADS[name][0], WORKLOADS[name][1], WORKLOADS[name][2]
    D = workload_head_dim(name)
    tdt = torch.float16 if dtype == "fp16" else torch.bfloat16
    q = torch.zeros((1, hq, n_ctx, D), dtype=tdt, device=dev)
    k = torch.zeros((1, hkv, n_ctx, D), dtype=tdt, device=dev)
    v = torch.zeros((1, hkv, n_ctx, D), dtype=tdt, device=dev)
    sm = 1.0 / math.sqrt(D)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    for i in range(8):
        if i == 3:
            ev[0].record()
        L, M, Acc = st.anchor_attn_step_1(q, k, v, 1, 1, 128, 16, 1, hq, n_ctx, D, sm)
        del L, M, Acc
    ev[1].record()
    torch.cuda.synchronize()
    ms = ev[0].elapsed_time(ev[1]) / 5
    f1 = flops(hq, n_ctx, 0, D=D)[0]
    del q, k, v
    n = 16384
    a = torch.zeros((n, n), dtype=torch.bfloat16, device=dev)
    b = torch.zeros((n, n), dtype=torch.bfloat16, device=dev)
    c = torch.empty((n, n), dtype=torch.bfloat16, device=dev)
    for i in range(8):
        if i == 3:
            ev[0].record()
        torch.matmul(a, b, out=c)
    ev[1].record()
    torch.cuda.synchronize()
    gemm_tflops = 2.0 * n ** 3 / (ev[0].elapsed_time(ev[1]) / 5) / 1e9
    tflops = f1 / ms / 1e9
    return {"ms": ms, "tflops": tflops, "frac_of_mfma_peak": tflops / PEAK_BF16_TFLOPS,
            "gemm_16384_on_zero_operands_tflops": gemm_tflops, "frac_of_that_gemm": tflops / gemm_tflops}


def stage3_dense_regime(dev, seed, dtype):
    """Stage 3 where it is bound by the matrix pipe: the 32k-token Llama shape with the literal reading of the generator
    (no shared query component), under which nearly every candidate key passes the difference test (ratio ~0.92), so the
    sparse kernel does almost the work of dense attention.  Timed by events around the stage-3 launch, after two
    untimed passes."""
    import torch
    name = "config1_llama8b_32k"
    q, k, v = make_inputs(name, seed, "literal", dev)
    if dtype == "fp16":
        q, k, v = q.to(torch.float16), k.to(torch.float16), v.to(torch.float16)
    out = torch.empty_like(q)
    staged_pass(q, k, v, 12.0, 2, out)
    st_ms, sum_counts = staged_pass(q, k, v, 12.0, 5, out)
    n_ctx, hq = WORKLOADS[name][0], WORKLOADS[name][1]
    f3 = flops(hq, n_ctx, sum_counts)[2]
    tflops = f3 / st_ms[3] / 1e9
    return {"workload": name + ", qbar_mode literal, theta 12", "ms": st_ms[3], "tflops": tflops,
            "frac_of_mfma_peak": tflops / PEAK_BF16_TFLOPS,
            "sparsity_ratio": sum_counts / ((hq * n_ctx * n_ctx / 2048) // 2), "F3": f3}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=10,
                    help="untimed calls before the timed ones (the first ~10 calls on an idle GPU run up to 25 %% slower "
                         "while its clocks ramp up)")
    ap.add_argument("--workload", default="config2_llama8b_128k", choices=sorted(WORKLOADS))
    ap.add_argument("--theta", type=float, default=12.0)
    ap.add_argument("--qbar-mode", default="shared", choices=["shared", "literal"])
    ap.add_argument("--seed", type=int, default=2024)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16"], help="element type of q, k, v and the output")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm-ref", action="store_true",
                    help="skip the library bf16 GEMM that is timed after the run as the practical MFMA rate of this box")
    ap.add_argument("--no-dense-regime", action="store_true",
                    help="skip the extra leg that times stage 3 where it is bound by the matrix pipe (32k tokens, "
                         "nearly every key selected)")
    ap.add_argument("--no-zero-operands", action="store_true",
                    help="skip the extra leg that times stage 1 (and the vendor GEMM) on all-zero operands, i.e. at the "
                         "nominal clock: the kernel's efficiency per cycle")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 1 GiB device copies (a kernel of known traffic) so that rocprofv3 "
                         "FETCH_SIZE/WRITE_SIZE readings of the attention kernels can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the operator is embarrassingly parallel over KV-head "
                 "groups, which would shard across GPUs with no exchange) - run with --gpus 1")

    import torch
    from anchor_attn.src.ops import _hip, anchor_attn_v4 as v4
    _hip.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    n_ctx, hq, hkv = WORKLOADS[args.workload][:3]
    D, BS, STEP, S = workload_head_dim(args.workload), 128, 16, 2048
    q, k, v = make_inputs(args.workload, args.seed, args.qbar_mode, dev)
    if args.dtype == "fp16":
        q, k, v = q.to(torch.float16), k.to(torch.float16), v.to(torch.float16)
    out = torch.empty_like(q)
    if args.calibrate_copy:
        src = torch.ones(2**28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        del src, dst
    torch.cuda.synchronize()

    # ---- timed region: K calls of the public operator -----------------------------------------
    for _ in range(args.warmup):
        v4.anchor_attn(q, k, v, difference=args.theta, return_computational_ratio=False, out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        v4.anchor_attn(q, k, v, difference=args.theta, return_computational_ratio=False, out=out)
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # ---- same kernels, staged, with events between them on the launch stream -------------------
    st_ms, sum_counts = staged_pass(q, k, v, args.theta, args.steps, out)
    f1, f2, f3 = flops(hq, n_ctx, sum_counts, D=D)
    ratio = sum_counts / ((1 * hq * n_ctx * n_ctx / (BS * STEP)) // 2)
    dense_flops = 4 * D * hq * n_ctx * (n_ctx + 1) / 2

    stage_tflops = [f1 / st_ms[0] / 1e9, None, f2 / st_ms[2] / 1e9, f3 / st_ms[3] / 1e9 if f3 else 0.0]
    # the dominant kernel is the one that takes the most time; both flash stages are MFMA-bound
    dom = max((0, 3), key=lambda j: st_ms[j])
    roof = {
        "kernel": "flash_kernel<anchor> (stage 1)" if dom == 0 else "flash_kernel<sparse> (stage 3)",
        "bound": "mfma",
        "achieved": stage_tflops[dom],
        "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s",
        "frac": stage_tflops[dom] / PEAK_BF16_TFLOPS,
        "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload, {}).get(dom) if (args.theta == 12.0 and args.qbar_mode == "shared") else None,
        "kernel_ms": st_ms[dom],
    }
    roof["traffic_source"] = TRAFFIC_SOURCE if roof["traffic"] is not None else None
    # stage 3 at this sparsity is bound by HBM (resume state in, output out), stage 2 and pooling likewise:
    # algorithmic bytes per launch over the event-timed duration
    b_pool = hq * n_ctx * D * 2 + hq * n_ctx * 4 + hq * (n_ctx // BS) * (D + 1) * 2
    b2 = hkv * n_ctx * D * 2 + hq * (n_ctx // BS) * (D * 2 + 2 + 4) + 4 * sum_counts + 4 * hq * (n_ctx // S)
    b3 = sum_counts * 2 * D * 2 + hq * n_ctx * D * 2 * 2 + 4 * sum_counts + hq * n_ctx * (D + 2) * 4
    stage_gbs = {"pool": b_pool / st_ms[1] / 1e6, "stage2": b2 / st_ms[2] / 1e6, "stage3": b3 / st_ms[3] / 1e6}
    rec = {
        "metric": "anchor_attn_prefill_layer_effective_tflops",
        "value": (f1 + f2 + f3) / ms_per_step / 1e9,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {"workload": args.workload, "n_ctx": n_ctx, "n_q_heads": hq, "n_kv_heads": hkv, "head_dim": D,
                   "theta": args.theta, "block_size": BS, "step": STEP, "qbar_mode": args.qbar_mode, "seed": args.seed},
        "sparsity_ratio": ratio,
        "computed_fraction_of_dense": (f1 + f3) / dense_flops,
        "stage_ms": {"stage1_anchor": st_ms[0], "pool": st_ms[1], "stage2_select": st_ms[2], "stage3_sparse": st_ms[3]},
        "stage_tflops": {"stage1": stage_tflops[0], "stage2": stage_tflops[2], "stage3": stage_tflops[3]},
        "stage_hbm_gbs": stage_gbs,
        "stage3_frac_of_hbm_peak": stage_gbs["stage3"] / PEAK_HBM_GBS,
        "flops": {"F1": f1, "F2": f2, "F3": f3, "dense_causal": dense_flops},
        "algorithmic_bytes": {"pool": b_pool, "stage2": b2, "stage3": b3},
        "roofline": roof,
    }
    if not args.no_dense_regime:
        del q, k, v, out
        rec["stage3_dense_regime"] = stage3_dense_regime(dev, args.seed, args.dtype)
    if not args.no_zero_operands:
        rec["stage1_on_zero_operands"] = stage1_on_zero_operands(dev, args.workload, args.dtype)
    if not args.no_gemm_ref:
        rec["mfma_reference"] = gemm_reference(dev)
        roof["frac_of_gemm_reference"] = roof["achieved"] / rec["mfma_reference"]["tflops"]
    if not args.no_cpu_baseline:
        rec["cpu_baseline"] = cpu_baseline()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()

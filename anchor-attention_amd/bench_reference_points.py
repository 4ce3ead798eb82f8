"""What this GPU sustains on plain library kernels: the yardsticks the operator's kernels are judged against.

Published peaks (2.5 PFLOP/s dense bf16, 8 TB/s HBM) are not reached by any kernel on real data; this script
measures, on the box it runs on, what the vendor's own kernels reach, so that a roofline fraction of the
operator's kernels can be read against a practical ceiling as well as against the published one:

  * bf16 GEMMs (hipBLASLt through torch.matmul) on N(0,1) operands and on all-zero operands - the difference
    is the power a matrix pipe draws when its inputs toggle;
  * the framework's dense causal attention and this library's own dense kernel on the same shape;
  * this library's own dense kernel on N(0,1), on all-zero and on half-zero operands: the same instruction stream at
    the clocks the power management grants for each kind of data;
  * streaming element-wise kernels at several read:write mixes (the HBM rates a memory-bound kernel can expect).

    python bench_reference_points.py            # prints one JSON object
"""
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def _time_ms(fn, reps, warm=3):
    import torch
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def main():
    import torch
    import torch.nn.functional as F

    from anchor_attn.src.ops import _hip

    dev = "cuda:0"
    torch.manual_seed(0)
    out = {"device": torch.cuda.get_device_name(0)}

    gemm = {}
    for n in (8192, 16384):
        for kind in ("normal", "zeros"):
            a = torch.randn(n, n, device=dev).to(torch.bfloat16) if kind == "normal" else torch.zeros(n, n, device=dev, dtype=torch.bfloat16)
            b = torch.randn(n, n, device=dev).to(torch.bfloat16) if kind == "normal" else torch.zeros(n, n, device=dev, dtype=torch.bfloat16)
            c = torch.empty(n, n, device=dev, dtype=torch.bfloat16)
            ms = _time_ms(lambda: torch.matmul(a, b, out=c), 20)
            gemm[f"{n}^3 {kind}"] = {"ms": ms, "tflops": 2.0 * n ** 3 / ms / 1e9}
            del a, b, c
    out["gemm_bf16"] = gemm

    # dense causal attention: the framework's library kernel and this library's own, 32/8 heads x 32k x 128
    n_ctx, hq, hkv, d = 32768, 32, 8, 128
    q = torch.randn(1, hq, n_ctx, d, device=dev).to(torch.bfloat16)
    k = torch.randn(1, hkv, n_ctx, d, device=dev).to(torch.bfloat16)
    v = torch.randn(1, hkv, n_ctx, d, device=dev).to(torch.bfloat16)
    flops = 4.0 * hq * d * (n_ctx * (n_ctx + 1) / 2)
    ms = _time_ms(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True), 5, warm=2)
    out["sdpa_causal_32k"] = {"ms": ms, "tflops": flops / ms / 1e9}
    o = torch.empty_like(q)
    lib = _hip.lib()
    stream = torch.cuda.current_stream().cuda_stream

    def own():
        _hip.check(lib.aa_dense_causal_fwd(*_hip.t3(q), *_hip.t3(k), *_hip.t3(v), *_hip.t3(o), 1, hq, hkv, n_ctx, d,
                                           d ** -0.5, _hip.AA_DTYPE_BF16, stream))

    ms = _time_ms(own, 5, warm=2)
    out["own_dense_causal_32k"] = {"ms": ms, "tflops": flops / ms / 1e9}
    # the same kernel, the same number of instructions, other operand data
    by_data = {}
    zq, zk, zv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    for name, (q_, k_, v_) in (("all-zero operands", (zq, zk, zv)), ("N(0,1) q and k, zero v", (q, k, zv)),
                               ("zero q and k, N(0,1) v", (zq, zk, v)), ("N(0,1) operands", (q, k, v))):
        def own_on():
            _hip.check(lib.aa_dense_causal_fwd(*_hip.t3(q_), *_hip.t3(k_), *_hip.t3(v_), *_hip.t3(o), 1, hq, hkv, n_ctx, d,
                                               d ** -0.5, _hip.AA_DTYPE_BF16, stream))
        ms = _time_ms(own_on, 5, warm=2)
        by_data[name] = {"ms": ms, "tflops": flops / ms / 1e9}
    out["own_dense_causal_32k_by_operand_data"] = by_data
    del q, k, v, o, zq, zk, zv

    # streaming kernels on 1 GiB fp32 tensors
    n = 2 ** 28
    a, b, c3 = (torch.randn(n, device=dev) for _ in range(3))
    c = torch.empty(n, device=dev)
    gib = float(2 ** 30)
    hbm = {}
    for name, fn, nbytes in (("fill (0 reads : 1 write)", lambda: c.fill_(1.0), gib),
                             ("copy (1:1)", lambda: c.copy_(a), 2 * gib),
                             ("add (2:1)", lambda: torch.add(a, b, out=c), 3 * gib),
                             ("addcmul (3:1)", lambda: torch.addcmul(a, b, c3, out=c), 4 * gib),
                             ("sum (1:0)", lambda: torch.sum(a), gib)):
        ms = _time_ms(fn, 10)
        hbm[name] = {"ms": ms, "GBps": nbytes / ms / 1e6}
    out["hbm_streaming"] = hbm
    print(json.dumps(out))


if __name__ == "__main__":
    main()

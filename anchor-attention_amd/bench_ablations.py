"""What each ingredient of the stage-1 and stage-3 kernels costs: timing-only builds against the product build.

`make -C anchor-attention_amd/csrc ablations` builds ten variants of the library that each leave one thing out
(AA_ABLATE in csrc/aa_flash.hip).  Their results are wrong on purpose, so they are never loaded as the operator;
this script opens them next to the product build, gives every build the SAME inputs - queries, keys, values, and
for stage 3 the statistics, accumulator state and index lists computed by the product build - and times one entry
point per build with events on the launch stream.  The workload is the headline one (Llama-3.1-8B layer shape,
131072 tokens, theta 12) unless --workload says otherwise.

    make -C anchor-attention_amd/csrc ablations && python anchor-attention_amd/bench_ablations.py

Prints one JSON object and a table.  The product build is timed first and last, so that drift of the box (clocks,
temperature) over the run can be read off the two figures.
"""
import argparse
import glob
import json
import math
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))

STAGE1 = {1: "exp2 of the soft-max replaced by a pass-through",
          2: "no soft-max arithmetic (mask, max, exp, sum); scores converted as they are",
          3: "no K/V tile loads inside the tile loop",
          8: "no work-group barrier at the end of a tile",
          9: "neither the barrier nor the wait for the tile's loads at the end of a tile",
          10: "nothing: the soft-max runs in full, but P.V takes a loop-invariant operand (dependency scores -> P -> P.V cut)"}
STAGE3 = {4: "no tile loop: statistics and accumulator state in, output out (the unused query loads are compiled away)",
          5: "accumulator state not loaded (tile loop kept)",
          6: "at most two tiles per query block",
          7: "no tile loop and no accumulator state: only the output is written (the unused query loads are compiled away)",
          1: "exp2 of the soft-max replaced by a pass-through",
          2: "no soft-max arithmetic",
          3: "no K/V tile loads inside the tile loop",
          8: "no work-group barrier at the end of a tile",
          9: "neither the barrier nor the wait for the tile's loads at the end of a tile",
          10: "nothing: the soft-max runs in full, but P.V takes a loop-invariant operand (dependency cut)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="config2_llama8b_128k")
    ap.add_argument("--theta", type=float, default=12.0)
    ap.add_argument("--seed", type=int, default=2024)
    ap.add_argument("--reps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=5)
    args = ap.parse_args()

    import torch

    import bench
    from anchor_attn.src.ops import _hip
    from anchor_attn.src.ops import anchor_step_1_2_v2 as st

    product = _hip.lib()
    variants = {}
    for path in sorted(glob.glob(os.path.join(HERE, "csrc", "_ablations", "libanchor_attn_hip.ablate*.so"))):
        handle = _hip.bind(path)
        n = handle.aa_version() - 1000
        assert n > 0, f"{path} is not a timing-only build"
        variants[n] = handle
    if not variants:
        sys.exit("no timing-only builds found: run `make -C anchor-attention_amd/csrc ablations` first")

    dev = "cuda:0"
    torch.cuda.set_device(0)
    q, k, v = bench.make_inputs(args.workload, args.seed, "shared", dev)
    B, H, N, D = q.shape
    Hkv = k.shape[1]
    BS, STEP = 128, 16
    sm = 1.0 / math.sqrt(D)
    stream = torch.cuda.current_stream().cuda_stream
    # what stage 3 resumes from, computed once by the product build
    L, M, acc = st.anchor_attn_step_1(q, k, v, 1, 1, BS, STEP, B, H, N, D, sm)
    coords, counts = st.select_stripes_packed(q, k, M, BS, STEP, args.theta * 1.44269504, B, H, N, D, sm)
    out = torch.empty_like(q)
    M2, L2, acc2 = torch.empty_like(M), torch.empty_like(L), torch.empty_like(acc)
    torch.cuda.synchronize()

    def stage1(lib):
        rc = lib.aa_stage1_anchor_fwd(*_hip.t3(q), *_hip.t3(k), *_hip.t3(v), M2.data_ptr(), L2.data_ptr(), acc2.data_ptr(),
                                      B, H, Hkv, N, D, BS, STEP, sm, _hip.AA_SCALE_BF16_CHAIN, _hip.AA_DTYPE_BF16, stream)
        assert rc == 0, lib.aa_last_error()

    def stage3(lib):
        rc = lib.aa_stage3_sparse_fwd(*_hip.t3(q), *_hip.t3(k), *_hip.t3(v), coords.data_ptr(), counts.data_ptr(),
                                      M.data_ptr(), L.data_ptr(), acc.data_ptr(), *_hip.t3(out), B, H, Hkv, N, D, BS, STEP, sm,
                                      _hip.AA_DTYPE_BF16, stream)
        assert rc == 0, lib.aa_last_error()

    def time_ms(fn, lib):
        for _ in range(args.warmup):
            fn(lib)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.reps):
            fn(lib)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.reps

    result = {"workload": args.workload, "theta": args.theta, "reps": args.reps, "stage1": [], "stage3": []}
    for name, fn, table in (("stage1", stage1, STAGE1), ("stage3", stage3, STAGE3)):
        base = time_ms(fn, product)
        result[name].append({"build": "product", "ms": base})
        for n, what in table.items():
            if n in variants:
                ms = time_ms(fn, variants[n])
                result[name].append({"build": f"AA_ABLATE={n}", "what": what, "ms": ms, "vs_product": ms / base - 1.0})
        result[name].append({"build": "product (again)", "ms": time_ms(fn, product)})
    print(json.dumps(result))
    for name in ("stage1", "stage3"):
        print(f"\n| {name}: build | what is left out | ms | vs product |\n|---|---|---|---|", file=sys.stderr)
        for r in result[name]:
            rel = f"{r['vs_product'] * 100:+.1f} %" if "vs_product" in r else ""
            print(f"| {r['build']} | {r.get('what', '')} | {r['ms']:.3f} | {rel} |", file=sys.stderr)


if __name__ == "__main__":
    main()

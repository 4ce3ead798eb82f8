"""End-to-end prefill of a Llama-architecture model whose attention is the AnchorAttention operator.

BASELINE config 4: the 32-layer Llama-3.1-8B architecture (hidden 4096, FFN 14336, 32/8 heads, vocab 128256,
RoPE base 5e5) with random-init bf16 weights and random token ids at N = 131072 on one GPU; reports the
prefill time with the operator and its attention share, and the same model with dense attention twice: on this
package's own MFMA kernel (pattern "dense", the baseline "built on the same kernels") and on the framework's
library attention (pattern "flash").
There is no checkpoint or dataset involved: weights and tokens are synthetic, so the sparsity a trained
model would show is not reproduced - the numbers are timings of the code path, and say so.

Next to the bare forward, each pattern is also timed the way the reference's driver measures "prefill time"
(test_hf.py:24-36): host wall-clock around ``model.generate(input_ids, attention_mask=ones, max_new_tokens=1,
num_beams=1, do_sample=False)``, which includes building the KV cache and the generation loop's bookkeeping.

    python bench_model_prefill.py                       # config 4
    python bench_model_prefill.py --layers 2 --n-ctx 8192   # quick check
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--n-ctx", type=int, default=131072)
    ap.add_argument("--theta", type=float, default=12.0)
    ap.add_argument("--reps", type=int, default=2)
    ap.add_argument("--no-dense", action="store_true", help="skip the dense-attention runs of the same model")
    args = ap.parse_args()

    import torch
    from transformers import LlamaConfig, LlamaForCausalLM

    from anchor_attn import patch_model
    from anchor_attn.src.modules.llama import anchor_attention as plug

    dev = "cuda:0"
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=args.layers, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=128256, max_position_embeddings=args.n_ctx,
                      rope_theta=5e5, tie_word_embeddings=False)
    t0 = time.time()
    with torch.device(dev):
        model = LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    print(f"# model built in {time.time() - t0:.1f} s: {sum(p.numel() for p in model.parameters()) / 1e9:.2f} G parameters", file=sys.stderr, flush=True)
    tokens = torch.randint(0, cfg.vocab_size, (1, args.n_ctx), device=dev)

    # time spent inside the attention plug, by events around every call
    spans = []
    plug.record_ratio = True  # the ratio stays a device tensor; it is read after the prefill has finished

    def timed_plug(inner):
        def timed(*a, **k):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = inner(*a, **k)
            e1.record()
            spans.append((e0, e1, plug.last_ratio if inner is plug.anchor_attention_forward else None))
            return r
        return timed

    def prefill(reps):
        best = None
        for _ in range(reps + 1):  # first pass is the warm-up
            spans.clear()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            with torch.no_grad():
                out = model(tokens, use_cache=False, logits_to_keep=1).logits
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1)
            attn = sum(a.elapsed_time(b) for a, b, _ in spans)
            if best is None or ms < best[0]:
                best = (ms, attn, [float(r) for _, _, r in spans if r is not None], out)
        return best

    def generate_one_token_ms(reps):
        """The reference's prefill metric: wall-clock of generate(max_new_tokens=1) (its return is a host-side token
        tensor, so the call ends synchronised, as in the reference)."""
        ones = torch.ones_like(tokens)
        best = None
        for _ in range(reps + 1):
            torch.cuda.synchronize()
            t = time.time()
            with torch.no_grad():
                seq = model.generate(input_ids=tokens, attention_mask=ones, max_new_tokens=1, num_beams=1, do_sample=False,
                                     pad_token_id=0)
            int(seq[0, -1])  # the token is on the host: the prefill has finished
            ms = (time.time() - t) * 1000.0
            best = ms if best is None else min(best, ms)
        assert seq.shape[1] == args.n_ctx + 1
        return best

    patch_model(model, "anchor_attn", {"theta": args.theta})
    from transformers import AttentionInterface
    AttentionInterface.register(plug.ATTN_NAME, timed_plug(plug.anchor_attention_forward))
    AttentionInterface.register(plug.DENSE_ATTN_NAME, timed_plug(plug.dense_attention_forward))
    ms, attn_ms, ratios, logits = prefill(args.reps)
    res = {"workload": f"llama3.1-8b architecture, {args.layers} layers, random-init bf16, N={args.n_ctx}, theta={args.theta}",
           "prefill_ms_anchor_attn": ms, "attention_ms": attn_ms, "attention_share": attn_ms / ms,
           "mean_sparsity_ratio": sum(ratios) / max(len(ratios), 1), "logits_finite": bool(torch.isfinite(logits).all())}
    res["generate_1_token_ms_anchor_attn"] = generate_one_token_ms(1)
    if not args.no_dense:
        patch_model(model, "dense")
        dms, dattn, _, dlogits = prefill(1)
        res["generate_1_token_ms_dense_own_kernel"] = generate_one_token_ms(1)
        res["prefill_ms_dense_own_kernel"] = dms
        res["attention_ms_dense_own_kernel"] = dattn
        res["speedup_vs_dense_own_kernel"] = dms / ms
        res["attention_speedup_vs_dense_own_kernel"] = dattn / attn_ms
        patch_model(model, "flash")
        fms, _, _, flogits = prefill(1)
        res["prefill_ms_dense_library_sdpa"] = fms
        res["speedup_vs_dense_library_sdpa"] = fms / ms
        res["dense_own_vs_library_max_logit_diff"] = float((dlogits.float() - flogits.float()).abs().max())
    AttentionInterface.register(plug.ATTN_NAME, plug.anchor_attention_forward)
    AttentionInterface.register(plug.DENSE_ATTN_NAME, plug.dense_attention_forward)
    print(json.dumps(res))


if __name__ == "__main__":
    main()

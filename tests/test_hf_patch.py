"""patch_model and the Hugging Face attention plug: host logic on the CPU (dense branches only - the
sparse branch needs the GPU and is covered by the gpu-marked tests below)."""
import types

import pytest
import torch


def _tiny(n_layers=2, head_dim=128, **kw):
    from transformers import LlamaConfig, LlamaForCausalLM
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=4 * head_dim, intermediate_size=1024, num_hidden_layers=n_layers, num_attention_heads=4,
                      num_key_value_heads=2, head_dim=head_dim, vocab_size=1000, max_position_embeddings=16384,
                      rope_theta=5e5, **kw)
    return LlamaForCausalLM(cfg).eval()


def test_patch_model_validation_and_config():
    from anchor_attn import get_config_example, patch_model
    assert get_config_example("anchor_attn") == {"block_size_M": 128, "theta": 12, "step": 16}
    m = _tiny(1)
    before = m.config._attn_implementation
    assert patch_model(m, "default") is m and m.config._attn_implementation == before
    with pytest.raises(ValueError):
        patch_model(m, "streaming_llm")  # competitor patterns are not part of this package
    with pytest.raises(ValueError):
        patch_model(torch.nn.Linear(2, 2), "anchor_attn")
    with pytest.raises(ValueError):
        patch_model(m, "anchor_attn", {"step": 8})
    patch_model(m, "anchor_attn", {"theta": 11})
    assert m.config._attn_implementation == "anchor_attn"
    assert (m.config.block_size_M, m.config.step, m.config.theta) == (128, 16, 11)
    patch_model(m, "flash")
    assert m.config._attn_implementation == "sdpa"
    # the reference's second name for the same forward and the same defaults (patch.py:41-45,142-144)
    assert get_config_example("anchor_attn_lite") == get_config_example("anchor_attn")
    patch_model(m, "anchor_attn_lite", {"theta": 13})
    assert m.config._attn_implementation == "anchor_attn" and m.config.theta == 13
    # dense attention on the package's own kernel
    patch_model(m, "dense")
    assert m.config._attn_implementation == "anchor_attn_dense"
    assert set(get_config_example()) == {"default", "flash", "dense", "anchor_attn", "anchor_attn_lite"}


def test_patch_model_takes_the_json_text_that_test_hf_passes():
    """The reference's driver hands ``--config`` through as the string it was typed as (test_hf.py:110-114,131;
    script/run_longbench_v1.sh:38 passes '{"theta":12,"step":16}'), and patch.py:62-74 parses it, fills the keys left
    out from the pattern's defaults and reports bad JSON as ValueError."""
    from anchor_attn import patch_model
    m = _tiny(1)
    patch_model(m, "anchor_attn", '{"theta":12,"step":16}')
    assert m.config._attn_implementation == "anchor_attn"
    assert (m.config.block_size_M, m.config.step, m.config.theta) == (128, 16, 12)
    patch_model(m, "anchor_attn_lite", '{"block_size_M": 64, "theta": 11.5, "step": 32}')
    assert (m.config.block_size_M, m.config.step, m.config.theta) == (64, 32, 11.5)
    patch_model(m, "anchor_attn", "{}")
    assert (m.config.block_size_M, m.config.step, m.config.theta) == (128, 16, 12)
    patch_model(m, "flash", "{}")
    assert m.config._attn_implementation == "sdpa"
    for bad in ('{"theta":12,', "theta=12", ""):
        with pytest.raises(ValueError, match="not valid JSON"):
            patch_model(m, "anchor_attn", bad)
    for not_a_dict in ("[1, 2]", "12", 12, ["theta"]):
        with pytest.raises(ValueError, match="dict"):
            patch_model(m, "anchor_attn", not_a_dict)
    with pytest.raises(ValueError):
        patch_model(m, "anchor_attn", '{"step": 8}')
    # the caller's dict is not written to
    mine = {"theta": 13}
    patch_model(m, "anchor_attn", mine)
    assert mine == {"theta": 13} and m.config.theta == 13


def test_model_level_patches_last_token_logits_and_chunked_mlp():
    """Every pattern but "default" also patches the model as the reference does (patch.py:146-157): the forward
    returns float32 logits of the last position only (causal_model_forward.py:124-125) and the MLPs run over chunks
    of the sequence (llama_mlp_forward.py:46-58) - neither changes a value."""
    from anchor_attn import patch_model
    from anchor_attn.src.modules import model_forward
    assert model_forward.MLP_CHUNK_TOKENS == 32768
    ref = _tiny()
    x = torch.randint(0, 1000, (2, 300))
    with torch.no_grad():
        full = ref(x).logits
    for pattern in ("flash", "dense", "anchor_attn", "anchor_attn_lite"):
        m = _tiny()
        m.load_state_dict(ref.state_dict())
        patch_model(m, pattern, {"mlp_chunk_tokens": 64})  # 300 positions = four full chunks and a ragged one
        assert all(layer.mlp._mlp_chunk_tokens == 64 for layer in m.model.layers)
        with torch.no_grad():
            last = m(x).logits
            assert last.shape == (2, 1, 1000) and last.dtype == torch.float32
            assert torch.allclose(last, full[:, -1:], atol=1e-5)
            # a caller that names the positions it wants, or passes labels, gets them
            assert torch.allclose(m(x, logits_to_keep=0).logits, full, atol=1e-5)
            assert m(x, logits_to_keep=7).logits.shape == (2, 7, 1000)
            with_loss = m(x, labels=x)
            assert with_loss.logits.shape == (2, 300, 1000)
            assert abs(float(with_loss.loss) - float(ref(x, labels=x).loss)) < 1e-5
            # the chunked MLP is the MLP
            h = torch.randn(2, 300, 512)
            assert torch.allclose(m.model.layers[0].mlp(h), ref.model.layers[0].mlp(h), atol=1e-6)
        # patching again wraps nothing twice and only moves the chunk size
        fwd, mlp_fwd = m.forward, m.model.layers[0].mlp.forward
        patch_model(m, pattern)
        assert m.forward is fwd and m.model.layers[0].mlp.forward is mlp_fwd
        assert m.model.layers[0].mlp._mlp_chunk_tokens == 32768
    # both can be declined
    m = _tiny()
    m.load_state_dict(ref.state_dict())
    patch_model(m, "anchor_attn", {"last_token_logits": False, "mlp_chunk_tokens": 0})
    with torch.no_grad():
        assert m(x).logits.shape == (2, 300, 1000)
    assert not hasattr(m.config, "last_token_logits") and not hasattr(m.config, "mlp_chunk_tokens")


def test_dense_pattern_on_cpu_is_plain_attention():
    """Without a GPU the dense plug has only its framework branch; a model patched with it computes what the
    unpatched model computes (prefill and cached decode)."""
    from anchor_attn import patch_model
    ref = _tiny()
    m = _tiny()
    m.load_state_dict(ref.state_dict())
    patch_model(m, "dense")
    x = torch.randint(0, 1000, (1, 200))
    with torch.no_grad():
        assert torch.allclose(ref(x).logits, m(x, logits_to_keep=0).logits, atol=1e-5)
        assert torch.equal(ref.generate(x, max_new_tokens=3, do_sample=False), m.generate(x, max_new_tokens=3, do_sample=False))


def test_short_prefill_and_decode_take_the_dense_branch():
    """Below one big block, and for single-token decode steps against a cache, the plug is dense attention:
    a patched model generates exactly what the unpatched one does."""
    from anchor_attn import patch_model
    ref = _tiny()
    m = _tiny()
    m.load_state_dict(ref.state_dict())
    patch_model(m, "anchor_attn")
    x = torch.randint(0, 1000, (2, 300))
    with torch.no_grad():
        a = ref(x).logits
        b = m(x, logits_to_keep=0).logits
        assert torch.allclose(a, b, atol=1e-5)
        ga = ref.generate(x, max_new_tokens=4, do_sample=False)
        gb = m.generate(x, max_new_tokens=4, do_sample=False)
    assert torch.equal(ga, gb)


def test_plug_dense_branch_matches_reference_math():
    """Direct call of the plug with a cache-style shape (fewer queries than keys): bottom-right causal."""
    from anchor_attn.src.modules.llama.anchor_attention import anchor_attention_forward
    mod = types.SimpleNamespace(config=types.SimpleNamespace(block_size_M=128, step=16, theta=12.0))
    torch.manual_seed(1)
    q, k, v = torch.randn(1, 4, 5, 128), torch.randn(1, 2, 37, 128), torch.randn(1, 2, 37, 128)
    out, w = anchor_attention_forward(mod, q, k, v, None, scaling=0.1)
    assert w is None and out.shape == (1, 5, 4, 128)
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    s = (q @ kk.transpose(-1, -2)) * 0.1
    rows = torch.arange(5)[:, None] + 32
    s = s.masked_fill(torch.arange(37)[None, :] > rows, float("-inf"))
    want = (s.softmax(-1) @ vv).transpose(1, 2)
    assert torch.allclose(out, want, atol=1e-5)


# ------------------------------------------------------------------------------------ GPU
@pytest.mark.gpu
@pytest.mark.parametrize("n_tokens", [2 * 2048 + 300, 2 * 2048])
def test_plug_sparse_branch_is_the_operator_plus_dense_tail(n_tokens, monkeypatch):
    """The plug on HF-layout (transposed, non-contiguous) tensors = anchor_attn on contiguous copies for the
    rows the operator covers (bit for bit) + dense attention for the tail rows; pad == 0 included."""
    from anchor_attn.src.modules.llama import anchor_attention as aa
    from anchor_attn.src.ops.anchor_attn_v4 import anchor_attn
    from anchor_attn.synthetic import make_qkv
    q, k, v, _ = make_qkv(n_tokens - n_tokens % 128 + 128 if n_tokens % 128 else n_tokens, 4, 2, n_stripes=64, seed=3)
    q, k, v = (t[:, :, :n_tokens].cuda() for t in (q, k, v))
    # what LlamaAttention hands over: [B,H,N,D] views of [B,N,H,D] storage
    qh, kh, vh = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
    mod = types.SimpleNamespace(config=types.SimpleNamespace(block_size_M=128, step=16, theta=12.0))
    aa.last_ratio = None
    plain, _ = aa.anchor_attention_forward(mod, qh, kh, vh, None, scaling=128 ** -0.5)
    assert aa.last_ratio is None  # by default the plug asks for no ratio, as the reference's caller does
    monkeypatch.setattr(aa, "record_ratio", True)
    out, _ = aa.anchor_attention_forward(mod, qh, kh, vh, None, scaling=128 ** -0.5)
    assert torch.equal(out, plain) and aa.last_ratio.is_cuda
    assert out.shape == (1, n_tokens, 4, 128) and out.is_contiguous()
    main = n_tokens - n_tokens % 2048
    want, ratio = anchor_attn(q[:, :, :main].contiguous(), k[:, :, :main].contiguous(), v[:, :, :main].contiguous())
    assert torch.equal(out.transpose(1, 2)[:, :, :main], want)
    assert float(aa.last_ratio) == float(ratio) and float(ratio) > 0
    if n_tokens > main:
        ref = torch.nn.functional.scaled_dot_product_attention(
            q.double(), k.double().repeat_interleave(2, 1), v.double().repeat_interleave(2, 1), is_causal=True)
        err = (out.transpose(1, 2)[:, :, main:].double() - ref[:, :, main:]).abs()
        assert err.max() < 2e-2


@pytest.mark.gpu
@pytest.mark.parametrize("head_dim", [128, 64])
def test_patched_model_equals_dense_model_when_the_window_covers_everything(head_dim):
    """theta -> -inf selects nothing; with two big blocks the stage-1 window [0,S) U [bb*S, r] is the whole causal
    prefix, so a patched model must reproduce the dense (SDPA) model's logits - prefill with a ragged tail.  Both head
    dimensions the kernels are built for (64: the Llama-3.2-1B / Qwen2.5-0.5B class of models)."""
    from anchor_attn import patch_model
    ref = _tiny(head_dim=head_dim).to(torch.bfloat16).cuda()
    m = _tiny(head_dim=head_dim).to(torch.bfloat16).cuda()
    m.load_state_dict(ref.state_dict())
    patch_model(m, "anchor_attn", {"theta": -1e4})
    x = torch.randint(0, 1000, (1, 2 * 2048 + 77), device="cuda")
    with torch.no_grad():
        a = ref(x, logits_to_keep=64).logits.float()
        b = m(x, logits_to_keep=64).logits.float()
    assert torch.isfinite(b).all()
    assert (a - b).abs().max() < 0.08 * a.abs().max()
    assert (a - b).abs().mean() < 0.01 * a.abs().mean() + 1e-3


def _generate_like_test_hf(model, input_ids, max_new_tokens):
    """What the reference's driver does (test_hf.py:24-47): tokenizer output = ids plus an all-ones mask, greedy."""
    with torch.no_grad():
        return model.generate(input_ids=input_ids, attention_mask=torch.ones_like(input_ids), max_new_tokens=max_new_tokens,
                              num_beams=1, do_sample=False, pad_token_id=0, output_scores=True, return_dict_in_generate=True)


@pytest.mark.gpu
def test_generate_with_a_cache_prefills_sparse_and_decodes_dense(monkeypatch):
    """The reference measures prefill as ``generate(max_new_tokens=1)`` and then generates more tokens against the
    cache (test_hf.py:24-47).  Under ``generate`` the plug is handed an all-ones attention mask (which must arrive
    as None) and keys/values that come out of the KV cache.  The prefill call of every layer must take the operator
    (big blocks) plus the dense tail, every decode step the dense branch; with theta -> -inf and two big blocks the
    window is the whole causal prefix, so the scores must be those of the unpatched model and the greedy tokens the
    same wherever the unpatched model's lead over the runner-up exceeds the numerical difference."""
    from anchor_attn import patch_model
    from anchor_attn.src.modules.llama import anchor_attention as plug
    n_prompt, n_new, n_layers = 2 * 2048 + 77, 4, 2
    ref = _tiny().to(torch.bfloat16).cuda()
    m = _tiny().to(torch.bfloat16).cuda()
    m.load_state_dict(ref.state_dict())
    patch_model(m, "anchor_attn", '{"theta": -1e4}')
    x = torch.randint(1, 1000, (1, n_prompt), device="cuda")
    sparse_calls, dense_calls = [], []
    op, dense = plug.anchor_attn, plug._dense

    def op_seen(q, k, v, **kw):
        sparse_calls.append((tuple(q.shape), tuple(k.shape), k.stride(-1), kw["out"].shape[2]))
        return op(q, k, v, **kw)

    def dense_seen(q, k, v, mask, *a):
        dense_calls.append((q.shape[2], k.shape[2], mask is not None))
        return dense(q, k, v, mask, *a)

    monkeypatch.setattr(plug, "anchor_attn", op_seen)
    monkeypatch.setattr(plug, "_dense", dense_seen)
    for new_tokens in (1, n_new):  # the reference's "prefill time" call, then its multi-token call
        sparse_calls.clear(), dense_calls.clear()
        got = _generate_like_test_hf(m, x, new_tokens)
        assert got.sequences.shape == (1, n_prompt + new_tokens)
        # prefill: every layer once through the operator on the two big blocks, K/V with their native heads ...
        assert sparse_calls == [((1, 4, 4096, 128), (1, 2, 4096, 128), 1, 4096)] * n_layers
        # ... then the 77 tail rows densely without a mask, then one dense call per layer and decode step
        want_dense = [(77, n_prompt, False)] * n_layers
        for t in range(1, new_tokens):
            want_dense += [(1, n_prompt + t, False)] * n_layers
        assert sorted(dense_calls) == sorted(want_dense), dense_calls
    monkeypatch.setattr(plug, "anchor_attn", op)
    monkeypatch.setattr(plug, "_dense", dense)
    want = _generate_like_test_hf(ref, x, n_new)
    for t in range(n_new):
        a, b = want.scores[t].float()[0], got.scores[t].float()[0]
        assert torch.isfinite(b).all()
        err = float((a - b).abs().max())
        assert err < 0.08 * float(a.abs().max()), (t, err)
        ta, tb = int(want.sequences[0, n_prompt + t]), int(got.sequences[0, n_prompt + t])
        if ta != tb:  # only a lead smaller than the difference may flip the greedy choice; later steps then differ
            assert float(a[ta] - a[tb]) <= 2 * err, (t, ta, tb, float(a[ta] - a[tb]), err)
            break
    # the default threshold: a real sparse prefill under generate stays finite and decodes
    patch_model(m, "anchor_attn", '{"theta":12,"step":16}')
    monkeypatch.setattr(plug, "record_ratio", True)
    y = torch.randint(1, 1000, (1, 3 * 2048 + 5), device="cuda")
    got = _generate_like_test_hf(m, y, 3)
    assert got.sequences.shape == (1, 3 * 2048 + 8) and all(torch.isfinite(s).all() for s in got.scores)
    assert 0 < float(plug.last_ratio) <= 1.0
    # a left-padded batch is not the case the operator is defined for: it must take the dense branch with its mask
    monkeypatch.setattr(plug, "_dense", dense_seen)
    dense_calls.clear()
    mask = torch.ones(2, 2048 + 64, dtype=torch.long, device="cuda")
    mask[1, :100] = 0
    ids = torch.randint(1, 1000, (2, 2048 + 64), device="cuda") * mask
    with torch.no_grad():
        padded = m.generate(input_ids=ids, attention_mask=mask, max_new_tokens=2, num_beams=1, do_sample=False, pad_token_id=0)
    assert padded.shape == (2, 2048 + 66)
    assert dense_calls and all(has_mask for _, _, has_mask in dense_calls), dense_calls


@pytest.mark.gpu
def test_patched_qwen2_model(monkeypatch):
    """The same plug under Qwen2 (attention biases, its own config class, optional sliding-window layers):
    window-covers-everything equality with the dense model, and a real sparse prefill that stays finite and reports a
    ratio.  A sliding-window layer arrives with a mask that is not purely causal and takes the plug's dense branch."""
    from transformers import Qwen2Config, Qwen2ForCausalLM

    from anchor_attn import patch_model
    import anchor_attn.src.modules.llama.anchor_attention as plug

    def config(**kw):  # a model keeps the config object it is given: one per model, or patching one patches both
        return Qwen2Config(hidden_size=512, intermediate_size=1024, num_hidden_layers=2, num_attention_heads=4,
                           num_key_value_heads=2, vocab_size=1000, max_position_embeddings=16384, rope_theta=1e6, **kw)

    assert config().hidden_size // config().num_attention_heads == 128
    for kw in ({}, {"use_sliding_window": True, "sliding_window": 1024, "max_window_layers": 1}):
        torch.manual_seed(0)
        ref = Qwen2ForCausalLM(config(**kw)).eval().to(torch.bfloat16).cuda()
        m = Qwen2ForCausalLM(config(**kw)).eval().to(torch.bfloat16).cuda()
        assert m.config is not ref.config
        m.load_state_dict(ref.state_dict())
        patch_model(m, "anchor_attn", {"theta": -1e4})
        assert ref.config._attn_implementation != plug.ATTN_NAME and m.config._attn_implementation == plug.ATTN_NAME
        if kw:
            assert m.config.layer_types == ["full_attention", "sliding_attention"]
        masks = []
        inner = plug._dense
        monkeypatch.setattr(plug, "_dense", lambda q, k, v, mask, *a: (masks.append(mask is not None), inner(q, k, v, mask, *a))[1])
        x = torch.randint(0, 1000, (1, 2 * 2048 + 5), device="cuda")
        with torch.no_grad():
            a = ref(x, logits_to_keep=32).logits.float()
            b = m(x, logits_to_keep=32).logits.float()
        assert torch.isfinite(b).all() and (a - b).abs().max() < 0.08 * a.abs().max()
        # full-attention layers: the operator plus a dense tail without a mask; the sliding layer: dense with its mask
        assert masks == ([False, True] if kw else [False, False]), masks
        monkeypatch.setattr(plug, "_dense", inner)
    patch_model(m, "anchor_attn", {"theta": 12})
    monkeypatch.setattr(plug, "record_ratio", True)
    y = torch.randint(0, 1000, (1, 3 * 2048), device="cuda")
    with torch.no_grad():
        c = m(y, logits_to_keep=1).logits
    assert torch.isfinite(c).all()
    assert 0 < float(plug.last_ratio) <= 1.0


@pytest.mark.gpu
def test_dense_plug_is_the_own_kernel_plus_tail():
    """The dense plug on HF-layout tensors with a ragged length: rows below the last multiple of 128 come from
    aa_dense_causal_fwd (bit for bit what dense_causal_attention returns), the tail from the framework; the whole
    agrees with float64 library attention."""
    from anchor_attn.src.modules.llama import anchor_attention as aa
    from anchor_attn.src.ops.anchor_attn_v4 import dense_causal_attention
    from anchor_attn.synthetic import make_qkv
    n = 2048 + 128 + 37
    q, k, v, _ = make_qkv(2048 + 256, 4, 2, n_stripes=16, seed=8)
    q, k, v = (t[:, :, :n].cuda() for t in (q, k, v))
    qh, kh, vh = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q, k, v))
    out, w = aa.dense_attention_forward(types.SimpleNamespace(config=None), qh, kh, vh, None, scaling=128 ** -0.5)
    assert w is None and out.shape == (1, n, 4, 128) and out.is_contiguous()
    main = n - n % 128
    want = dense_causal_attention(q[:, :, :main].contiguous(), k[:, :, :main].contiguous(), v[:, :, :main].contiguous())
    assert torch.equal(out.transpose(1, 2)[:, :, :main], want)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.double(), k.double().repeat_interleave(2, 1), v.double().repeat_interleave(2, 1), is_causal=True)
    err = (out.transpose(1, 2).double() - ref).abs()
    assert err.max() < 2e-2 and err.mean() < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("n_layers", [2, 32])
def test_llama8b_prefill_at_128k_all_patterns(n_layers):
    """BASELINE config 4: the Llama-3.1-8B architecture (hidden 4096, FFN 14336, 32/8 heads, vocab 128256, RoPE base
    5e5) with random-init bf16 weights at the full 131072 tokens - all 32 layers (16 GB of weights; patterns
    "anchor_attn" and "dense"), and two layers through the library-attention pattern "flash" as well.  Every layer's
    attention goes through the plug exactly once; the sparse prefill causes no host synchronisation inside the plug
    (the ratio stays on the device); logits are finite; the dense pattern (own kernel) and the flash pattern
    (library attention) agree."""
    import gc

    from transformers import AttentionInterface, LlamaConfig, LlamaForCausalLM

    from anchor_attn import patch_model
    from anchor_attn.src.modules.llama import anchor_attention as plug
    n_ctx = 131072
    gc.collect()
    torch.cuda.empty_cache()
    torch.manual_seed(0)
    cfg = LlamaConfig(hidden_size=4096, intermediate_size=14336, num_hidden_layers=n_layers, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, vocab_size=128256, max_position_embeddings=n_ctx,
                      rope_theta=5e5, tie_word_embeddings=False)
    with torch.device("cuda"):
        model = LlamaForCausalLM(cfg).to(torch.bfloat16).eval()
    tokens = torch.randint(0, cfg.vocab_size, (1, n_ctx), device="cuda")
    calls = {"anchor": 0, "dense": 0}
    ratios = []
    sparse_inner, dense_inner = plug.anchor_attention_forward, plug.dense_attention_forward

    def sparse_counted(*a, **k):
        calls["anchor"] += 1
        torch.cuda.set_sync_debug_mode("error")  # any host<-device wait inside the plug raises
        try:
            r = sparse_inner(*a, **k)
        finally:
            torch.cuda.set_sync_debug_mode("default")
        ratios.append(plug.last_ratio)
        return r

    def dense_counted(*a, **k):
        calls["dense"] += 1
        return dense_inner(*a, **k)

    def prefill():
        with torch.no_grad():
            return model(tokens, use_cache=False, logits_to_keep=4).logits.float()

    patch_model(model, "anchor_attn")
    old_flag = plug.record_ratio
    try:
        plug.record_ratio = True
        AttentionInterface.register(plug.ATTN_NAME, sparse_counted)
        AttentionInterface.register(plug.DENSE_ATTN_NAME, dense_counted)
        sparse = prefill()
        assert calls == {"anchor": n_layers, "dense": 0}
        assert all(r is not None and r.is_cuda and r.dim() == 0 for r in ratios)
        assert all(0.0 < float(r) <= 1.0 for r in ratios)
        patch_model(model, "dense")
        dense = prefill()
        assert calls == {"anchor": n_layers, "dense": n_layers}
    finally:
        plug.record_ratio = old_flag
        AttentionInterface.register(plug.ATTN_NAME, sparse_inner)
        AttentionInterface.register(plug.DENSE_ATTN_NAME, dense_inner)
    assert sparse.shape == dense.shape == (1, 4, cfg.vocab_size)
    assert torch.isfinite(sparse).all() and torch.isfinite(dense).all()
    if n_layers == 2:
        patch_model(model, "flash")
        flash = prefill()
        assert torch.isfinite(flash).all()
        scale = flash.abs().max()
        assert (dense - flash).abs().max() < 0.05 * scale and (dense - flash).abs().mean() < 0.01 * flash.abs().mean() + 1e-3
    del model
    gc.collect()
    torch.cuda.empty_cache()

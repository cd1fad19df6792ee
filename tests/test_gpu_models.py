"""GPU parity: whole decode steps of the Llama-family and GPT-2 assemblies against
the oracle's restatement of the reference's CPU transformers, on identical
quantized bytes.  Logits: |gpu - ref| <= 1e-3 * max|ref| (fp32 accumulate).
Greedy token ids on the tiny model must be identical."""
import numpy as np
import pytest

import oracle as orc
import wgml_amd as W
from wgml_amd.models import (GPT2_124M, TINY_LLAMA, Gpt2, Gpt2Params, HostMatrix, Llama2, Llama2Config,
                             LlamaModelType, synth_gpt2, synth_llama)

pytestmark = pytest.mark.gpu

MICRO = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=2,
                     vocab_size=320, seq_len=32, rope_base_freq=10000.0, rms_norm_eps=1e-5)


def logits_close(got, ref):
    scale = float(np.abs(ref).max())
    err = float(np.abs(got.astype(np.float64) - ref).max())
    return err <= 1e-3 * scale, err / scale


def spice(w, cfg, seed, biases):
    rng = np.random.default_rng(seed)
    for l in w.layers:
        l["attn_norm"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
        l["ffn_norm"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
        if biases:
            l["attn_q_bias"] = (0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
            l["attn_k_bias"] = (0.1 * rng.standard_normal(cfg.kv_dim)).astype(np.float32)
            l["attn_v_bias"] = (0.1 * rng.standard_normal(cfg.kv_dim)).astype(np.float32)
    w.output_norm = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)


@pytest.mark.parametrize("scheme", ["q8_0", "q4_k", "q6_k", "q4_k_m", "f32"])
@pytest.mark.parametrize("model_type", [LlamaModelType.Llama, LlamaModelType.Qwen2])
@pytest.mark.parametrize("fusion", [0, 1, 2, 3])
def test_llama_micro_logits_and_kv(gpu, scheme, model_type, fusion):
    w = synth_llama(MICRO, seed=21, scheme=scheme)
    spice(w, MICRO, 5, biases=model_type == LlamaModelType.Qwen2)
    ref = orc.Llama2(w, rope_variant=model_type)
    m = Llama2(gpu, MICRO, model_type).load(w)
    m.set_fusion(fusion)
    toks = [3, 300, 17, 17, 250, 9, 1, 77, 12]
    for pos, t in enumerate(toks):
        want = ref.forward(t, pos)
        got = m.forward_logits(pos, t)
        ok, e = logits_close(got, want)
        assert ok, (pos, e)
    for layer in range(MICRO.n_layers):
        for which, ref_c in ((0, ref.key_cache(layer)), (1, ref.value_cache(layer))):
            want_c = ref_c[:len(toks)]
            np.testing.assert_allclose(m.kv_download(layer, which, 0, len(toks)), want_c,
                                       rtol=0, atol=1e-3 * np.abs(want_c).max())


def test_tiny_llama_greedy_tokens_identical(gpu):
    # the tiny Llama-2 configuration: Q8_0 weights, 16-token seeded prompt, 128 greedy tokens
    cfg = TINY_LLAMA
    w = synth_llama(cfg, seed=1, scheme="q8_0")
    prompt = W.prompt_tokens(1, 16, cfg.vocab_size)
    n_total = 16 + 128
    want, margins = orc.Llama2(w, predequantize=True).generate_greedy(prompt, n_total)
    m = Llama2(gpu, cfg).load(w)
    got = m.generate_greedy(prompt, n_total)
    print(f"top-2 logit margin: min {margins.min():.3e}, median {np.median(margins):.3e}; "
          f"{m.launches_per_token()} launches/token")
    assert np.array_equal(got, want)
    # and once more without any fusion (one launch per reference op)
    m2 = Llama2(gpu, cfg).load(w)
    m2.set_fusion(0)
    assert np.array_equal(m2.generate_greedy(prompt, n_total), want)
    # the recorded loop (device-side sampling, no host round trip) and the loop that reads
    # every token back must agree, from any start position, and be repeatable
    a = m.decode_greedy(int(want[15]), 16, 64)
    b = m.decode_greedy_sync(int(want[15]), 16, 64)
    assert np.array_equal(a, want[16:80]) and np.array_equal(b, want[16:80])
    assert np.array_equal(m.decode_greedy(int(want[15]), 16, 64), a)


@pytest.mark.parametrize("model_type", [LlamaModelType.Llama, LlamaModelType.Qwen2])
def test_llama_recorded_loop_matches_oracle(gpu, model_type):
    # grouped-query micro model with biases: the recorded step must handle the
    # position-dependent KV-cache column, RoPE variant and forced prompt tokens
    w = synth_llama(MICRO, seed=31, scheme="q4_k_m")
    spice(w, MICRO, 6, biases=model_type == LlamaModelType.Qwen2)
    prompt = W.prompt_tokens(31, 5, MICRO.vocab_size)
    want, _ = orc.Llama2(w, rope_variant=model_type).generate_greedy(prompt, MICRO.seq_len)
    for fusion in (0, 1, 2, 3):
        m = Llama2(gpu, MICRO, model_type).load(w)
        m.set_fusion(fusion)
        assert np.array_equal(m.generate_greedy(prompt, MICRO.seq_len), want), fusion


def test_tuning_change_rerecords_the_step(gpu):
    # a launch-shape override set after a model has recorded its step must take effect: the
    # captures are dropped and made again.  Seventeen workgroups per head are more than the output
    # projection merges itself, so each layer gains a merge launch; tokens stay the same.
    w = synth_llama(MICRO, seed=21, scheme="q8_0")
    spice(w, MICRO, 5, biases=False)
    m = Llama2(gpu, MICRO).load(w)
    prompt = [3, 300, 17]
    base = m.generate_greedy(prompt, 20)
    n0 = m.launches_per_token()
    gpu.set_tuning(gpu.TUNE_ATTN_WIDE_POSITIONS, 1)  # no single-workgroup plan at this length
    gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, 17)
    try:
        again = m.generate_greedy(prompt, 20)
        assert m.launches_per_token() == n0 + MICRO.n_layers
    finally:
        gpu.set_tuning(gpu.TUNE_ATTN_WIDE_POSITIONS, 0)
        gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, 0)
    assert np.array_equal(base, again)
    assert np.array_equal(m.generate_greedy(prompt, 20), base)
    assert m.launches_per_token() == n0
    for key, bad in ((gpu.TUNE_GEMV_WG_PER_CU, 9), (gpu.TUNE_ATTN_WIDE_POSITIONS, (1 << 20) + 1),
                     (gpu.TUNE_GEMV_WAVES_PER_WG, 5), (gpu.TUNE_ATTN_SPLITS, 65),
                     (gpu.TUNE_ATTN_MERGE, 2)):
        with pytest.raises(W.WgmlError):
            gpu.set_tuning(key, bad)


def test_recording_steps_ahead_of_time(gpu):
    # record_steps captures what the token loop replays (single steps and runs of eight) for a
    # range of positions without touching caches or logits; the loop that follows gives the
    # oracle's tokens, also for step counts that are no multiple of eight
    w = synth_llama(MICRO, seed=23, scheme="q8_0")
    spice(w, MICRO, 7, biases=False)
    prompt = W.prompt_tokens(8, 3, MICRO.vocab_size)
    want_t, _ = orc.Llama2(w).generate_greedy(prompt, 29)
    m = Llama2(gpu, MICRO).load(w)
    m.record_steps(0, MICRO.seq_len)
    for n in (29, 8, 7, 17):
        assert np.array_equal(m.generate_greedy(prompt, n), want_t[:n]), n
    # a decode that continues from a cache the caller filled: recording must leave it, and
    # the logits of the last step, alone (a changed override drops what was recorded)
    kv0 = m.kv_download(0, 0, 0, 8).copy()
    logits0 = m.logits().copy()
    gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, 3)
    try:
        m.record_steps(8, 16)
    finally:
        gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, 0)
    assert np.array_equal(m.kv_download(0, 0, 0, 8), kv0)
    assert np.array_equal(m.logits(), logits0)
    with pytest.raises(W.WgmlError):
        m.record_steps(MICRO.seq_len - 1, 2)


def test_output_projection_merging_attention_partials(gpu):
    # on request the layer's output projection merges attention's partial results itself: the
    # step keeps its launch count at a short context (no merge launch either way) and its tokens
    w = synth_llama(MICRO, seed=22, scheme="q4_k")
    spice(w, MICRO, 6, biases=False)
    prompt = W.prompt_tokens(6, 5, MICRO.vocab_size)
    want_t, _ = orc.Llama2(w).generate_greedy(prompt, 24)
    m = Llama2(gpu, MICRO).load(w)
    assert np.array_equal(m.generate_greedy(prompt, 24), want_t)
    n0 = m.launches_per_token()
    gpu.set_tuning(gpu.TUNE_ATTN_MERGE, 1)
    try:
        got = m.generate_greedy(prompt, 24)
        assert m.launches_per_token() == n0
    finally:
        gpu.set_tuning(gpu.TUNE_ATTN_MERGE, 0)
    assert np.array_equal(got, want_t)


@pytest.mark.parametrize("scheme", ["q8_0", "q4_k", "q6_k", "q4_k_m"])
@pytest.mark.parametrize("model_type", [LlamaModelType.Llama, LlamaModelType.Qwen2])
def test_llama_micro_fp32_activations_fused(gpu, scheme, model_type):
    # the step with fp32 activations in every GEMV (the arithmetic of the reference's shaders)
    # takes the same fused launches as the integer-dot step: 5 launches per layer
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 1)
    try:
        w = synth_llama(MICRO, seed=21, scheme=scheme)
        spice(w, MICRO, 5, biases=model_type == LlamaModelType.Qwen2)
        ref = orc.Llama2(w, rope_variant=model_type)
        m = Llama2(gpu, MICRO, model_type).load(w)
        for pos, t in enumerate([3, 300, 17, 17, 250, 9, 1]):
            want = ref.forward(t, pos)
            got = m.forward_logits(pos, t)
            scale = float(np.abs(want).max())
            assert np.abs(got - want).max() <= 2e-4 * scale, pos
        extra = MICRO.n_layers if model_type == LlamaModelType.Qwen2 else 0  # Neox RoPE launch
        assert m.launches_per_token() == 1 + 5 * MICRO.n_layers + 1 + extra
        prompt = W.prompt_tokens(5, 4, MICRO.vocab_size)
        want_t, _ = orc.Llama2(w, rope_variant=model_type).generate_greedy(prompt, 24)
        assert np.array_equal(Llama2(gpu, MICRO, model_type).load(w).generate_greedy(prompt, 24), want_t)
    finally:
        gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 0)


def test_llama_decode_from_uploaded_kv(gpu):
    # pre-filled cache then decode, as the long-context configuration does
    w = synth_llama(MICRO, seed=23, scheme="q6_k")
    ref = orc.Llama2(w)
    m = Llama2(gpu, MICRO).load(w)
    rng = np.random.default_rng(1)
    n_pre = 20
    for layer in range(MICRO.n_layers):
        k = rng.standard_normal((n_pre, MICRO.kv_dim)).astype(np.float32)
        v = rng.standard_normal((n_pre, MICRO.kv_dim)).astype(np.float32)
        ref.key_cache(layer)[:n_pre] = k
        ref.value_cache(layer)[:n_pre] = v
        m.kv_upload(layer, 0, 0, k)
        m.kv_upload(layer, 1, 0, v)
    tok = 7
    want = []
    for pos in range(n_pre, n_pre + 6):
        tok = orc.argmax(ref.forward(tok, pos))
        want.append(tok)
    got = m.decode_greedy(7, n_pre, 6)
    assert list(got) == want


def test_llama_from_gguf_file(gpu, tmp_path):
    # weights written to a GGUF file under the reference's tensor / key names, loaded back
    # through the GGUF reader: same greedy tokens as the oracle on the original weights
    import gguf_writer as gw

    w = synth_llama(MICRO, seed=41, scheme="q4_k_m")
    spice(w, MICRO, 8, biases=True)
    path = tmp_path / "micro.gguf"
    gw.llama_to_gguf(path, w, model_name="qwen2")
    prompt = W.prompt_tokens(41, 4, MICRO.vocab_size)
    want, _ = orc.Llama2(w, rope_variant=LlamaModelType.Qwen2).generate_greedy(prompt, 24)
    g = W.Gguf(path)
    m = Llama2.from_gguf(gpu, g, LlamaModelType.Qwen2)
    assert m.config.dim == MICRO.dim and m.config.vocab_size == MICRO.vocab_size
    assert np.array_equal(m.generate_greedy(prompt, 24), want)


def test_llama_sampled_generation(gpu):
    # temperature / top-p sampling on the host from logits read back every step, seeded coins:
    # the same tokens as the oracle's forward + the oracle's sampler with the same coins.
    # (Top-2 margins in probability space are wide on this model, so fp32 differences between
    # the two forwards do not move a token across a coin.)
    w = synth_llama(MICRO, seed=51, scheme="q8_0")
    prompt = W.prompt_tokens(51, 3, MICRO.vocab_size)
    n_total, temperature, topp, seed = 20, 0.7, 0.95, 1234
    coins = W.rng_uniform(seed, n_total)
    ref = orc.Llama2(w)
    want, tok, gaps = [], int(prompt[0]), []
    for pos in range(n_total):
        logits = ref.forward(tok, pos).astype(np.float32)
        nxt = orc.sample(logits, temperature, topp, float(coins[pos]))
        want.append(nxt)
        tok = int(prompt[pos + 1]) if pos + 1 < len(prompt) else nxt
    m = Llama2(gpu, MICRO).load(w)
    got = m.generate_sampled(prompt, n_total, temperature, topp, seed)
    assert list(got) == want
    assert list(m.generate_sampled(prompt, n_total, temperature, topp, seed)) == want  # seeded
    assert len(set(want)) > 5  # it really samples
    greedy = m.generate_sampled(prompt, n_total, 0.0, 0.9, seed)
    assert np.array_equal(greedy, m.generate_greedy(prompt, n_total))


def test_llama_argument_checks(gpu):
    m = Llama2(gpu, MICRO)
    with pytest.raises(W.WgmlError, match="unset weights"):
        m.forward(0, 0)
    w = synth_llama(MICRO, seed=2, scheme="q8_0")
    bad = w.layers[0]["ffn_down"]
    with pytest.raises(W.WgmlError, match="expected"):
        m.set_matrix("attn_q", 0, bad)
    m.load(w)
    with pytest.raises(W.WgmlError):
        m.forward(MICRO.vocab_size, 0)
    with pytest.raises(W.WgmlError):
        m.forward(0, MICRO.seq_len)


@pytest.mark.parametrize("fusion", [0, 1])
def test_gpt2_micro_logits(gpu, fusion):
    p = Gpt2Params(n_vocab=300, n_seq=32, n_embd=64, n_head=4, n_layer=2, ff_len=256, attn_b=192)
    w = synth_gpt2(p, seed=5)
    rng = np.random.default_rng(4)
    for l in w.layers:
        for g in ("ln_1_g", "ln_2_g"):
            l[g] = (1 + 0.1 * rng.standard_normal(p.n_embd)).astype(np.float32)
        for b in ("ln_1_b", "ln_2_b"):
            l[b] = (0.1 * rng.standard_normal(p.n_embd)).astype(np.float32)
    ref = orc.Gpt2(w)
    m = Gpt2(gpu, p).load(w)
    m.set_fusion(fusion)
    for pos, t in enumerate([1, 250, 33, 7, 7, 100]):
        want = ref.forward(t, pos)
        m.forward(t, pos)
        ok, e = logits_close(m.logits(), want)
        assert ok, (pos, e)


def test_gpt2_from_gguf_file(gpu, tmp_path):
    # weights written under the reference's GPT-2 tensor / key names and loaded back through
    # the GGUF reader: same greedy tokens as the oracle on the original weights (lm_head is the
    # f32 token_embd tensor here, as in the reference)
    import gguf_writer as gw

    p = Gpt2Params(n_vocab=320, n_seq=32, n_embd=64, n_head=4, n_layer=2, ff_len=256, attn_b=192)
    w = synth_gpt2(p, seed=9)
    w.lm_head = HostMatrix(W.F32, p.n_vocab, p.n_embd,
                           np.ascontiguousarray(w.wte, np.float32).view(np.uint8).reshape(-1))
    path = tmp_path / "gpt2.gguf"
    gw.gpt2_to_gguf(path, w)
    prompt = W.prompt_tokens(9, 4, p.n_vocab)
    want, _ = orc.Gpt2(w).generate_greedy(prompt, 20)
    m = Gpt2.from_gguf(gpu, W.Gguf(path))
    assert m.params == p
    assert np.array_equal(m.generate_greedy(prompt, 20), want)


def test_gpt2_124m_greedy_prefix(gpu):
    # GPT-2 124M shape, Q8_0; a 32-token prompt and the first 24 generated tokens against the
    # oracle (the full run to position 1024 is a benchmark, not a CPU-checkable case)
    p = GPT2_124M
    w = synth_gpt2(p, seed=3)
    prompt = W.prompt_tokens(3, 32, p.n_vocab)
    n_total = 32 + 24
    want, margins = orc.Gpt2(w, predequantize=True).generate_greedy(prompt, n_total)
    m = Gpt2(gpu, p).load(w)
    got = m.generate_greedy(prompt, n_total)  # recorded step, folded launches
    print(f"gpt2 top-2 logit margin: min {margins.min():.3e}; {m.launches_per_token()} launches/token")
    assert np.array_equal(got, want)
    assert np.array_equal(m.generate_greedy(prompt, n_total), want)  # replayable
    m.set_fusion(0)  # one launch per op group, host round trip per token
    assert np.array_equal(m.generate_greedy(prompt, n_total), want)


def _same_where_decided(got, want, margins, scale):
    # the oracle's arg-max is only binding where its top-2 margin is wider than the logit
    # error the kernels may have (1e-3 of the logit scale, twice)
    decided = margins > 2e-3 * scale
    assert decided.mean() > 0.5
    assert np.array_equal(got[decided], want[decided]), np.nonzero(got != want)[0]


def test_gpt2_124m_long_prompt_across_recorded_ranges(gpu):
    # the recorded step is captured once per range of positions (attention planned for 256,
    # 512, 1024 positions): a forced 540-token prompt + 8 generated tokens walk through all three
    p = GPT2_124M
    w = synth_gpt2(p, seed=3)
    n_prompt, n_total = 540, 548
    prompt = W.prompt_tokens(5, n_prompt, p.n_vocab)
    orc.set_threads(8)
    try:
        ref = orc.Gpt2(w, predequantize=True)
        want, margins = ref.generate_greedy(prompt, n_total)
        scale = float(np.abs(ref.forward(int(prompt[0]), 0)).max())
    finally:
        orc.set_threads(1)
    m = Gpt2(gpu, p).load(w)
    got = m.generate_greedy(prompt, n_total)
    _same_where_decided(got, want, margins, scale)
    assert np.array_equal(m.generate_greedy(prompt, n_total), got)  # replayable


def test_llama_micro_long_prompt_across_recorded_ranges(gpu):
    cfg = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=2, vocab_size=500,
                       seq_len=1100, rope_base_freq=10000.0, rms_norm_eps=1.0e-5)
    w = synth_llama(cfg, seed=21, scheme="q4_k_m")
    n_prompt, n_total = 1050, 1060
    prompt = W.prompt_tokens(6, n_prompt, cfg.vocab_size)
    ref = orc.Llama2(w)
    want, margins = ref.generate_greedy(prompt, n_total)
    scale = float(np.abs(ref.forward(int(prompt[0]), 0)).max())
    m = Llama2(gpu, cfg).load(w)
    got = m.generate_greedy(prompt, n_total)
    _same_where_decided(got, want, margins, scale)
    # a second run that starts inside the second range, from the KV cache the first one left
    # (only its first step sees the forced prompt's context and nothing else)
    tail = m.decode_greedy(int(prompt[300]), 300, 4)
    if margins[300] > 2e-3 * scale:
        assert int(tail[0]) == int(want[300])


def test_gpt2_micro_greedy_with_norm_affine(gpu):
    # non-trivial LayerNorm gains / shifts and biases through the folded, recorded loop
    p = Gpt2Params(n_vocab=300, n_seq=48, n_embd=128, n_head=4, n_layer=3, ff_len=512, attn_b=384)
    w = synth_gpt2(p, seed=9)
    rng = np.random.default_rng(2)
    for l in w.layers:
        for g in ("ln_1_g", "ln_2_g"):
            l[g] = (1 + 0.2 * rng.standard_normal(p.n_embd)).astype(np.float32)
        for b in ("ln_1_b", "ln_2_b"):
            l[b] = (0.2 * rng.standard_normal(p.n_embd)).astype(np.float32)
    w.ln_f_g = (1 + 0.2 * rng.standard_normal(p.n_embd)).astype(np.float32)
    w.ln_f_b = (0.2 * rng.standard_normal(p.n_embd)).astype(np.float32)
    prompt = W.prompt_tokens(9, 6, p.n_vocab)
    want, _ = orc.Gpt2(w).generate_greedy(prompt, p.n_seq)
    m = Gpt2(gpu, p).load(w)
    m.record_steps(p.n_seq)  # ahead of the first run; step counts that are no multiple of eight
    for n in (p.n_seq, 13, 8, 3):
        assert np.array_equal(m.generate_greedy(prompt, n), want[:n]), n
    with pytest.raises(W.WgmlError):
        m.record_steps(p.n_seq + 1)
    m.set_fusion(0)
    m.record_steps(p.n_seq)  # nothing to record for the loop with one launch per op
    assert np.array_equal(m.generate_greedy(prompt, p.n_seq), want)


def test_gpt2_matrix_replaced_after_a_recorded_run(gpu):
    # the recorded step holds device pointers of the matrices: replacing one (and freeing the
    # old one) must re-record, not replay launches that read freed memory
    from wgml_amd.models import _rand_matrix

    p = Gpt2Params(n_vocab=300, n_seq=40, n_embd=128, n_head=4, n_layer=2, ff_len=512, attn_b=384)
    w = synth_gpt2(p, seed=13)
    prompt = W.prompt_tokens(13, 5, p.n_vocab)
    m = Gpt2(gpu, p).load(w)
    want0, _ = orc.Gpt2(w).generate_greedy(prompt, p.n_seq)
    assert np.array_equal(m.generate_greedy(prompt, p.n_seq), want0)  # records the step
    for name, layer, shape in (("mlp_fc_w", 0, (p.ff_len, p.n_embd)), ("attn_w", 1, (p.attn_b, p.n_embd)),
                               ("lm_head", 0, (p.n_vocab, p.n_embd))):
        new = _rand_matrix(9000 + layer, shape[0], shape[1], W.Q8_0, std=0.05)
        if name == "lm_head":
            w.lm_head = new
        else:
            w.layers[layer][name] = new
        m.set_matrix(name, layer, new)  # releases the matrix it replaces
        import gc
        gc.collect()
        want, _ = orc.Gpt2(w).generate_greedy(prompt, p.n_seq)
        assert np.array_equal(m.generate_greedy(prompt, p.n_seq), want), name
    assert not np.array_equal(want, want0)


@pytest.mark.parametrize("qtype", [W.Q4_0, W.Q4_1, W.Q5_0, W.Q5_1, W.Q5_K, W.Q8_K])
def test_llama_micro_in_the_remaining_block_formats(gpu, qtype):
    # a model whose matrices are all in one of the formats beside Q8_0 / Q4_K / Q6_K: they
    # stay quantized on the device and take the same fused Q/K/V and gate/up launches (a launch
    # holds matrices of one format) and the batched prompt pass; logits, KV rows and greedy
    # tokens against the oracle, and the fused step against the step with one launch per matrix
    import npref

    w = synth_llama(MICRO, seed=61, scheme="f32")
    for layer in w.layers:
        for name, v in list(layer.items()):
            if isinstance(v, HostMatrix):
                vals = v.data.view(np.float32)
                layer[name] = HostMatrix(qtype, v.nrows, v.ncols, npref.encode_simple(qtype, vals))
    w.output = HostMatrix(qtype, w.output.nrows, w.output.ncols,
                          npref.encode_simple(qtype, w.output.data.view(np.float32)))
    spice(w, MICRO, 9, biases=False)
    ref = orc.Llama2(w)
    m = Llama2(gpu, MICRO).load(w)
    toks = [3, 300, 17, 250, 9, 1]
    for pos, t in enumerate(toks):
        ok, e = logits_close(m.forward_logits(pos, t), ref.forward(t, pos))
        assert ok, (pos, e)
    assert m.launches_per_token() == 1 + 5 * MICRO.n_layers + 1  # embed, 5 per layer, output
    want_k = ref.key_cache(1)[:len(toks)].copy()
    np.testing.assert_allclose(m.kv_download(1, 0, 0, len(toks)), want_k, rtol=0,
                               atol=1e-3 * np.abs(want_k).max())
    unfused = Llama2(gpu, MICRO).load(w)
    unfused.set_fusion(2)
    for pos, t in enumerate(toks):
        lg = unfused.forward_logits(pos, t)
    assert unfused.launches_per_token() > m.launches_per_token()
    assert np.abs(lg - m.forward_logits(len(toks) - 1, toks[-1])).max() <= 1e-4 * np.abs(lg).max()
    m2 = Llama2(gpu, MICRO).load(w)
    m2.prefill(toks)  # the batched prompt pass
    ok, e = logits_close(m2.logits(), ref.forward(toks[-1], len(toks) - 1))
    assert ok, e
    prompt = W.prompt_tokens(61, 4, MICRO.vocab_size)
    want, _ = orc.Llama2(w).generate_greedy(prompt, 20)
    assert np.array_equal(Llama2(gpu, MICRO).load(w).generate_greedy(prompt, 20), want)

"""Composition checks of the oracle's model forwards (no GPU needed).

The reference holds no golden logits; what can be pinned is that the C
restatement of cpu.rs composes its ops the way the architecture says, by
comparing with a separately written float64 numpy forward.
"""
import numpy as np
import pytest

import npref
import oracle as orc
import wgml_amd as W
from wgml_amd.models import Gpt2Params, Llama2Config, synth_gpt2, synth_llama

MICRO = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=2,
                     vocab_size=320, seq_len=16, rope_base_freq=10000.0, rms_norm_eps=1e-5)


@pytest.mark.parametrize("scheme", ["q8_0", "q4_k", "q6_k", "q4_k_m"])
@pytest.mark.parametrize("variant", [0, 1])
def test_llama_forward_vs_float64_numpy(scheme, variant):
    w = synth_llama(MICRO, seed=11, scheme=scheme)
    rng = np.random.default_rng(3)
    # non-trivial norms and (for the Neox / Qwen2 variant) q/k/v biases
    for l in w.layers:
        l["attn_norm"] = (1 + 0.1 * rng.standard_normal(MICRO.dim)).astype(np.float32)
        l["ffn_norm"] = (1 + 0.1 * rng.standard_normal(MICRO.dim)).astype(np.float32)
        if variant == 1:
            l["attn_q_bias"] = (0.1 * rng.standard_normal(MICRO.dim)).astype(np.float32)
            l["attn_k_bias"] = (0.1 * rng.standard_normal(MICRO.kv_dim)).astype(np.float32)
            l["attn_v_bias"] = (0.1 * rng.standard_normal(MICRO.kv_dim)).astype(np.float32)
    toks = [5, 17, 300, 42, 8]
    m = orc.Llama2(w, rope_variant=variant)
    for pos, t in enumerate(toks):
        got = m.forward(t, pos)
    want = npref.llama_forward_f64(w, toks, rope_variant=variant)
    scale = np.abs(want).max()
    np.testing.assert_allclose(got, want, atol=1e-4 * scale)
    # pre-dequantized weights give bit-identical logits (same arithmetic, other storage)
    m2 = orc.Llama2(w, rope_variant=variant, predequantize=True)
    for pos, t in enumerate(toks):
        got2 = m2.forward(t, pos)
    assert np.array_equal(got, got2)


def test_gpt2_forward_vs_float64_numpy():
    p = Gpt2Params(n_vocab=300, n_seq=16, n_embd=64, n_head=4, n_layer=2, ff_len=256, attn_b=192)
    w = synth_gpt2(p, seed=5)
    rng = np.random.default_rng(4)
    for l in w.layers:
        for g in ("ln_1_g", "ln_2_g"):
            l[g] = (1 + 0.1 * rng.standard_normal(p.n_embd)).astype(np.float32)
        for b in ("ln_1_b", "ln_2_b"):
            l[b] = (0.1 * rng.standard_normal(p.n_embd)).astype(np.float32)
    w.ln_f_g = (1 + 0.1 * rng.standard_normal(p.n_embd)).astype(np.float32)
    w.ln_f_b = (0.1 * rng.standard_normal(p.n_embd)).astype(np.float32)
    toks = [1, 250, 33, 7]
    m = orc.Gpt2(w)
    for pos, t in enumerate(toks):
        got = m.forward(t, pos)
    want = npref.gpt2_forward_f64(w, toks)
    np.testing.assert_allclose(got, want, atol=1e-4 * np.abs(want).max())


def test_greedy_loop_contract():
    w = synth_llama(MICRO, seed=12, scheme="q8_0")
    m = orc.Llama2(w)
    prompt = W.prompt_tokens(12, 4, MICRO.vocab_size)
    out, margins = m.generate_greedy(prompt, 10)
    assert out.shape == (10,) and (out < MICRO.vocab_size).all() and (margins >= 0).all()
    # position p consumes prompt[p] while p < len(prompt): regenerate with a longer prompt that
    # extends the old one by its own continuation -> same tokens
    m2 = orc.Llama2(w)
    longer = np.concatenate([prompt, out[3:6]])
    out2, _ = m2.generate_greedy(longer, 10)
    assert np.array_equal(out, out2)


def test_thread_count_of_the_timing_mode_does_not_change_results():
    from wgml_amd.models import Llama2Config, synth_llama

    cfg = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=2,
                       vocab_size=320, seq_len=16)
    w = synth_llama(cfg, seed=3, scheme="q4_k_m")
    a = orc.Llama2(w, predequantize=True)
    b = orc.Llama2(w)
    try:
        for pos, t in enumerate([5, 17, 300]):
            orc.set_threads(1)
            want = a.forward(t, pos)
            orc.set_threads(4)
            assert np.array_equal(b.forward(t, pos), want)
            raw = w.layers[0]["ffn_gate"]
            x = W.rng_normal(pos, cfg.dim)
            orc.set_threads(1)
            r1 = orc.gemv_quant(raw.qtype, raw.data, raw.nrows, raw.ncols, x)
            orc.set_threads(4)
            r4 = orc.gemv_quant(raw.qtype, raw.data, raw.nrows, raw.ncols, x)
            assert np.array_equal(r1[0], r4[0]) and np.array_equal(r1[1], r4[1])
    finally:
        orc.set_threads(1)

"""GPU parity of the two large benchmark configurations as ASSEMBLED models (the kernels are
covered at these sizes one by one elsewhere; this file measures how their errors add up over
the depth of a real model):

  * the full 32-layer Llama-2-7B shape in the Q4_K_M mix: single-token steps and the batched
    prompt pass against the oracle's step-by-step forward;
  * the Llama-3-8B widths (32 query / 8 KV heads, hidden 14336, vocabulary 128256, RoPE base
    500000, Q6_K) cut to 2 layers, KV caches filled to position 8191, steps at positions >= 8192.

Bar: |gpu - ref| <= 1e-3 * max|ref| on the logits (fp32 accumulate); the observed error is printed
next to that budget for every path."""
import time

import numpy as np
import pytest

import oracle as orc
import wgml_amd as W
from wgml_amd.models import LLAMA2_7B, Llama2, Llama2Config, synth_llama

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(1500)]

BUDGET = 1e-3


def rel_err(got, ref):
    return float(np.abs(got.astype(np.float64) - ref).max() / np.abs(ref).max())


def test_llama2_7b_q4_k_m_assembled(gpu):
    cfg = LLAMA2_7B
    t0 = time.perf_counter()
    w = synth_llama(cfg, seed=4, scheme="q4_k_m")
    ref = orc.Llama2(w, predequantize=True)
    print(f"\n7B weights + f32 oracle copy built in {time.perf_counter() - t0:.0f}s", flush=True)
    n_prompt, n_steps = 8, 3
    prompt = W.prompt_tokens(4, n_prompt, cfg.vocab_size)
    # oracle: the prompt one token at a time, then greedy steps
    want, toks = [], []
    tok = int(prompt[0])
    t0 = time.perf_counter()
    for pos in range(n_prompt + n_steps):
        logits = ref.forward(tok, pos)
        want.append(logits)
        nxt = orc.argmax(logits)
        toks.append(nxt)
        tok = int(prompt[pos + 1]) if pos + 1 < n_prompt else nxt
    print(f"oracle: {n_prompt + n_steps} steps in {time.perf_counter() - t0:.0f}s", flush=True)
    top2 = np.partition(want[-1], -2)[-2:]
    print(f"top-2 logit margin at the last step: {top2[1] - top2[0]:.3e}, max|logit| "
          f"{np.abs(want[-1]).max():.3e}", flush=True)

    m = Llama2(gpu, cfg).load(w)
    # (1) the decode step as benchmarked (fused launches, integer-dot GEMV with 16-bit block
    # fixed-point activations), token by token with the oracle's tokens
    worst = 0.0
    feed = [int(prompt[0])] + [int(prompt[p + 1]) if p + 1 < n_prompt else toks[p]
                               for p in range(n_prompt + n_steps - 1)]
    for pos, t in enumerate(feed):
        got = m.forward_logits(pos, t)
        e = rel_err(got, want[pos])
        worst = max(worst, e)
        assert e <= BUDGET, (pos, e)
    print(f"7B step, integer-dot path: worst logit error {worst:.2e} of max|logit| "
          f"(budget {BUDGET:.0e}) over {len(feed)} positions", flush=True)
    # KV rows of the first and last layer after those steps
    for layer in (0, cfg.n_layers - 1):
        for which, ref_c in ((0, ref.key_cache(layer)), (1, ref.value_cache(layer))):
            want_c = ref_c[:len(feed)]
            got_c = m.kv_download(layer, which, 0, len(feed))
            assert np.abs(got_c - want_c).max() <= BUDGET * np.abs(want_c).max(), (layer, which)

    # (2) the recorded loop (HIP graph replay, device-side arg-max): same tokens as the oracle
    # wherever the oracle's top-2 margin is wider than twice the error budget
    got_toks = m.generate_greedy(prompt, n_prompt + n_steps)
    for pos in range(n_prompt + n_steps):
        t2 = np.partition(want[pos], -2)[-2:]
        if t2[1] - t2[0] > 2 * BUDGET * np.abs(want[pos]).max():
            assert int(got_toks[pos]) == toks[pos], pos

    # (3) the batched prompt pass, both precisions, then steps that continue from its KV cache
    for level, name, budget in ((1, "split f16", BUDGET), (0, "plain f16", 1e-2)):
        gpu.set_gemm_precision(level)
        m.prefill(prompt)
        e = rel_err(m.logits(), want[n_prompt - 1])
        worst = e
        for i in range(n_steps):
            pos = n_prompt + i
            e2 = rel_err(m.forward_logits(pos, feed[pos]), want[pos])
            worst = max(worst, e2)
        print(f"7B prompt pass ({name}), {n_prompt} tokens: logit error {e:.2e}; worst over the "
              f"{n_steps} steps that follow {worst:.2e} (budget {budget:.0e})", flush=True)
        assert worst <= budget, (name, worst)
    gpu.set_gemm_precision(1)
    m.close()


def test_llama3_8b_gqa_long_context_assembled(gpu):
    # the widths of the long-context configuration, cut to 2 layers so that the oracle (and its
    # 2 x 8448-row KV caches) stays small; everything that depends on depth is covered by the
    # 7B test above, everything that depends on width, GQA, theta and position is here
    cfg = Llama2Config(dim=4096, hidden_dim=14336, n_layers=2, n_q_heads=32, n_kv_heads=8,
                       vocab_size=128256, seq_len=8448, rope_base_freq=500000.0,
                       rms_norm_eps=1.0e-5)
    t0 = time.perf_counter()
    w = synth_llama(cfg, seed=5, scheme="q6_k")
    ref = orc.Llama2(w, predequantize=True)
    m = Llama2(gpu, cfg).load(w)
    n_pre = 8192
    for layer in range(cfg.n_layers):
        for which in (0, 1):
            kv = W.rng_normal(1000 + 2 * layer + which, n_pre * cfg.kv_dim).reshape(n_pre, cfg.kv_dim)
            (ref.key_cache(layer) if which == 0 else ref.value_cache(layer))[:n_pre] = kv
            m.kv_upload(layer, which, 0, kv)
    print(f"\n8B-width 2-layer model + caches built in {time.perf_counter() - t0:.0f}s", flush=True)
    tok, want, toks = 7, [], []
    for pos in range(n_pre, n_pre + 3):
        logits = ref.forward(tok, pos)
        want.append(logits)
        tok = orc.argmax(logits)
        toks.append(tok)
    feed = [7] + toks[:-1]
    worst = 0.0
    for i, t in enumerate(feed):
        e = rel_err(m.forward_logits(n_pre + i, t), want[i])
        worst = max(worst, e)
    print(f"8B-width GQA steps at positions {n_pre}..{n_pre + 2}: worst logit error {worst:.2e} "
          f"of max|logit| (budget {BUDGET:.0e})", flush=True)
    assert worst <= BUDGET
    for which, ref_c in ((0, ref.key_cache(1)), (1, ref.value_cache(1))):
        want_c = ref_c[n_pre:n_pre + 3]
        got_c = m.kv_download(1, which, n_pre, 3)
        assert np.abs(got_c - want_c).max() <= BUDGET * np.abs(want_c).max(), which
    # the recorded loop from the same uploaded caches (the steps above rewrote rows 8192.. with
    # the same values, so the state is the one the oracle started from)
    got = m.decode_greedy(7, n_pre, 3)
    for i in range(3):
        t2 = np.partition(want[i], -2)[-2:]
        if t2[1] - t2[0] > 2 * BUDGET * np.abs(want[i]).max():
            assert int(got[i]) == toks[i], i
    m.close()

"""GPU parity: the batched matrix product and the batched prompt pass ("prefill").

The reference has neither: it runs the prompt through its batch-1 step token by token
(wgml-chat/src/chat_llama2.rs:155-228).  The batched path is therefore held against that
sequence -- the oracle's N single-token steps on the same quantized bytes.

Two precisions (wgml_ctx_set_gemm_precision), both tested:
  1 (default)  operands as pairs of f16 numbers (high + low part), fp32 sums: products agree with
               the exact product of the dequantized weights to fp32 rounding.  Bounds:
               |gpu - ref| <= 1e-4 * |ref| + 2e-5 * rms(ref) for products, 2e-4 * max|ref| for
               logits and cache rows after a whole model pass (the tolerance of the step itself is
               1e-3; observed ~1e-6 and ~2e-5).
  0            operands rounded to f16 once: a product's error is about 2^-11 / sqrt(3) per term,
               random in sign, ~3e-4 of rms(ref) observed.  Bounds: 1e-3 * |ref| + 2e-3 * rms(ref)
               for products, 3e-3 * max|ref| after a whole pass of the 2-layer models.
"""
import numpy as np
import pytest

import npref
import oracle as orc
import wgml_amd as W
from wgml_amd._lib import E_UNSUPPORTED

pytestmark = pytest.mark.gpu
QT = [W.Q8_0, W.Q4_K, W.Q6_K]


@pytest.fixture(params=[0, 1, 2, 3, 8], ids=["ksplit_auto", "ksplit1", "ksplit2", "ksplit3", "ksplit8"])
def k_split(request, gpu):
    # workgroups that share the K range of a product (their partial sums are added by a
    # second kernel): chosen by matrix shape, or forced
    gpu.set_tuning(gpu.TUNE_GEMM_K_SPLIT, request.param)
    yield request.param
    gpu.set_tuning(gpu.TUNE_GEMM_K_SPLIT, 0)


TOL = {"prod_rel": 1e-4, "prod_rms": 2e-5, "model": 2e-4}


@pytest.fixture(params=[1, 0], ids=["split_f16", "plain_f16"], autouse=True)
def precision(request, gpu):
    gpu.set_gemm_precision(request.param)
    if request.param:
        TOL.update(prod_rel=1e-4, prod_rms=2e-5, model=2e-4)
    else:
        TOL.update(prod_rel=1e-3, prod_rms=2e-3, model=3e-3)
    yield request.param
    gpu.set_gemm_precision(1)
    TOL.update(prod_rel=1e-4, prod_rms=2e-5, model=2e-4)


def gemm(gpu, qtype, raw, nrows, ncols, x):
    T = x.shape[0]
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    xv = W.GpuVector.init(gpu, x.reshape(-1))
    out = W.GpuVector.init(gpu, np.full(T * nrows, np.nan, dtype=np.float32))
    W.GemmQuant.from_device(gpu).dispatch(out, m, xv, T)
    return out.read().reshape(T, nrows)


def reference(qtype, raw, nrows, ncols, x):
    w = orc.dequantize(qtype, raw, nrows * ncols).reshape(nrows, ncols).astype(np.float64)
    return x.astype(np.float64) @ w.T


def check(got, ref):
    rms = float(np.sqrt((ref ** 2).mean())) or 1.0
    err = np.abs(got.astype(np.float64) - ref)
    assert np.isfinite(got).all()
    assert (err <= TOL["prod_rel"] * np.abs(ref) + TOL["prod_rms"] * rms).all(), float(err.max() / rms)
    return float(err.max() / rms)


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("T", [1, 5, 16, 17, 37, 64, 100, 128])
@pytest.mark.parametrize("nrows,ncols", [(16, 256), (5, 512), (100, 768), (333, 2048)])
def test_gemm_matches_dequantized_product(gpu, k_split, qtype, T, nrows, ncols):
    raw = W.quantize(qtype, W.rng_normal(10 + nrows, nrows * ncols, 0, 0.02))
    x = W.rng_normal(20 + T, T * ncols).reshape(T, ncols)
    check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))


@pytest.mark.parametrize("ncols", [32, 96, 160, 2080])
@pytest.mark.parametrize("T", [3, 40])
def test_gemm_q8_0_rows_not_a_multiple_of_64(gpu, k_split, ncols, T):
    nrows = 21
    raw = W.quantize(W.Q8_0, W.rng_normal(3, nrows * ncols, 0, 0.02))
    x = W.rng_normal(4, T * ncols).reshape(T, ncols)
    check(gemm(gpu, W.Q8_0, raw, nrows, ncols, x), reference(W.Q8_0, raw, nrows, ncols, x))


OTHER = [W.Q4_0, W.Q4_1, W.Q5_0, W.Q5_1, W.Q5_K, W.Q8_K]


def small_blocks(qtype, n_elems, seed):
    """Blocks of a format that has no quantizer here: the closest-value encoder of the test
    helpers over N(0, 0.02) values (weights of ordinary size, well inside the f16 operands)."""
    vals = W.rng_normal(seed, n_elems, 0, 0.02)
    return npref.encode_simple(qtype, vals)


@pytest.mark.parametrize("qtype", OTHER)
@pytest.mark.parametrize("T", [1, 17, 64, 128])
@pytest.mark.parametrize("nrows,ncols", [(16, 256), (100, 768), (333, 2048)])
def test_gemm_in_the_remaining_block_formats(gpu, k_split, qtype, T, nrows, ncols):
    # the batched product for Q4_0 / Q4_1 / Q5_0 / Q5_1 / Q5_K / Q8_K: same bounds as for the
    # three main formats, against the exact product of the bit-exactly dequantized weights
    raw = small_blocks(qtype, nrows * ncols, 40 + nrows)
    x = W.rng_normal(50 + T, T * ncols).reshape(T, ncols)
    check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))


@pytest.mark.parametrize("qtype", [W.Q4_0, W.Q4_1, W.Q5_0, W.Q5_1])
@pytest.mark.parametrize("ncols", [32, 96, 160, 2080])
def test_gemm_32_element_blocks_rows_not_a_multiple_of_64(gpu, k_split, qtype, ncols):
    nrows, T = 21, 9
    raw = small_blocks(qtype, nrows * ncols, 3)
    x = W.rng_normal(4, T * ncols).reshape(T, ncols)
    check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))


@pytest.mark.parametrize("qtype", OTHER)
def test_gemm_remaining_formats_random_block_bits(gpu, qtype):
    # every bit pattern of quants, fifth bits and 6-bit scales (scales kept small enough for the
    # weights to fit the f16 operands: matrices beyond that are refused, see the limit test)
    nrows, ncols, T = 48, 1024, 20
    raw = npref.random_blocks(qtype, nrows * ncols // npref.BLOCK_ELEMS[qtype], seed=77)
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    x = W.rng_normal(78, T * ncols).reshape(T, ncols)
    w = orc.dequantize(qtype, raw, nrows * ncols)
    assert m.weight_bound() >= float(np.abs(w).max()) * (1 - 1e-6)
    if m.weight_bound() <= 255.875:
        check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))
    else:
        with pytest.raises(W.WgmlError):
            gemm(gpu, qtype, raw, nrows, ncols, x)


@pytest.mark.parametrize("qtype", QT)
def test_gemm_agrees_with_gemv_per_token(gpu, qtype):
    nrows, ncols, T = 512, 4096, 24
    raw = W.quantize(qtype, W.rng_normal(7, nrows * ncols, 0, 0.02))
    x = W.rng_normal(8, T * ncols).reshape(T, ncols)
    got = gemm(gpu, qtype, raw, nrows, ncols, x)
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    op = W.GemvQuant.from_device(gpu)
    for t in range(T):
        out = W.GpuVector.init(gpu, np.zeros(nrows, dtype=np.float32))
        op.dispatch(out, m, W.GpuVector.init(gpu, x[t]))
        # the GEMV itself is within 5e-4 * rms of the exact product (16-bit block fixed-point
        # activations, tests/test_gpu_gemv.py): the two agree within the sum of their bounds
        ref = out.read().astype(np.float64)
        rms = float(np.sqrt((ref ** 2).mean()))
        err = np.abs(got[t] - ref)
        assert (err <= TOL["prod_rel"] * np.abs(ref) + (TOL["prod_rms"] + 5e-4) * rms).all(), float(err.max() / rms)


@pytest.mark.parametrize("qtype", QT)
def test_gemm_large_activations_stay_finite(gpu, k_split, qtype):
    # values far beyond the f16 range (65504): the per-token power-of-two scale absorbs them
    nrows, ncols, T = 48, 1024, 9
    raw = W.quantize(qtype, W.rng_normal(1, nrows * ncols, 0, 0.02))
    x = W.rng_normal(2, T * ncols).reshape(T, ncols)
    x[0] *= 1e6
    x[3] *= 3e4
    x[5] = 0.0
    got = gemm(gpu, qtype, raw, nrows, ncols, x)
    ref = reference(qtype, raw, nrows, ncols, x)
    for t in range(T):
        check(got[t:t + 1], ref[t:t + 1])
    assert (got[5] == 0).all()


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("x_scale,w_std", [(1e-3, 0.02), (300.0, 0.02), (1.0, 1.0), (1.0, 1e-3), (1.0, 20.0)])
def test_gemm_operand_magnitudes(gpu, qtype, x_scale, w_std):
    # The low parts of the split operands are small numbers: activations are scaled per token into
    # (512, 1024] (up as well as down) and weights expanded times 2^8 so that they stay f16
    # numbers.  Small and large activations, small and large weights (|w| <= 255.875 is the limit),
    # one outlier in a row: the bounds hold unchanged (observed 2e-7 rms, 2e-6 worst, split f16).
    nrows, ncols, T = 96, 2048, 40
    raw = W.quantize(qtype, W.rng_normal(31, nrows * ncols, 0, w_std))
    x = (W.rng_normal(32, T * ncols) * np.float32(x_scale)).reshape(T, ncols)
    x[3, 17] = 40 * x_scale
    check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))


@pytest.mark.parametrize("qtype", QT)
def test_gemm_weight_magnitude_limit(gpu, qtype):
    # Weights pass through f16 times 2^8, so a matrix is taken only while a bound on its largest
    # dequantized weight stays within 65504 / 256 = 255.875 (computed when the matrix is created: exact for Q8_0,
    # the ends of each sub-block's quant range for Q4_K, |d| |scale| 32 for Q6_K).  Just inside the limit the product
    # is as accurate as anywhere else; at or beyond it the call is refused and the per-token
    # product, which takes any value, still answers.
    nrows, ncols, T = 64, 1024, 20
    u = W.rng_normal(41, nrows * ncols)
    u = np.clip(u / 3.0, -1.0, 1.0).astype(np.float32)
    x = W.rng_normal(42, T * ncols).reshape(T, ncols)
    inside = {W.Q8_0: 250.0, W.Q6_K: 240.0, W.Q4_K: 150.0}[qtype]
    raw = W.quantize(qtype, u * np.float32(inside))
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    w = orc.dequantize(qtype, raw, nrows * ncols)
    assert float(np.abs(w).max()) <= m.weight_bound() <= 255.875
    check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))
    for amp in (256.0, 300.0, 7e4):
        vals = u * np.float32(amp)
        vals[5] = amp  # the largest weight itself reaches the amplitude
        raw = W.quantize(qtype, vals)
        m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
        w = orc.dequantize(qtype, raw, nrows * ncols)
        if not np.isfinite(w).all():
            continue  # beyond what the format's f16 scale holds
        assert m.weight_bound() >= float(np.abs(w).max()) >= 255.0
        if m.weight_bound() <= 255.875:
            # the f16 scale rounded the largest weight to within the limit: taken
            check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))
            continue
        xv = W.GpuVector.init(gpu, x.reshape(-1))
        out = W.GpuVector.init(gpu, np.zeros(T * nrows, dtype=np.float32))
        with pytest.raises(W.WgmlError) as e:
            W.GemmQuant.from_device(gpu).dispatch(out, m, xv, T)
        assert e.value.code == E_UNSUPPORTED
        o1 = W.GpuVector.init(gpu, np.zeros(nrows, dtype=np.float32))
        W.GemvQuant.from_device(gpu).dispatch(o1, m, W.GpuVector.init(gpu, x[0]))
        ref = reference(qtype, raw, nrows, ncols, x[:1])[0]
        assert np.abs(o1.read() - ref).max() <= 5e-4 * np.abs(ref).max()


@pytest.mark.parametrize("qtype", QT)
def test_gemm_7b_shapes(gpu, qtype):
    # the down projection's shape: linearity in x is the size-independent property checked
    # beside the oracle on a slice of rows
    nrows, ncols, T = 4096, 11008, 128
    raw = W.quantize(qtype, W.rng_normal(5, nrows * ncols, 0, 0.02))
    x = W.rng_normal(6, T * ncols).reshape(T, ncols)
    got = gemm(gpu, qtype, raw, nrows, ncols, x)
    rows = np.r_[0:40, 2000:2040, nrows - 40:nrows]
    blk = W.quant_bytes(qtype, ncols)
    sub = np.concatenate([raw[r * blk:(r + 1) * blk] for r in rows])
    check(got[:, rows], reference(qtype, sub, len(rows), ncols, x))
    x2 = np.concatenate([x[:64] + x[64:], 2.0 * x[:64]])  # exact in f32? no: compare loosely
    got2 = gemm(gpu, qtype, raw, nrows, ncols, x2)
    check(got2[:64], (got[:64].astype(np.float64) + got[64:]))
    check(got2[64:], 2.0 * got[:64].astype(np.float64))


def test_gemm_with_views_that_are_not_16_byte_aligned(gpu):
    # x and out are views at odd offsets into larger buffers (the reference's ops take views)
    nrows, ncols, T = 40, 512, 7
    raw = W.quantize(W.Q4_K, W.rng_normal(1, nrows * ncols, 0, 0.02))
    m = W.GpuQuantMatrix(gpu, W.Q4_K, nrows, ncols, raw)
    x = W.rng_normal(2, T * ncols).reshape(T, ncols)
    xbuf = W.GpuVector.init(gpu, np.concatenate([np.zeros(3, np.float32), x.reshape(-1)]))
    obuf = W.GpuVector.init(gpu, np.full(5 + T * nrows, np.nan, dtype=np.float32))
    W.GemmQuant.from_device(gpu).dispatch(obuf.rows(5, T * nrows), m, xbuf.rows(3, T * ncols), T)
    got = obuf.read()
    assert np.isnan(got[:5]).all()
    check(got[5:].reshape(T, nrows), reference(W.Q4_K, raw, nrows, ncols, x))


def test_gemm_rejects_bad_arguments(gpu):
    raw = W.quantize(W.Q8_0, W.rng_normal(1, 8 * 64, 0, 0.02))
    m = W.GpuQuantMatrix(gpu, W.Q8_0, 8, 64, raw)
    op = W.GemmQuant.from_device(gpu)
    x = W.GpuVector.init(gpu, np.zeros(3 * 64, dtype=np.float32))
    out = W.GpuVector.init(gpu, np.zeros(3 * 8, dtype=np.float32))
    with pytest.raises(W.WgmlError):
        op.dispatch(out, m, x, 2)
    with pytest.raises(W.WgmlError):
        op.dispatch(out, m, x, 0)
    with pytest.raises(W.WgmlError):
        op.dispatch(out, m, x, 129)
    f = W.GpuQuantMatrix(gpu, W.F16, 8, 64, np.zeros(8 * 64 * 2, dtype=np.uint8))
    with pytest.raises(W.WgmlError):
        op.dispatch(out, f, x, 3)
    with pytest.raises(W.WgmlError):
        gpu.set_gemm_precision(2)


# ---- the whole prompt pass against the oracle's token-by-token steps -----------------
from wgml_amd.models import TINY_LLAMA, Llama2, Llama2Config, LlamaModelType, synth_llama  # noqa: E402

MICRO = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=2,
                     vocab_size=320, seq_len=40, rope_base_freq=10000.0, rms_norm_eps=1e-5)


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


@pytest.fixture(params=[0, 1], ids=["attn16tok", "attn1tok"])
def attn_mode(request, gpu):
    # attention over a run: 16 tokens per workgroup on the fp32 matrix cores (head sizes that are
    # multiples of 16 up to 128), or one workgroup per (head, token) for every head size
    gpu.set_tuning(gpu.TUNE_PREFILL_ATTENTION_PER_TOKEN, request.param)
    yield request.param
    gpu.set_tuning(gpu.TUNE_PREFILL_ATTENTION_PER_TOKEN, 0)


def assert_state_matches(m, ref, cfg, n_pos, want_logits, tol=None):
    tol = tol or TOL["model"]
    got = m.logits()
    scale = float(np.abs(want_logits).max())
    err = float(np.abs(got.astype(np.float64) - want_logits).max()) / scale
    assert err <= tol, err
    for layer in range(cfg.n_layers):
        for which, ref_c in ((0, ref.key_cache(layer)), (1, ref.value_cache(layer))):
            want_c = ref_c[:n_pos]
            np.testing.assert_allclose(m.kv_download(layer, which, 0, n_pos), want_c, rtol=0,
                                       atol=tol * np.abs(want_c).max())
    return err


@pytest.mark.parametrize("scheme", ["q8_0", "q4_k", "q6_k", "q4_k_m"])
@pytest.mark.parametrize("model_type", [LlamaModelType.Llama, LlamaModelType.Qwen2])
@pytest.mark.parametrize("n_prompt", [1, 9, 33])
def test_prefill_matches_stepwise_oracle(gpu, attn_mode, scheme, model_type, n_prompt):
    w = synth_llama(MICRO, seed=21, scheme=scheme)
    spice(w, MICRO, 5, biases=model_type == LlamaModelType.Qwen2)
    ref = orc.Llama2(w, rope_variant=model_type)
    toks = W.prompt_tokens(3, n_prompt, MICRO.vocab_size)
    for pos, t in enumerate(toks):
        want = ref.forward(int(t), pos)
    m = Llama2(gpu, MICRO, model_type).load(w)
    m.prefill(toks)
    assert_state_matches(m, ref, MICRO, n_prompt, want)
    # decoding continues from the state the prompt pass left
    nxt = int(np.argmax(want))
    want2 = ref.forward(nxt, n_prompt)
    got2 = m.forward_logits(n_prompt, nxt)
    assert np.abs(got2 - want2).max() <= max(TOL["model"], 1e-3) * np.abs(want2).max()


def test_prefill_in_two_calls_and_in_runs_of_128(gpu, attn_mode):
    cfg = Llama2Config(dim=256, hidden_dim=512, n_layers=2, n_q_heads=4, n_kv_heads=4,
                       vocab_size=320, seq_len=300, rope_base_freq=10000.0, rms_norm_eps=1e-5)
    w = synth_llama(cfg, seed=4, scheme="q4_k_m")
    spice(w, cfg, 6, biases=False)
    ref = orc.Llama2(w)
    toks = W.prompt_tokens(9, 290, cfg.vocab_size)
    for pos, t in enumerate(toks):
        want = ref.forward(int(t), pos)
    m = Llama2(gpu, cfg).load(w)
    m.prefill(toks[:37])  # one call
    m.prefill(toks[37:287], start_pos=37)  # 250 tokens: runs of 128 + 122
    for pos in (287, 288, 289):  # and runs of a single token
        m.prefill(toks[pos:pos + 1], start_pos=pos)
    assert_state_matches(m, ref, cfg, 290, want)


@pytest.mark.parametrize("dim,heads,kv_heads,hidden", [(320, 4, 2, 448), (96, 2, 1, 160), (512, 4, 4, 1024),
                                                       (512, 2, 1, 768)])
def test_prefill_head_sizes_and_partial_chunks(gpu, attn_mode, k_split, dim, heads, kv_heads, hidden):
    # head sizes 80, 48, 128 and 256; row lengths that are not multiples of 64 (Q8_0 only)
    cfg = Llama2Config(dim=dim, hidden_dim=hidden, n_layers=2, n_q_heads=heads, n_kv_heads=kv_heads,
                       vocab_size=300, seq_len=24, rope_base_freq=10000.0, rms_norm_eps=1e-5)
    w = synth_llama(cfg, seed=2, scheme="q8_0")
    spice(w, cfg, 3, biases=True)
    ref = orc.Llama2(w, rope_variant=LlamaModelType.Qwen2)
    toks = W.prompt_tokens(5, 19, cfg.vocab_size)
    for pos, t in enumerate(toks):
        want = ref.forward(int(t), pos)
    m = Llama2(gpu, cfg, LlamaModelType.Qwen2).load(w)
    m.prefill(toks)
    assert_state_matches(m, ref, cfg, 19, want)


def test_prefill_then_greedy_tokens_on_tiny_llama(gpu):
    # the tiny configuration: Q8_0, 16-token seeded prompt, greedy continuation.  The prompt
    # pass rounds operands to f16, so a near-tie between the two best logits may resolve
    # differently: tokens must be identical up to the first step whose top-2 margin in the
    # oracle is below the error bound of the logits (TOL['model'] of their range; with the
    # default split-f16 products that bound is below every margin and all tokens must agree)
    cfg = TINY_LLAMA
    w = synth_llama(cfg, seed=1, scheme="q8_0")
    prompt = W.prompt_tokens(1, 16, cfg.vocab_size)
    n_new = 64
    oracle_model = orc.Llama2(w, predequantize=True)
    want, margins = oracle_model.generate_greedy(prompt, 16 + n_new - 1)
    m = Llama2(gpu, cfg).load(w)
    got = m.prefill_decode_greedy(prompt, n_new)
    want_new, margins_new = want[15:], np.asarray(margins)[15:]
    m.prefill(prompt)
    logit_range = float(np.abs(m.logits()).max())
    risky = np.nonzero(margins_new < TOL["model"] * logit_range)[0]
    upto = int(risky[0]) if risky.size else n_new
    print(f"identical tokens required for the first {upto} of {n_new}; min margin "
          f"{margins_new.min():.3e}, logit range {logit_range:.3e}")
    assert upto >= 8
    assert np.array_equal(got[:upto], want_new[:upto])
    # and the token-by-token device loop gives the same continuation from the same state
    stepwise = m.generate_greedy(prompt, 16 + n_new - 1)[15:]
    assert np.array_equal(got[:upto], stepwise[:upto])


def test_prefill_rejects_bad_arguments(gpu):
    w = synth_llama(MICRO, seed=21, scheme="q8_0")
    m = Llama2(gpu, MICRO).load(w)
    with pytest.raises(W.WgmlError):
        m.prefill([])
    with pytest.raises(W.WgmlError):
        m.prefill([1, 2, MICRO.vocab_size])
    with pytest.raises(W.WgmlError):
        m.prefill([1] * 10, start_pos=MICRO.seq_len - 9)
    # a model whose matrices have no batched product (dense f32 here) is stepped through the
    # prompt token by token instead: same logits as the single steps
    f = Llama2(gpu, MICRO).load(synth_llama(MICRO, seed=21, scheme="f32"))
    f.prefill([1, 2, 3])
    got = f.logits().copy()
    g = Llama2(gpu, MICRO).load(synth_llama(MICRO, seed=21, scheme="f32"))
    for pos, t in enumerate([1, 2, 3]):
        want = g.forward_logits(pos, t)
    assert np.array_equal(got, want)


def test_prefill_steps_through_a_model_with_large_weights(gpu):
    # one matrix whose weights do not fit the batched product: the prompt then goes through the
    # per-token steps, and the state equals the oracle's as for any other model
    w = synth_llama(MICRO, seed=21, scheme="q8_0")
    spice(w, MICRO, 5, biases=False)
    hm = w.layers[1]["ffn_down"]
    vals = orc.dequantize(hm.qtype, hm.data, hm.nrows * hm.ncols).copy()
    vals[7] = 300.0
    w.layers[1]["ffn_down"] = type(hm)(hm.qtype, hm.nrows, hm.ncols, W.quantize(hm.qtype, vals))
    ref = orc.Llama2(w)
    toks = W.prompt_tokens(3, 9, MICRO.vocab_size)
    for pos, t in enumerate(toks):
        want = ref.forward(int(t), pos)
    m = Llama2(gpu, MICRO).load(w)
    m.prefill(toks)
    assert np.isfinite(m.logits()).all()
    assert_state_matches(m, ref, MICRO, 9, want, tol=1e-3)


@pytest.mark.parametrize("qtype", OTHER)
def test_prefill_in_the_remaining_block_formats(gpu, qtype):
    # a model all in one of the six other formats goes through the batched prompt pass too
    from wgml_amd.models import HostMatrix
    w = synth_llama(MICRO, seed=61, scheme="f32")
    for layer in w.layers:
        for name, v in list(layer.items()):
            if isinstance(v, HostMatrix):
                layer[name] = HostMatrix(qtype, v.nrows, v.ncols,
                                         npref.encode_simple(qtype, v.data.view(np.float32)))
    w.output = HostMatrix(qtype, w.output.nrows, w.output.ncols,
                          npref.encode_simple(qtype, w.output.data.view(np.float32)))
    spice(w, MICRO, 9, biases=False)
    ref = orc.Llama2(w)
    toks = W.prompt_tokens(3, 19, MICRO.vocab_size)
    for pos, t in enumerate(toks):
        want = ref.forward(int(t), pos)
    m = Llama2(gpu, MICRO).load(w)
    m.prefill(toks)
    assert m.launches_per_token() < 19 * 5  # batched: far fewer launches than 19 steps
    assert_state_matches(m, ref, MICRO, 19, want)

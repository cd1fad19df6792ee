"""Host-side input makers: ggml reference quantizers and the seeded generator.

The reference contains no quantizer (it only de-quantizes), so these are
pinned by what the formats fix: Q8_0 has a closed form; the K-quants must
round-trip within half a quantization step, respect their field widths, map a
zero block to zero bytes, and be deterministic and thread-count independent.
Parity tests never depend on the quantizer being "right": GPU and oracle always
consume the same bytes.
"""
import numpy as np
import pytest

import npref
import wgml_amd as W


def test_rng_is_counter_based_and_normal():
    a = W.rng_normal(42, 100001, 0.0, 1.0, nthreads=1)
    b = W.rng_normal(42, 100001, 0.0, 1.0, nthreads=7)
    assert np.array_equal(a, b)                       # independent of threading
    assert np.array_equal(a[:1000], W.rng_normal(42, 1000))  # prefix property
    assert not np.array_equal(a[:1000], W.rng_normal(43, 1000))
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1) < 0.02
    assert abs((np.abs(a) < 1).mean() - 0.6827) < 0.01
    t = W.rng_tokens(1, 10000, 32000)
    assert t.max() < 32000 and len(np.unique(t)) > 8000


def test_q8_0_closed_form():
    x = W.rng_normal(1, 32 * 50, 0, 0.02)
    raw = W.quantize(W.Q8_0, x).reshape(-1, 34)
    xb = x.reshape(-1, 32)
    amax = np.abs(xb).max(1)
    d = (amax / np.float32(127)).astype(np.float32)
    assert np.array_equal(raw[:, :2].copy().view(np.float16)[:, 0], d.astype(np.float16))
    inv = np.where(d != 0, np.float32(1) / d, 0).astype(np.float32)
    v = (xb * inv[:, None]).astype(np.float32)
    q = np.where(v >= 0, np.floor(v + 0.5), -np.floor(-v + 0.5)).astype(np.int8)  # roundf
    assert np.array_equal(raw[:, 2:].view(np.int8), q)


@pytest.mark.parametrize("qtype,levels", [(W.Q4_K, 15), (W.Q6_K, 63)])
def test_k_quant_round_trip(qtype, levels):
    n = 256 * 64
    x = W.rng_normal(2 + qtype, n, 0, 0.02)
    raw = W.quantize(qtype, x)
    assert raw.size == W.quant_bytes(qtype, n)
    y = npref.DEQUANT[qtype](raw)
    sub = 32 if qtype == W.Q4_K else 16
    xs, ys = x.reshape(-1, sub), y.reshape(-1, sub)
    rng_ = xs.max(1) - np.minimum(xs.min(1), 0) if qtype == W.Q4_K else 2 * np.abs(xs).max(1)
    step = rng_ / levels
    err = np.abs(xs - ys).max(1)
    # within one step everywhere (the error-minimising scale search may clip the extreme
    # element of a sub-block by more than half a step); the RMS bound below is the tight one
    assert (err <= 1.0 * step + 1e-6).all(), float((err / step).max())
    assert np.sqrt(((x - y) ** 2).mean()) < (0.08 if qtype == W.Q4_K else 0.02) * x.std()
    # deterministic and independent of the thread count
    assert np.array_equal(raw, W.quantize(qtype, x, nthreads=1))
    assert np.array_equal(raw, W.quantize(qtype, x, nthreads=5))


def test_q4_k_field_widths_and_zero_block():
    x = np.zeros(512, dtype=np.float32)
    for qtype in (W.Q4_K, W.Q6_K, W.Q8_0):
        assert not W.quantize(qtype, x).any()
        assert not npref.DEQUANT[qtype](W.quantize(qtype, x)).any()
    raw = W.quantize(W.Q4_K, W.rng_normal(9, 256 * 8, 0, 1.0)).reshape(-1, 144)
    sc, m = npref._scale_min_k4(raw[:, 4:16])
    assert sc.max() <= 63 and m.max() <= 63 and sc.max() == 63  # the largest scale maps to 63


def test_quantize_errors():
    with pytest.raises(W.WgmlError):
        W.quantize(W.Q4_K, np.zeros(100, dtype=np.float32))   # not a whole block
    with pytest.raises(W.WgmlError):
        W.quantize(2, np.zeros(32, dtype=np.float32))         # Q4_0: outside this path
    assert W.quant_bytes(W.Q8_0, 4096 * 11008) == 47906816
    assert W.quant_bytes(W.Q4_K, 4096 * 11008) == 25362432
    assert W.quant_bytes(W.Q6_K, 4096 * 11008) == 36986880


@pytest.mark.parametrize("qtype", [1, 2, 3, 6, 7, 8, 12, 13, 14, 15])
def test_dequantize_host_matches_oracle(qtype):
    # Block*::dequantize on the host (what the reference does for tensors it keeps in f32)
    import npref
    import oracle as orc
    nb = 300
    raw = npref.random_blocks(qtype, nb, seed=40 + qtype)
    n = nb * npref.BLOCK_ELEMS[qtype]
    got = W.dequantize_host(qtype, raw, n)
    want = orc.dequantize(qtype, raw, n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    with pytest.raises(W.WgmlError):
        W.dequantize_host(10, raw, 256)  # Q2_K: unsupported

"""GPU parity: the batched matrix product and the batched prompt pass ("prefill").

The reference has neither: it runs the prompt through its batch-1 step token by token
(wgml-chat/src/chat_llama2.rs:155-228).  The batched path is therefore held against that
sequence -- the oracle's N single-token steps on the same quantized bytes.

Tolerance: the batched products take f16 operands (weights dequantized with the reference's
arithmetic, then rounded; activations rounded) with fp32 sums, so a product's error is about
2^-11 / sqrt(3) per term, random in sign: ~3e-4 of rms(ref) observed.  The bound used is
|gpu - ref| <= 1e-3 * |ref| + 2e-3 * rms(ref) for products and 3e-3 * max|ref| for logits and
cache rows after a whole model pass.
"""
import numpy as np
import pytest

import oracle as orc
import wgml_amd as W

pytestmark = pytest.mark.gpu
QT = [W.Q8_0, W.Q4_K, W.Q6_K]


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
    assert (err <= 1e-3 * np.abs(ref) + 2e-3 * rms).all(), float(err.max() / rms)
    return float(err.max() / rms)


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("T", [1, 5, 16, 17, 37, 64, 100, 128])
@pytest.mark.parametrize("nrows,ncols", [(16, 256), (5, 512), (100, 768), (333, 2048)])
def test_gemm_matches_dequantized_product(gpu, qtype, T, nrows, ncols):
    raw = W.quantize(qtype, W.rng_normal(10 + nrows, nrows * ncols, 0, 0.02))
    x = W.rng_normal(20 + T, T * ncols).reshape(T, ncols)
    check(gemm(gpu, qtype, raw, nrows, ncols, x), reference(qtype, raw, nrows, ncols, x))


@pytest.mark.parametrize("ncols", [32, 96, 160, 2080])
@pytest.mark.parametrize("T", [3, 40])
def test_gemm_q8_0_rows_not_a_multiple_of_64(gpu, ncols, T):
    nrows = 21
    raw = W.quantize(W.Q8_0, W.rng_normal(3, nrows * ncols, 0, 0.02))
    x = W.rng_normal(4, T * ncols).reshape(T, ncols)
    check(gemm(gpu, W.Q8_0, raw, nrows, ncols, x), reference(W.Q8_0, raw, nrows, ncols, x))


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
        check(got[t:t + 1], out.read().astype(np.float64)[None])


@pytest.mark.parametrize("qtype", QT)
def test_gemm_large_activations_stay_finite(gpu, qtype):
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

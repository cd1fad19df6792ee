"""GPU parity: quantized GEMV (GemvQuant) and dense f32 GEMV against the oracle.

Tolerance (stated by the task): relative 1e-3 with fp32 accumulation.  It is
applied as |gpu - ref| <= 1e-3 * |ref| + 1e-3 * rms(ref), with ref the float64
dot product of the bit-exact dequantized weights; the observed error is
typically 1e-6 * rms.  The reference has no numerical GEMV test of its own
(only a shader-compilation check, crates/wgml/src/ops/gemv_quant.rs:350).
"""
import numpy as np
import pytest

import npref
import oracle as orc
import wgml_amd as W

pytestmark = pytest.mark.gpu
QT = [W.Q8_0, W.Q4_K, W.Q6_K]

# Two GEMV implementations sit behind the same entry point: the default integer-dot path
# (activations staged as 16-bit block fixed point, rounding <= 2^-16 of a block's maximum) and
# the fp32-activation path.  Observed error / rms(ref): ~3e-5 and ~1e-6 respectively.
MODES = {"int_dot": 5e-4, "f32_act": 1e-4}


@pytest.fixture(params=list(MODES))
def mode(request, gpu):
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 1 if request.param == "f32_act" else 0)
    yield request.param
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 0)


def close(got, ref):
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt((ref ** 2).mean())) or 1.0
    err = np.abs(got.astype(np.float64) - ref)
    ok = err <= 1e-3 * np.abs(ref) + 1e-3 * rms
    return bool(ok.all()), float(err.max() / rms)


def gemv(gpu, qtype, raw, nrows, ncols, x):
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    xv = W.GpuVector.init(gpu, x)
    out = W.GpuVector.init(gpu, np.full(nrows, np.nan, dtype=np.float32))
    W.GemvQuant.from_device(gpu).dispatch(out, m, xv)
    return out.read()


def weights(qtype, nrows, ncols, seed):
    return W.quantize(qtype, W.rng_normal(seed, nrows * ncols, 0, 0.02))


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("nrows,ncols", [(4, 256), (8, 512), (1, 256), (5, 768), (13, 2304),
                                         (33, 4096), (260, 11008), (7, 14336)])
def test_gemv_small_and_ragged(gpu, mode, qtype, nrows, ncols):
    raw = weights(qtype, nrows, ncols, 100 + nrows)
    x = W.rng_normal(200 + ncols, ncols)
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    ok, e = close(gemv(gpu, qtype, raw, nrows, ncols, x), ref)
    assert ok, e
    assert e < MODES[mode], e


@pytest.mark.parametrize("ncols", [32, 288, 96])
def test_gemv_q8_0_unpaired_block_counts(gpu, mode, ncols):
    # the reference needs ncols % 64 == 0 (% 128 in its kernel) and otherwise falls back to f32
    # (gguf.rs:146-159); the tiny Llama has 288 columns = 9 blocks
    nrows = 50
    raw = weights(W.Q8_0, nrows, ncols, 3)
    x = W.rng_normal(4, ncols)
    _, ref = orc.gemv_quant(W.Q8_0, raw, nrows, ncols, x)
    ok, e = close(gemv(gpu, W.Q8_0, raw, nrows, ncols, x), ref)
    assert ok, e


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("r", [1, 2])
@pytest.mark.parametrize("depth", [0, 2])
def test_gemv_rows_per_wave_variants(gpu, mode, qtype, r, depth):
    nrows, ncols = 1030, 1024  # not a multiple of rows-per-workgroup
    raw = weights(qtype, nrows, ncols, 8)
    x = W.rng_normal(9, ncols)
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    gpu.set_tuning(gpu.TUNE_GEMV_ROWS_PER_WAVE, r)
    gpu.set_tuning(gpu.TUNE_GEMV_DEPTH, depth)
    try:
        ok, e = close(gemv(gpu, qtype, raw, nrows, ncols, x), ref)
        # tall and short: many rows per wave (pipelined rounds) and fewer rows than waves
        for nr in (40000, 24):
            raw2 = weights(qtype, nr, 256, 11)
            x2 = W.rng_normal(12, 256)
            _, ref2 = orc.gemv_quant(qtype, raw2, nr, 256, x2)
            ok2, e2 = close(gemv(gpu, qtype, raw2, nr, 256, x2), ref2)
            assert ok2, (nr, e2)
    finally:
        gpu.set_tuning(gpu.TUNE_GEMV_ROWS_PER_WAVE, 0)
        gpu.set_tuning(gpu.TUNE_GEMV_DEPTH, 0)
    assert ok, e


@pytest.mark.parametrize("qtype", QT)
def test_gemv_one_hot_gives_dequantized_column(gpu, mode, qtype):
    nrows, ncols = 16, 512
    be = npref.BLOCK_ELEMS[qtype]
    raw = npref.random_blocks(qtype, nrows * ncols // be, seed=5)
    deq = orc.dequantize(qtype, raw, nrows * ncols).reshape(nrows, ncols)
    for j in (0, 31, 32, 100, 255, 256, 511):
        x = np.zeros(ncols, dtype=np.float32)
        x[j] = 1.0
        got = gemv(gpu, qtype, raw, nrows, ncols, x)
        # same value up to the rounding of the regrouped scale arithmetic (and, on the
        # integer-dot path, of 1.0 in 16-bit block fixed point: 32512/32512 exactly)
        np.testing.assert_allclose(got, deq[:, j], rtol=4e-6, atol=1e-6 * np.abs(deq[:, j]).max())


@pytest.mark.parametrize("qtype", QT)
def test_gemv_random_block_bits(gpu, mode, qtype):
    # wgml-bench feeds random raw bits (gemv_quant.rs:83-101): every scale/min pattern occurs
    nrows, ncols = 64, 1024
    raw = npref.random_blocks(qtype, nrows * ncols // npref.BLOCK_ELEMS[qtype], seed=21)
    x = W.rng_normal(22, ncols)
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    ok, e = close(gemv(gpu, qtype, raw, nrows, ncols, x), ref)
    assert ok, e


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("nrows,ncols", [(4096, 4096), (11008, 4096), (4096, 11008),
                                         (32000, 4096)])
def test_gemv_benchmark_shapes(gpu, mode, qtype, nrows, ncols):
    raw = weights(qtype, nrows, ncols, 1000 + qtype)
    x = W.rng_normal(31, ncols)
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    op = W.GemvQuant.from_device(gpu)
    xv, out = W.GpuVector.init(gpu, x), W.GpuVector.uninit(gpu, nrows)
    op.dispatch(out, m, xv)
    got = out.read()
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    ok, e = close(got, ref)
    assert ok, e
    # linearity at full size: M(2x - 3y) = 2 Mx - 3 My
    y = W.rng_normal(32, ncols)
    yv = W.GpuVector.init(gpu, y)
    zv = W.GpuVector.init(gpu, 2 * x - 3 * y)
    oy, oz = W.GpuVector.uninit(gpu, nrows), W.GpuVector.uninit(gpu, nrows)
    op.dispatch(oy, m, yv)
    op.dispatch(oz, m, zv)
    ok, e = close(oz.read(), 2.0 * got.astype(np.float64) - 3.0 * oy.read().astype(np.float64))
    assert ok, e
    # repeatable bit for bit (fixed reduction order)
    op.dispatch(oy, m, xv)
    assert np.array_equal(oy.read(), got)


def test_gemv_output_into_view(gpu):
    # the K/V GEMVs write straight into a cache column (models/llama2/transformer.rs:326-341)
    nrows, ncols = 64, 256
    raw = weights(W.Q8_0, nrows, ncols, 1)
    x = W.rng_normal(2, ncols)
    cache = W.GpuMatrix(gpu, nrows, 8)
    cache.write(np.zeros(nrows * 8, dtype=np.float32))
    m = W.GpuQuantMatrix(gpu, W.Q8_0, nrows, ncols, raw)
    W.GemvQuant.from_device(gpu).dispatch(cache.column(3), m, W.GpuVector.init(gpu, x))
    full = cache.read().reshape(8, nrows)
    _, ref = orc.gemv_quant(W.Q8_0, raw, nrows, ncols, x)
    assert close(full[3], ref)[0]
    assert not full[[0, 1, 2, 4, 5, 6, 7]].any()


def test_gemv_f32_matrix_and_dense_op(gpu):
    rng = np.random.default_rng(0)
    nrows, ncols = 37, 288
    a = rng.standard_normal((nrows, ncols)).astype(np.float32)
    x = rng.standard_normal(ncols).astype(np.float32)
    ref = orc.gemv_f64(a, x)
    assert close(gemv(gpu, W.F32, a.view(np.uint8), nrows, ncols, x), ref)[0]
    g = W.Gemv.from_device(gpu)
    av, xv, out = W.GpuVector.init(gpu, a), W.GpuVector.init(gpu, x), W.GpuVector.uninit(gpu, nrows)
    g.dispatch(out, av, nrows, ncols, xv)
    assert close(out.read(), ref)[0]
    # transposed (GemvTr): out = A^T v
    v = rng.standard_normal(nrows).astype(np.float32)
    out_t = W.GpuVector.uninit(gpu, ncols)
    g.dispatch(out_t, av, nrows, ncols, W.GpuVector.init(gpu, v), transposed=True)
    assert close(out_t.read(), a.astype(np.float64).T @ v.astype(np.float64))[0]


def test_gemv_dimension_mismatch(gpu):
    raw = weights(W.Q8_0, 8, 64, 1)
    m = W.GpuQuantMatrix(gpu, W.Q8_0, 8, 64, raw)
    op = W.GemvQuant.from_device(gpu)
    with pytest.raises(W.WgmlError, match="dimension mismatch"):
        op.dispatch(W.GpuVector.uninit(gpu, 8), m, W.GpuVector.uninit(gpu, 32))
    with pytest.raises(W.WgmlError, match="dimension mismatch"):
        op.dispatch(W.GpuVector.uninit(gpu, 4), m, W.GpuVector.uninit(gpu, 64))


@pytest.mark.parametrize("qtype,nrows,ncols", [(W.Q8_0, 300000, 64), (W.Q4_K, 270000, 256),
                                               (W.Q6_K, 135001, 256)])
def test_gemv_more_than_64_rows_per_wave(gpu, qtype, nrows, ncols):
    # tall matrices: a wave owns more rows than it has lanes to park results in, so its rows
    # are handled in several segments with the epilogue in between
    raw = weights(qtype, nrows, ncols, 77)
    x = W.rng_normal(78, ncols)
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    ok, e = close(gemv(gpu, qtype, raw, nrows, ncols, x), ref)
    assert ok, e


@pytest.mark.parametrize("nrows,ncols", [(140000, 256), (1001, 512), (11008, 4096)])
def test_fused_gate_up_silu_launch(gpu, nrows, ncols):
    # the decoder's fused gate/up launch on its own (through the benchmark entry point, one
    # launch): out = up * silu(gate) with the RMSNorm of x folded in.  140000 rows make a wave
    # own more than 32 (gate, up) pairs, i.e. several segments.
    import ctypes as C

    from wgml_amd._lib import call

    gate_raw, up_raw = weights(W.Q4_K, nrows, ncols, 5), weights(W.Q4_K, nrows, ncols, 6)
    x = W.rng_normal(7, ncols)
    nw = (1.0 + 0.1 * W.rng_normal(8, ncols)).astype(np.float32)
    gate = W.GpuQuantMatrix(gpu, W.Q4_K, nrows, ncols, gate_raw)
    up = W.GpuQuantMatrix(gpu, W.Q4_K, nrows, ncols, up_raw)
    out = W.GpuVector.init(gpu, np.full(nrows, np.nan, dtype=np.float32))
    xv, nwv = W.GpuVector.init(gpu, x), W.GpuVector.init(gpu, nw)
    a, b = (C.c_void_p * 1)(gate.handle), (C.c_void_p * 1)(up.handle)
    modes, ms, nview = (C.c_int * 1)(2), C.c_float(), nwv.view()
    call("wgml_bench_gemv_fused", gpu.handle, a, b, modes, 1, 1, out.view(), nrows, xv.view(),
         C.byref(nview), 1, C.byref(ms))
    xn = orc.rms_norm(x, nw, 1e-5)
    _, g = orc.gemv_quant(W.Q4_K, gate_raw, nrows, ncols, xn)
    _, u = orc.gemv_quant(W.Q4_K, up_raw, nrows, ncols, xn)
    ref = u * (g / (1.0 + np.exp(-g)))
    ok, e = close(out.read(), ref)
    assert ok, e


OTHER = [W.Q4_0, W.Q4_1, W.Q5_0, W.Q5_1, W.Q5_K, W.Q8_K]


@pytest.mark.parametrize("qtype", QT + OTHER)
@pytest.mark.parametrize("nrows", [1, 3, 9, 15])
@pytest.mark.parametrize("ncols", [256, 1024, 8192])
def test_gemv_fewer_rows_than_waves(gpu, qtype, nrows, ncols):
    # Workgroups of 8 or 16 waves, fewer rows than that: the waves without a row either stage a
    # share of x and wait at the barrier, or (no share either: 256 columns need one staging wave
    # in four, 8192 all of them) end before it.  The barrier counts only waves that are still
    # running (a terminated wave is not waited for on this hardware), which this case relies on.
    be = npref.BLOCK_ELEMS[qtype]
    raw = npref.random_blocks(qtype, nrows * ncols // be, seed=500 + qtype + nrows)
    x = W.rng_normal(600 + ncols, ncols)
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    ok, e = close(gemv(gpu, qtype, raw, nrows, ncols, x), ref)
    assert ok, e


@pytest.mark.parametrize("qtype", QT)
@pytest.mark.parametrize("nrows", [1, 2, 7])
def test_fused_launch_with_fewer_row_pairs_than_waves(gpu, qtype, nrows):
    # the multi-matrix launch with so few (gate, up) pairs that most waves of its one
    # workgroup have none
    import ctypes as C

    from wgml_amd._lib import call

    ncols = 512
    gate_raw, up_raw = weights(qtype, nrows, ncols, 15), weights(qtype, nrows, ncols, 16)
    x = W.rng_normal(17, ncols)
    gate = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, gate_raw)
    up = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, up_raw)
    out = W.GpuVector.init(gpu, np.full(nrows, np.nan, dtype=np.float32))
    xv = W.GpuVector.init(gpu, x)
    a, b = (C.c_void_p * 1)(gate.handle), (C.c_void_p * 1)(up.handle)
    modes, ms = (C.c_int * 1)(2), C.c_float()
    call("wgml_bench_gemv_fused", gpu.handle, a, b, modes, 1, 1, out.view(), nrows, xv.view(), None, 1,
         C.byref(ms))
    _, g = orc.gemv_quant(qtype, gate_raw, nrows, ncols, x)
    _, u = orc.gemv_quant(qtype, up_raw, nrows, ncols, x)
    ok, e = close(out.read(), u * (g / (1.0 + np.exp(-g))))
    assert ok, e


@pytest.mark.parametrize("qtype", OTHER)
@pytest.mark.parametrize("nrows,ncols", [(4, 256), (1, 512), (37, 768), (33, 4096), (260, 11008),
                                         (4096, 4096), (7, 14336)])
def test_gemv_remaining_block_formats(gpu, qtype, nrows, ncols):
    # the formats the reference's to_gpu_matrix also keeps quantized (gguf.rs:172-182), random
    # block bits with finite scales: result against the float64 dot product of the bit-exact
    # dequantized weights
    be = npref.BLOCK_ELEMS[qtype]
    raw = npref.random_blocks(qtype, nrows * ncols // be, seed=3000 + qtype + nrows)
    x = W.rng_normal(4000 + ncols, ncols)
    _, ref = orc.gemv_quant(qtype, raw, nrows, ncols, x)
    ok, e = close(gemv(gpu, qtype, raw, nrows, ncols, x), ref)
    assert ok, e


@pytest.mark.parametrize("qtype", OTHER)
def test_gemv_remaining_formats_all_ones_vector_sums_rows(gpu, qtype):
    # x = 1 is exact in the block fixed-point staging, so the result is the row sum of the
    # dequantized weights up to fp32 rounding of the per-block scaling
    be = npref.BLOCK_ELEMS[qtype]
    nrows, ncols = 8, 1024
    raw = npref.random_blocks(qtype, nrows * ncols // be, seed=77)
    w = orc.dequantize(qtype, raw, nrows * ncols).reshape(nrows, ncols).astype(np.float64)
    x = np.ones(ncols, np.float32)
    got = gemv(gpu, qtype, raw, nrows, ncols, x)
    np.testing.assert_allclose(got, w.sum(axis=1), rtol=2e-5, atol=2e-5 * np.abs(w).sum(axis=1).max())


def _fused(gpu, mats, partner, modes, nrows, x, norm_w=None):
    """One fused launch through the benchmark entry point; returns the concatenated outputs."""
    import ctypes as C

    from wgml_amd._lib import call

    nj = len(mats)
    out = W.GpuVector.init(gpu, np.full(nj * nrows, np.nan, dtype=np.float32))
    xv = W.GpuVector.init(gpu, x)
    a = (C.c_void_p * nj)(*[m.handle for m in mats])
    b = (C.c_void_p * nj)(*[(p.handle if p is not None else None) for p in partner]) if any(partner) else None
    ms = C.c_float()
    nwv = None
    if norm_w is not None:
        nwv = W.GpuVector.init(gpu, norm_w)
        view = nwv.view()
    call("wgml_bench_gemv_fused", gpu.handle, a, b, (C.c_int * nj)(*modes), nj, 1, out.view(), nrows,
         xv.view(), C.byref(view) if norm_w is not None else None, 1, C.byref(ms))
    return out.read().reshape(nj, nrows)


def _rope0(v):
    return v  # rotation at position 0 is the identity


@pytest.mark.parametrize("qtype", QT + OTHER)
@pytest.mark.parametrize("ncols", [512, 4096, 8192])
def test_fused_launches_in_every_format(gpu, mode, qtype, ncols):
    # Q/K/V-like (two rotated matrices + a plain one; position 0, so the rotation is the identity)
    # and gate/up-like launches with all matrices in one format, for the nine quantized formats
    # on the integer-dot path and the three main ones with fp32 activations
    if mode == "f32_act" and qtype in OTHER:
        pytest.skip("fp32 activations exist for Q8_0 / Q4_K / Q6_K")
    nrows = 96
    be = npref.BLOCK_ELEMS[qtype]
    raws = [npref.random_blocks(qtype, nrows * ncols // be, seed=700 + qtype + i) for i in range(3)]
    mats = [W.GpuQuantMatrix(gpu, qtype, nrows, ncols, r) for r in raws]
    x = W.rng_normal(800 + ncols, ncols)
    nw = (1.0 + 0.1 * W.rng_normal(801, ncols)).astype(np.float32)
    xn = orc.rms_norm(x, nw, 1e-5)
    refs = [orc.gemv_quant(qtype, r, nrows, ncols, xn)[1] for r in raws]
    got = _fused(gpu, mats, [None] * 3, [1, 1, 0], nrows, x, nw)
    for i in range(3):
        ok, e = close(got[i], refs[i])
        assert ok, (i, e)
    got = _fused(gpu, mats[:1], mats[1:2], [2], nrows, x, nw)
    g, u = refs[0], refs[1]
    ok, e = close(got[0], u * (g / (1.0 + np.exp(-g))))
    assert ok, e


def test_fused_launch_refuses_a_mix_with_the_other_formats(gpu):
    nrows, ncols = 32, 512
    a = W.GpuQuantMatrix(gpu, W.Q4_K, nrows, ncols, weights(W.Q4_K, nrows, ncols, 1))
    b = W.GpuQuantMatrix(gpu, W.Q5_K, nrows, ncols,
                         npref.random_blocks(W.Q5_K, nrows * ncols // 256, seed=2))
    with pytest.raises(W.WgmlError):
        _fused(gpu, [a, b], [None, None], [0, 0], nrows, W.rng_normal(3, ncols))


def test_bench_read_chain_runs_and_checks_its_arguments(gpu):
    # the bare chain of read-only launches that prices the machine (bench.py --ceiling):
    # a time comes back for both ways of launching; sizes beyond half its pool are refused
    import ctypes as C

    from wgml_amd._lib import call

    ms = C.c_float(-1.0)
    for use_graph in (0, 1):
        call("wgml_bench_read_chain", gpu.handle, 4096, 8, use_graph, C.byref(ms))
        assert 0 < ms.value < 50.0
    with pytest.raises(W.WgmlError):
        call("wgml_bench_read_chain", gpu.handle, 400000, 8, 0, C.byref(ms))
    with pytest.raises(W.WgmlError):
        call("wgml_bench_read_chain", gpu.handle, 0, 8, 0, C.byref(ms))


def test_context_stream_handle(gpu):
    # the stream every call of the context enqueues on: a stable, non-null handle
    assert gpu.stream() != 0
    assert gpu.stream() == gpu.stream()

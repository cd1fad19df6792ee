"""GPU parity: KV-cache attention against the oracle's restatement of
BatchedMultiqueryAttention::run_cpu.  Shapes follow the reference tests
(crates/wgml/src/ops/batched_multiquery_attention.rs:210-413: seq 1024, kv_dim
768, 12 heads x 64, pos 0..8, epsilon 1e-5) plus the grouped-query and
long-context cases of the benchmark configurations."""
import numpy as np
import pytest

import npref
import oracle as orc
import wgml_amd as W

pytestmark = pytest.mark.gpu


def rnd(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def run(gpu, seq_len, kv_mul, n_heads, hs, pos, with_att, seed=0):
    kv_dim = n_heads // kv_mul * hs
    q = rnd(n_heads * hs, seed + 1)
    kc, vc = rnd(seq_len * kv_dim, seed + 2), rnd(seq_len * kv_dim, seed + 3)
    p = W.BatchedMultiqueryAttentionParams(seq_len, kv_dim, kv_mul, n_heads, hs, pos)
    gq, gk, gv = (W.GpuVector.init(gpu, a) for a in (q, kc, vc))
    att = W.GpuVector.init(gpu, np.zeros(seq_len * n_heads, dtype=np.float32)) if with_att else None
    xb = W.GpuVector.init(gpu, np.full(n_heads * hs, np.nan, dtype=np.float32))
    W.BatchedMultiqueryAttention.from_device(gpu).dispatch(p, gq, gk, gv, att, xb)
    want_xb, want_att = orc.attention(seq_len, kv_dim, kv_mul, n_heads, hs, pos, q, kc, vc)
    got_att = att.read().reshape(n_heads, seq_len) if with_att else None
    return xb.read(), want_xb, got_att, want_att


@pytest.mark.parametrize("pos", list(range(9)))
def test_attention_reference_shape_with_weights(gpu, pos):  # `gpu_attention`: xb and att
    xb, wxb, att, watt = run(gpu, 1024, 1, 12, 64, pos, True)
    np.testing.assert_allclose(xb, wxb, rtol=0, atol=1e-5)
    np.testing.assert_allclose(att[:, :pos + 1], watt[:, :pos + 1], rtol=0, atol=1e-5)
    assert not att[:, pos + 1:].any()  # nothing written past pos


@pytest.mark.parametrize("pos", [0, 1, 8, 63, 64, 100, 1023])
def test_attention_multi(gpu, pos):  # `gpu_attention_multi`: xb only
    xb, wxb, _, _ = run(gpu, 1024, 1, 12, 64, pos, False)
    np.testing.assert_allclose(xb, wxb, rtol=0, atol=1e-5)


@pytest.mark.parametrize("kv_mul,n_heads,hs", [(4, 32, 128), (2, 8, 64), (8, 16, 128), (3, 6, 32),
                                               (1, 6, 48), (1, 32, 128), (1, 2, 256), (6, 12, 128)])
@pytest.mark.parametrize("pos", [5, 383])
def test_attention_grouped_and_head_sizes(gpu, kv_mul, n_heads, hs, pos):
    xb, wxb, _, _ = run(gpu, 512, kv_mul, n_heads, hs, pos, False, seed=kv_mul)
    np.testing.assert_allclose(xb, wxb, rtol=0, atol=2e-5)


@pytest.mark.parametrize("with_att", [False, True])
def test_attention_long_context_gqa(gpu, with_att):
    # Llama-3-8B-like head layout at a long position: many workgroups per KV head + merge
    xb, wxb, att, watt = run(gpu, 8448, 4, 32, 128, 8300, with_att, seed=9)
    np.testing.assert_allclose(xb, wxb, rtol=0, atol=2e-5)
    if with_att:
        np.testing.assert_allclose(att[:, :8301], watt[:, :8301], rtol=0, atol=1e-6)


@pytest.mark.parametrize("wide,splits", [(1024, 0), (0, 2), (0, 5), (0, 16), (0, 17), (0, 64)])
@pytest.mark.parametrize("pos", [3, 140, 700])
def test_attention_plans_agree(gpu, wide, splits, pos):
    # every way of sharing a head's positions out over workgroups (one workgroup per head; 2..64
    # workgroups with a merge of 16 or 64 partials at a time, most of them without a position
    # at a short context) gives the oracle's result
    gpu.set_tuning(gpu.TUNE_ATTN_WIDE_POSITIONS, wide)
    gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, splits)
    try:
        xb, wxb, _, _ = run(gpu, 1024, 2, 8, 128, pos, False, seed=3)
    finally:
        gpu.set_tuning(gpu.TUNE_ATTN_WIDE_POSITIONS, 0)
        gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, 0)
    np.testing.assert_allclose(xb, wxb, rtol=0, atol=2e-5)


@pytest.fixture(params=["merge_launch", "merged_by_product"])
def fold(gpu, request):
    """Both ways the pair runs: attention's own merge launch (the default), and the product
    merging the partial results while it stages its input."""
    gpu.set_tuning(gpu.TUNE_ATTN_MERGE, 1 if request.param == "merged_by_product" else 0)
    yield request.param
    gpu.set_tuning(gpu.TUNE_ATTN_MERGE, 0)


def run_with_projection(gpu, qtype, seq_len, kv_mul, n_heads, hs, pos, nrows, accumulate, seed=0):
    """attention + output projection as one call, against the oracle's attention followed by the
    exact product of the dequantized matrix with it (f64)."""
    kv_dim = n_heads // kv_mul * hs
    dim = n_heads * hs
    q = rnd(dim, seed + 1)
    kc, vc = rnd(seq_len * kv_dim, seed + 2), rnd(seq_len * kv_dim, seed + 3)
    vals = rnd(nrows * dim, seed + 4, 0.02)
    if qtype == W.F32:
        raw, w = vals.view(np.uint8), vals
    elif qtype in (W.Q8_0, W.Q4_K, W.Q6_K):
        raw = W.quantize(qtype, vals)
        w = orc.dequantize(qtype, raw, nrows * dim)
    else:  # no quantizer for these: random blocks with finite scales
        raw = npref.random_blocks(qtype, nrows * dim // npref.BLOCK_ELEMS[qtype], seed=seed + 4)
        w = orc.dequantize(qtype, raw, nrows * dim)
    m = W.GpuQuantMatrix(gpu, qtype, nrows, dim, raw)
    p = W.BatchedMultiqueryAttentionParams(seq_len, kv_dim, kv_mul, n_heads, hs, pos)
    gq, gk, gv = (W.GpuVector.init(gpu, a) for a in (q, kc, vc))
    xb = W.GpuVector.init(gpu, np.full(dim, np.nan, dtype=np.float32))
    out0 = rnd(nrows, seed + 5)
    out = W.GpuVector.init(gpu, out0)
    W.BatchedMultiqueryAttention.from_device(gpu).dispatch_with_projection(p, gq, gk, gv, xb, m, out,
                                                                            accumulate)
    want_xb, _ = orc.attention(seq_len, kv_dim, kv_mul, n_heads, hs, pos, q, kc, vc)
    want = w.reshape(nrows, dim).astype(np.float64) @ want_xb.astype(np.float64)
    if accumulate:
        want = want + out0
    return out.read(), want


@pytest.mark.parametrize("qtype", [W.Q4_K, W.Q6_K, W.Q8_0])
@pytest.mark.parametrize("pos", [0, 3, 31, 140, 255, 256, 700, 1023])
def test_attention_with_projection(gpu, fold, qtype, pos):
    # with `fold` the product merges attention's per-workgroup partial results while it stages
    # its input (2 to 16 partial results per head, depending on the position; at the first
    # positions most of them are neutral); GEMV tolerance as in tests/test_gpu_gemv.py
    got, want = run_with_projection(gpu, qtype, 1024, 1, 8, 128, pos, 192, False, seed=pos)
    assert np.abs(got - want).max() <= 5e-4 * np.abs(want).max()


@pytest.mark.parametrize("kv_mul,n_heads,hs", [(4, 32, 128), (2, 8, 64), (1, 12, 64), (1, 6, 48), (8, 16, 128),
                                               (1, 2, 256)])
@pytest.mark.parametrize("pos", [5, 383])
def test_attention_with_projection_head_layouts(gpu, fold, kv_mul, n_heads, hs, pos):
    # grouped queries, head sizes that fill a lane group only partly (48) and that need the
    # four-wave kernel (256), accumulation into the output
    dim = n_heads * hs
    qtype = W.Q8_0 if dim % 256 else W.Q4_K
    got, want = run_with_projection(gpu, qtype, 512, kv_mul, n_heads, hs, pos, 96, True, seed=kv_mul)
    assert np.abs(got - want).max() <= 5e-4 * np.abs(want).max()


@pytest.mark.parametrize("wide,splits", [(1024, 0), (0, 2), (0, 8), (0, 9), (0, 16), (0, 17), (0, 64)])
def test_attention_with_projection_plans(gpu, fold, wide, splits):
    # forced plans: one workgroup per head (nothing to merge), 2..16 partial results merged by the
    # product (eight at a time), 17 and 64 through the merge launch
    gpu.set_tuning(gpu.TUNE_ATTN_WIDE_POSITIONS, wide)
    gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, splits)
    try:
        for pos in (3, 140, 700):
            got, want = run_with_projection(gpu, W.Q4_K, 1024, 2, 8, 128, pos, 128, True, seed=3)
            assert np.abs(got - want).max() <= 5e-4 * np.abs(want).max(), pos
    finally:
        gpu.set_tuning(gpu.TUNE_ATTN_WIDE_POSITIONS, 0)
        gpu.set_tuning(gpu.TUNE_ATTN_SPLITS, 0)


@pytest.mark.parametrize("qtype", [W.F32, W.Q5_K, W.Q4_0])
def test_attention_with_projection_other_formats(gpu, fold, qtype):
    # formats without a merging product: the two launches run as they would on their own
    got, want = run_with_projection(gpu, qtype, 256, 1, 4, 64, 77, 64, True, seed=11)
    assert np.abs(got - want).max() <= 5e-4 * np.abs(want).max()


def test_attention_with_projection_fp32_activations(gpu, fold):
    gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 1)
    try:
        got, want = run_with_projection(gpu, W.Q4_K, 512, 1, 8, 128, 300, 64, False, seed=2)
    finally:
        gpu.set_tuning(gpu.TUNE_GEMV_F32_ACTIVATIONS, 0)
    assert np.abs(got - want).max() <= 1e-4 * np.abs(want).max()


def test_attention_with_projection_argument_checks(gpu):
    a = W.BatchedMultiqueryAttention.from_device(gpu)
    raw = W.quantize(W.Q8_0, rnd(32 * 128, 1, 0.02))
    m = W.GpuQuantMatrix(gpu, W.Q8_0, 32, 128, raw)
    v = W.GpuVector.uninit(gpu, 4096)
    p = W.BatchedMultiqueryAttentionParams(16, 128, 1, 2, 64, 3)
    with pytest.raises(W.WgmlError):  # out does not have the matrix's rows
        a.dispatch_with_projection(p, v.rows(0, 128), v.rows(0, 2048), v.rows(0, 2048), v.rows(0, 128), m,
                                   v.rows(0, 31))
    bad = W.BatchedMultiqueryAttentionParams(16, 64, 1, 1, 64, 3)
    with pytest.raises(W.WgmlError):  # attention output shorter than the matrix's columns
        a.dispatch_with_projection(bad, v.rows(0, 64), v.rows(0, 1024), v.rows(0, 1024), v.rows(0, 64), m,
                                   v.rows(0, 32))


def test_bench_attention_runs_and_checks_its_arguments(gpu):
    import ctypes as C

    from wgml_amd._lib import AttnParams, View, call

    seq_len, kv_mul, n_heads, hs, pos = 512, 2, 8, 64, 300
    kv_dim = n_heads // kv_mul * hs
    q = W.GpuVector.init(gpu, rnd(n_heads * hs, 1))
    ks = [W.GpuVector.init(gpu, rnd(seq_len * kv_dim, 2 + i)) for i in range(2)]
    vs = [W.GpuVector.init(gpu, rnd(seq_len * kv_dim, 5 + i)) for i in range(2)]
    xb = W.GpuVector.uninit(gpu, n_heads * hs)
    kv = (View * 2)(*[k.view() for k in ks])
    vv = (View * 2)(*[v.view() for v in vs])
    p = AttnParams(seq_len, kv_dim, kv_mul, n_heads, hs, pos)
    ms = C.c_float(-1.0)
    # 5 launches: the last one reads cache set 0, and leaves its result in xb
    call("wgml_bench_attention", gpu.handle, C.byref(p), 512, q.view(), kv, vv, 2, xb.view(), 5, C.byref(ms))
    assert ms.value > 0
    want, _ = orc.attention(seq_len, kv_dim, kv_mul, n_heads, hs, pos, q.read(), ks[0].read(), vs[0].read())
    np.testing.assert_allclose(xb.read(), want, rtol=0, atol=2e-5)
    with pytest.raises(W.WgmlError):  # planned for fewer positions than the position itself
        call("wgml_bench_attention", gpu.handle, C.byref(p), 256, q.view(), kv, vv, 2, xb.view(), 5, C.byref(ms))
    with pytest.raises(W.WgmlError):  # caches shorter than seq_len rows
        bad = AttnParams(2 * seq_len, kv_dim, kv_mul, n_heads, hs, pos)
        call("wgml_bench_attention", gpu.handle, C.byref(bad), 1024, q.view(), kv, vv, 2, xb.view(), 5, C.byref(ms))


def test_attention_invariants(gpu):
    seq_len, n_heads, hs, kv_mul = 64, 8, 64, 2
    kv_dim = n_heads // kv_mul * hs
    q = rnd(n_heads * hs, 1)
    vc = rnd(seq_len * kv_dim, 3)
    kc = np.tile(rnd(kv_dim, 2), seq_len)  # identical keys -> uniform weights -> mean of V
    p = W.BatchedMultiqueryAttentionParams(seq_len, kv_dim, kv_mul, n_heads, hs, 39)
    xb = W.GpuVector.uninit(gpu, n_heads * hs)
    W.BatchedMultiqueryAttention.from_device(gpu).dispatch_multi(
        p, W.GpuVector.init(gpu, q), W.GpuVector.init(gpu, kc), W.GpuVector.init(gpu, vc), xb)
    vm = vc.reshape(seq_len, kv_dim)[:40].astype(np.float64).mean(0)
    got = xb.read()
    for h in range(n_heads):
        g = h // kv_mul
        np.testing.assert_allclose(got[h * hs:(h + 1) * hs], vm[g * hs:(g + 1) * hs], atol=1e-5)


def test_attention_argument_checks(gpu):
    a = W.BatchedMultiqueryAttention.from_device(gpu)
    v = W.GpuVector.uninit(gpu, 1024)
    with pytest.raises(W.WgmlError):  # pos outside seq_len
        a.dispatch(W.BatchedMultiqueryAttentionParams(4, 64, 1, 1, 64, 4), v.rows(0, 64), v, v,
                   None, v.rows(0, 64))
    with pytest.raises(W.WgmlError):  # kv_dim inconsistent with heads
        a.dispatch(W.BatchedMultiqueryAttentionParams(4, 32, 1, 1, 64, 0), v.rows(0, 64), v, v,
                   None, v.rows(0, 64))

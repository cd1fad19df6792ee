"""GPU parity: per-token vector ops against the CPU oracle.  Shapes, lengths and
tolerances follow the reference's own op tests (odd LEN = 1757; see each test)."""
import numpy as np
import pytest

import oracle as orc
import wgml_amd as W

pytestmark = pytest.mark.gpu
LEN = 1757


def rnd(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def vec(gpu, a):
    return W.GpuVector.init(gpu, a)


@pytest.mark.parametrize("n", [LEN, 288, 4096, 1])
@pytest.mark.parametrize("eps", [1e-5, 1e-6])
def test_rms_norm(gpu, n, eps):  # ops/rms_norm.rs:77-136, epsilon 1e-4
    a, w = rnd(n, 1), rnd(n, 2)
    out = W.GpuVector.uninit(gpu, n)
    W.RmsNorm.from_device(gpu).dispatch(W.RmsNormConfig(eps), out, vec(gpu, a), vec(gpu, w))
    np.testing.assert_allclose(out.read(), orc.rms_norm(a, w, eps), rtol=0, atol=1e-5)


@pytest.mark.parametrize("n", [LEN, 768, 3])
def test_layernorm(gpu, n):  # ops/layernorm.rs:67-102, epsilon 1e-5
    v = rnd(n, 3, 2.0) + 0.5
    out = W.GpuVector.uninit(gpu, n)
    W.LayerNorm.from_device(gpu).dispatch(out, vec(gpu, v))
    np.testing.assert_allclose(out.read(), orc.layernorm(v), rtol=0, atol=1e-5)


def test_layernorm_dimension_mismatch(gpu):
    with pytest.raises(W.WgmlError, match="dimension mismatch"):
        W.LayerNorm.from_device(gpu).dispatch(W.GpuVector.uninit(gpu, 4), W.GpuVector.uninit(gpu, 5))


@pytest.mark.parametrize("variant", [W.RoPEVariant.Original, W.RoPEVariant.Neox])
@pytest.mark.parametrize("pos,base,tol", [(10, 1.0e4, 1e-5), (0, 1.0e4, 0.0), (255, 1.0e4, 1e-4),
                                          (8300, 5.0e5, 4e-3)])
def test_rope(gpu, variant, pos, base, tol):  # ops/rope.rs:131-198: hs 128, 13 q / 9 k heads
    hs = 128
    q, k = rnd(13 * hs, 4), rnd(9 * hs, 5)
    gq, gk = vec(gpu, q), vec(gpu, k)
    W.RoPE.from_device(gpu).dispatch(variant, W.RoPEConfig(hs, 9 * hs, pos, base), gq, gk)
    wq, wk = orc.rope(q, k, hs, 9 * hs, pos, base, variant)
    # both sides form the angle in f32; an ulp of difference in powf moves it by |angle| * 6e-8
    np.testing.assert_allclose(gq.read(), wq, rtol=0, atol=tol)
    np.testing.assert_allclose(gk.read(), wk, rtol=0, atol=tol)


def test_rope_kv_dim_smaller_than_k(gpu):
    hs = 64
    q, k = rnd(8 * hs, 6), rnd(4 * hs, 7)
    gq, gk = vec(gpu, q), vec(gpu, k)
    W.RoPE.from_device(gpu).dispatch(0, W.RoPEConfig(hs, 2 * hs, 33, 1e4), gq, gk)
    wq, wk = orc.rope(q, k, hs, 2 * hs, 33, 1e4, 0)
    np.testing.assert_allclose(gk.read(), wk, atol=1e-5)
    assert np.array_equal(gk.read()[2 * hs:], k[2 * hs:])


def test_rope_asserts(gpu):  # ops/rope.rs:51-56
    r = W.RoPE.from_device(gpu)
    cfg = W.RoPEConfig(2, 2, 1, 1e4)
    with pytest.raises(W.WgmlError):
        r.dispatch(0, cfg, W.GpuVector.uninit(gpu, 7), W.GpuVector.uninit(gpu, 4))
    with pytest.raises(W.WgmlError, match="Query vector must be larger"):
        r.dispatch(0, cfg, W.GpuVector.uninit(gpu, 4), W.GpuVector.uninit(gpu, 8))


@pytest.mark.parametrize("n", [LEN, 7, 9000])
def test_softmax(gpu, n):  # ops/softmax.rs:63-95, epsilon 1e-7
    v = rnd(n, 8, 3.0)
    g = vec(gpu, v)
    W.SoftMax.from_device(gpu).dispatch(g)
    np.testing.assert_allclose(g.read(), orc.softmax(v), rtol=1e-5, atol=1e-7)


def test_softmax_columns_with_stride(gpu):
    nrows, ncols, stride = 37, 5, 64
    m = rnd(ncols * stride, 9, 2.0)
    g = vec(gpu, m)
    W.SoftMax.from_device(gpu).dispatch(g, nrows, ncols, stride)
    got = g.read().reshape(ncols, stride)
    for j in range(ncols):
        np.testing.assert_allclose(got[j, :nrows], orc.softmax(m.reshape(ncols, stride)[j, :nrows]),
                                   rtol=1e-5, atol=1e-7)
        assert np.array_equal(got[j, nrows:], m.reshape(ncols, stride)[j, nrows:])


@pytest.mark.parametrize("n", [LEN, 768, 11008])
def test_silu(gpu, n):  # ops/silu.rs:57-98, epsilon 1e-5
    h1, h2 = rnd(n, 10, 2.0), rnd(n, 11)
    g1 = vec(gpu, h1)
    W.Silu.from_device(gpu).dispatch(g1, vec(gpu, h2))
    np.testing.assert_allclose(g1.read(), orc.silu(h1, h2), rtol=1e-5, atol=1e-5)


def _unary_ref(op, x, a):
    x64 = x.astype(np.float64)
    U = W.UnaryOp
    sig = lambda t: 1 / (1 + np.exp(-t))  # noqa: E731
    table = {
        U.Abs: np.abs(x64), U.Sgn: np.sign(x64), U.Neg: -x64, U.Step: (x64 > 0) * 1.0,
        U.Elu: np.where(x64 > 0, x64, np.exp(x64) - 1),
        U.Gelu: orc.gelu(x).astype(np.float64),
        U.GeluQuick: x64 * sig(1.702 * x64), U.Silu: x64 * sig(x64), U.Tanh: np.tanh(x64),
        U.Relu: np.maximum(x64, 0), U.Sigmoid: sig(x64),
        U.HardSigmoid: np.clip((x64 + 3) / 6, 0, 1), U.HardSwish: x64 * np.clip((x64 + 3) / 6, 0, 1),
        U.Sqr: x64 * x64, U.Sqrt: np.sqrt(np.abs(x64)), U.Log: np.log(np.abs(x64) + 1e-3),
        U.LeakyRelu: np.maximum(x64, 0) + np.minimum(x64, 0) * a[0],
        U.Clamp: np.clip(x64, a[0], a[1]), U.Scale: x64 * a[0], U.AddScalar: x64 + a[0],
    }
    return table[op]


@pytest.mark.parametrize("op", list(range(20)))
def test_unary_ops(gpu, op):  # ops/unary.rs:273-348, epsilon 1e-5
    x = rnd(LEN, 12, 2.0)
    args = [0.25, 0.75, 0.0, 0.0] if op != W.UnaryOp.Clamp else [-0.5, 0.7, 0.0, 0.0]
    src = x
    if op == W.UnaryOp.Sqrt:
        src = np.abs(x)
    if op == W.UnaryOp.Log:
        src = (np.abs(x) + 1e-3).astype(np.float32)
    g = vec(gpu, src)
    W.UnaryInplace(gpu, op).dispatch(g, args if op >= W.UnaryOp.LeakyRelu else None)
    np.testing.assert_allclose(g.read(), _unary_ref(op, x, args), rtol=1e-5, atol=1e-5)


def test_unary_sgn_at_zero_follows_the_shader(gpu):
    # WGSL sign (ops/unary.wgsl:27) is 0 at both zeros; the reference's CPU twin (f32::signum,
    # ops/unary.rs:90) would give +1 / -1 there.  The device op follows the shader; its test in
    # the reference (ops/unary.rs:273-348) draws random values and never meets a zero.
    x = np.array([0.0, -0.0, 1e-30, -1e-30, 3.5, -2.0, np.inf, -np.inf], dtype=np.float32)
    g = vec(gpu, x)
    W.UnaryInplace(gpu, W.UnaryOp.Sgn).dispatch(g, None)
    assert g.read().tolist() == [0.0, 0.0, 1.0, -1.0, 1.0, -1.0, 1.0, -1.0]


def test_unary_needs_args(gpu):  # ops/unary.rs:173-176
    with pytest.raises(W.WgmlError, match="needs arguments"):
        W.UnaryInplace(gpu, W.UnaryOp.Scale).dispatch(W.GpuVector.uninit(gpu, 4), None)


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_op_assign_on_views(gpu, variant):
    a, b = rnd(2304, 13), rnd(768, 14)
    ga, gb = vec(gpu, a), vec(gpu, b)
    W.OpAssign(gpu, variant).dispatch(ga.rows(768, 768), gb)  # curr_2304.rows(768, 768)
    want = a.copy()
    if variant == 0:
        want[768:1536] += b
    elif variant == 1:
        want[768:1536] *= b
    else:
        want[768:1536] = b
    assert np.array_equal(ga.read(), want)


def test_argmax_first_maximum(gpu):  # models/sampler.rs:54-56
    s = W.Sampler(gpu)
    for n, seed in ((32000, 1), (128256, 2), (50257, 3), (5, 4)):
        v = rnd(n, seed)
        assert s.sample_argmax(vec(gpu, v)) == orc.argmax(v)
    v = np.zeros(70000, dtype=np.float32)
    v[[123, 45000, 69999]] = 7.0  # ties: the first index wins
    assert s.sample_argmax(vec(gpu, v)) == 123
    assert s.sample_argmax(vec(gpu, np.full(3000, -np.inf, dtype=np.float32))) == 0
    # sub-views that do not start on a 16-byte boundary, every length down to one element
    v = rnd(9000, 5)
    whole = vec(gpu, v)
    for start, count in ((1, 8999), (2, 8000), (3, 4097), (1, 3), (3, 2), (2, 1), (5, 70)):
        assert s.sample_argmax(whole.rows(start, count)) == orc.argmax(v[start:start + count])
    v[1] = v[4000] = v[8999] = 99.0  # a tie between the unaligned head, the middle and the tail
    assert s.sample_argmax(vec(gpu, v).rows(1, 8999)) == 0

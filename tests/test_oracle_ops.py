"""Pins the CPU oracle's per-token ops against closed forms / torch (no GPU)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc

LEN = 1757  # the odd length the reference's own op tests use


def rnd(n, seed, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(n) * scale).astype(np.float32)


def test_rms_norm_vs_torch():
    a, w = rnd(LEN, 1), rnd(LEN, 2)
    for eps in (1e-5, 1e-6):
        want = F.rms_norm(torch.from_numpy(a).double(), (LEN,), torch.from_numpy(w).double(),
                          eps=eps).numpy()
        np.testing.assert_allclose(orc.rms_norm(a, w, eps), want, rtol=0, atol=1e-5)
    # a dropped eps or a missing sqrt would fail this special case: constant input c -> w*c/|c|
    np.testing.assert_allclose(orc.rms_norm(np.full(64, 3.0), np.ones(64), 0.0), 1.0, atol=1e-6)


def test_layernorm_vs_torch():
    v = rnd(LEN, 3, 2.0) + 0.7
    want = F.layer_norm(torch.from_numpy(v).double(), (LEN,), eps=1e-5).numpy()
    np.testing.assert_allclose(orc.layernorm(v), want, rtol=0, atol=1e-5)


def test_softmax_vs_torch():
    v = rnd(LEN, 4, 3.0)
    got = orc.softmax(v)
    want = torch.softmax(torch.from_numpy(v).double(), 0).numpy()
    np.testing.assert_allclose(got, want, rtol=0, atol=1e-7)
    assert abs(got.sum() - 1) < 1e-5
    # shift invariance (the max subtraction): large inputs must not overflow
    np.testing.assert_allclose(orc.softmax(v + 500), got, atol=1e-6)


def test_silu_gate_vs_torch():
    h1, h2 = rnd(LEN, 5, 2.0), rnd(LEN, 6)
    want = (F.silu(torch.from_numpy(h1).double()) * torch.from_numpy(h2).double()).numpy()
    np.testing.assert_allclose(orc.silu(h1, h2), want, rtol=0, atol=1e-5)


def test_gelu_vs_torch():
    x = rnd(LEN, 7, 2.0)
    want = F.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    np.testing.assert_allclose(orc.gelu(x), want, rtol=0, atol=1e-5)


def _rope_closed_form(q, k, hs, kv_dim, pos, base, variant):
    q, k = q.astype(np.float64).copy(), k.astype(np.float64).copy()

    def rot(v, limit):
        out = v.copy()
        for i in range(0, limit, 2):
            ang = pos * base ** (-(i % hs) / hs)
            if variant == 0:
                a, b = i, i + 1
            else:
                a = i // 2 + (i // hs) * (hs // 2)
                b = a + hs // 2
            z = complex(v[a], v[b]) * np.exp(1j * ang)
            out[a], out[b] = z.real, z.imag
        return out

    return rot(q, q.size), rot(k, kv_dim)


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("pos,base", [(10, 1.0e4), (8300, 5.0e5)])
def test_rope_complex_rotation(variant, pos, base):
    hs = 128
    q, k = rnd(13 * hs, 8), rnd(9 * hs, 9)  # reference test shape (ops/rope.rs:139-148)
    kv_dim = 9 * hs
    gq, gk = orc.rope(q, k, hs, kv_dim, pos, base, variant)
    wq, wk = _rope_closed_form(q, k, hs, kv_dim, pos, base, variant)
    # the angle is formed in f32 (pos * theta) as ops/rope.wgsl:38-41 does, so at
    # pos 8300 it carries a rounding error of about |angle| * 6e-8 ~ 5e-4 rad
    tol = 1e-5 if pos < 100 else 4e-3
    np.testing.assert_allclose(gq, wq, atol=tol)
    np.testing.assert_allclose(gk, wk, atol=tol)


def test_rope_invariants():
    hs = 64
    q, k = rnd(8 * hs, 10), rnd(8 * hs, 11)
    kv_dim = 2 * hs
    # pos 0 is the identity
    gq, gk = orc.rope(q, k, hs, kv_dim, 0, 1e4)
    assert np.array_equal(gq, q) and np.array_equal(gk, k)
    gq, gk = orc.rope(q, k, hs, kv_dim, 77, 1e4)
    # k untouched beyond kv_dim, changed below it
    assert np.array_equal(gk[kv_dim:], k[kv_dim:])
    assert not np.array_equal(gk[:kv_dim], k[:kv_dim])
    # pairs keep their norm
    np.testing.assert_allclose(gq[0::2] ** 2 + gq[1::2] ** 2, q[0::2] ** 2 + q[1::2] ** 2,
                               rtol=1e-5)
    # the first pair of every head turns by exactly `pos` radians (theta = 1)
    ang = np.arctan2(gq[1::hs], gq[0::hs]) - np.arctan2(q[1::hs], q[0::hs])
    np.testing.assert_allclose(np.mod(ang - 77 + np.pi, 2 * np.pi) - np.pi, 0, atol=1e-4)


def _attention_torch(seq_len, kv_dim, kv_mul, n_heads, hs, pos, q, kc, vc):
    q = torch.from_numpy(q).double().view(n_heads, hs)
    k = torch.from_numpy(kc).double().view(seq_len, n_heads // kv_mul, hs)[:pos + 1]
    v = torch.from_numpy(vc).double().view(seq_len, n_heads // kv_mul, hs)[:pos + 1]
    k = k.repeat_interleave(kv_mul, dim=1)  # head h uses kv head h // kv_mul
    v = v.repeat_interleave(kv_mul, dim=1)
    s = torch.einsum("hd,thd->ht", q, k) / np.sqrt(hs)
    p = torch.softmax(s, dim=1)
    return torch.einsum("ht,thd->hd", p, v).reshape(-1).numpy(), p.numpy()


@pytest.mark.parametrize("kv_mul", [1, 4])
@pytest.mark.parametrize("pos", [0, 6, 8])
def test_attention_vs_torch(kv_mul, pos):
    # reference test shape (ops/batched_multiquery_attention.rs:219-226): 12 heads x 64
    seq_len, n_heads, hs = 1024, 12, 64
    kv_dim = n_heads // kv_mul * hs
    q = rnd(n_heads * hs, 12)
    kc, vc = rnd(seq_len * kv_dim, 13), rnd(seq_len * kv_dim, 14)
    xb, att = orc.attention(seq_len, kv_dim, kv_mul, n_heads, hs, pos, q, kc, vc)
    wx, wp = _attention_torch(seq_len, kv_dim, kv_mul, n_heads, hs, pos, q, kc, vc)
    np.testing.assert_allclose(xb, wx, atol=1e-5)
    np.testing.assert_allclose(att[:, :pos + 1], wp, atol=1e-6)


def test_attention_invariants():
    seq_len, n_heads, hs, kv_mul = 32, 4, 16, 2
    kv_dim = n_heads // kv_mul * hs
    q = rnd(n_heads * hs, 15)
    kc, vc = rnd(seq_len * kv_dim, 16), rnd(seq_len * kv_dim, 17)
    # pos 0: the output of head h is V[0] of its kv head
    xb, _ = orc.attention(seq_len, kv_dim, kv_mul, n_heads, hs, 0, q, kc, vc)
    for h in range(n_heads):
        g = h // kv_mul
        assert np.allclose(xb[h * hs:(h + 1) * hs], vc[g * hs:(g + 1) * hs], atol=1e-7)
    # identical keys -> uniform weights -> mean of V
    kc2 = np.tile(kc[:kv_dim], seq_len)
    xb, att = orc.attention(seq_len, kv_dim, kv_mul, n_heads, hs, 9, q, kc2, vc)
    np.testing.assert_allclose(att[:, :10], 0.1, atol=1e-6)
    vm = vc.reshape(seq_len, kv_dim)[:10].mean(0)
    for h in range(n_heads):
        g = h // kv_mul
        np.testing.assert_allclose(xb[h * hs:(h + 1) * hs], vm[g * hs:(g + 1) * hs], atol=1e-6)


def test_argmax_first_maximum():
    v = np.array([1.0, 5.0, 3.0, 5.0, -2.0], dtype=np.float32)
    assert orc.argmax(v) == 1
    assert orc.argmax(np.array([-3.0], dtype=np.float32)) == 0

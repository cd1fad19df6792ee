"""The CPU sampler (models/sampler.rs:14-130): the oracle's restatement is pinned by what the
algorithm fixes (closed forms on small distributions, an independent numpy construction of the
nucleus, the empirical distribution over many coins); the library's sampler must then return
the oracle's token for every coin.  No GPU needed."""
import numpy as np
import pytest

import oracle as orc
import wgml_amd as W


def np_topp(p, topp, coin):
    """Independent construction: nucleus = shortest prefix of the descending order whose mass
    exceeds topp; draw proportionally inside it."""
    n = p.size
    cand = np.flatnonzero(p >= np.float32((1.0 - topp) / (n - 1)))
    order = cand[np.argsort(-p[cand], kind="stable")]
    cum = np.cumsum(p[order], dtype=np.float32)
    over = np.flatnonzero(cum > np.float32(topp))
    last = over[0] if over.size else order.size - 1
    r = np.float32(coin) * cum[last]
    inside = np.flatnonzero(np.float32(r) < cum[:last + 1])
    return int(order[inside[0]] if inside.size else order[last])


def test_mult_closed_form():
    p = np.float32([0.1, 0.2, 0.3, 0.4])
    for coin, want in ((0.0, 0), (0.0999, 0), (0.1, 1), (0.29, 1), (0.31, 2), (0.61, 3), (0.999, 3)):
        assert orc.sample_mult(p, coin) == want
    assert orc.sample_mult(np.float32([0.5, 0.25]), 0.9) == 1  # rounding guard: last index


def test_topp_closed_form():
    p = np.float32([0.05, 0.5, 0.15, 0.3])
    # descending: 1 (0.5), 3 (0.3), 2 (0.15), 0 (0.05); topp 0.7 -> nucleus {1, 3} (0.8 > 0.7)
    for coin in np.linspace(0, 0.999, 50):
        t = orc.sample_topp(p, 0.7, float(coin))
        assert t == (1 if coin * 0.8 < 0.5 else 3)
    # topp 0.4 -> nucleus {1} only
    assert {orc.sample_topp(p, 0.4, c) for c in (0.0, 0.5, 0.99)} == {1}
    # ties keep index order (stable sort): 0.4, 0.4 -> index 0 comes first and is the nucleus
    assert {orc.sample_topp(np.float32([0.4, 0.4, 0.2]), 0.3, c) for c in (0.0, 0.5, 0.99)} == {0}


def test_oracle_matches_independent_nucleus_and_distribution():
    rng = np.random.default_rng(0)
    logits = (rng.standard_normal(500) * 3).astype(np.float32)
    p = np.exp(logits - logits.max()).astype(np.float32)
    p /= p.sum(dtype=np.float32)
    for topp in (0.3, 0.9, 0.95):
        for coin in rng.random(200):
            assert orc.sample_topp(p, topp, float(coin)) == np_topp(p, topp, float(coin))
    # multinomial branch: empirical frequencies follow p
    coins = (np.arange(20000) + 0.5) / 20000
    counts = np.bincount([orc.sample_mult(p, float(c)) for c in coins], minlength=p.size)
    np.testing.assert_allclose(counts / coins.size, p, atol=2e-4)


@pytest.mark.parametrize("temperature,topp", [(0.0, 0.9), (0.7, 0.95), (1.3, 0.0), (1.0, 1.0),
                                              (0.2, 0.5)])
def test_library_sampler_equals_oracle(temperature, topp):
    rng = np.random.default_rng(5)
    s = W.Sampler(None, temperature, topp)
    for trial in range(40):
        logits = (rng.standard_normal(1000) * 2).astype(np.float32)
        if trial % 5 == 0:
            logits[17] = logits[400] = logits.max() + 1  # a tie at the top
        coin = float(W.rng_uniform(trial, 1)[0])
        assert s.sample(logits.copy(), coin) == orc.sample(logits, temperature, topp, coin)


def test_temperature_zero_is_argmax_and_probabilities_are_written_back():
    logits = np.float32([0.5, 2.0, 2.0, -1.0])
    assert W.Sampler(None, 0.0, 0.9).sample(logits.copy(), 0.3) == 1
    v = logits.copy()
    W.Sampler(None, 0.5, 0.0).sample(v, 0.3)
    e = np.exp((logits / np.float32(0.5)) - np.float32(4.0))
    np.testing.assert_allclose(v, e / e.sum(), rtol=1e-6)


def test_argument_checks_and_coins():
    with pytest.raises(W.WgmlError):
        W.Sampler(None, 1.0, 0.5).sample(np.zeros(4, np.float32), 1.0)  # coin must be < 1
    with pytest.raises(W.WgmlError):
        W.Sampler(None, -1.0, 0.5).sample(np.zeros(4, np.float32), 0.5)
    c = W.rng_uniform(9, 10000)
    assert c.min() >= 0.0 and c.max() < 1.0 and abs(c.mean() - 0.5) < 0.02
    assert np.array_equal(c[:100], W.rng_uniform(9, 100))

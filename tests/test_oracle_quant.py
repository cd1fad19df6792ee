"""Pins the CPU oracle's f16 decoding, dequantizers and GEMV (no GPU needed)."""
import os

import numpy as np
import pytest

import npref
import oracle as orc

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "dequant_fixtures.npz"))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def test_decode_f16_exhaustive_vs_numpy():
    # quantization.rs:392-409 against the library half->float conversion, all 65536 inputs
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([orc.decode_f16(int(b)) for b in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got[~nan]), bits(want[~nan]))  # includes subnormals, +-0, +-inf
    # spot values fixed by the format itself
    assert orc.decode_f16(0x3C00) == 1.0
    assert orc.decode_f16(0x0001) == 2.0 ** -24
    assert orc.decode_f16(123) == 123 * 2.0 ** -24  # the Q6_K fixture's d
    assert orc.decode_f16(0x3CF0) == 1.234375
    assert orc.decode_f16(0x45AE) == 5.6796875


ALL_FIXTURES = [("q8_0", orc.Q8_0), ("q4_k", orc.Q4_K), ("q6_k", orc.Q6_K), ("q4_0", orc.Q4_0),
                ("q4_1", orc.Q4_1), ("q5_0", orc.Q5_0), ("q5_1", orc.Q5_1), ("q5_k", orc.Q5_K),
                ("q8_k", orc.Q8_K)]
ALL_TYPES = [t for _, t in ALL_FIXTURES]


@pytest.mark.parametrize("name,qtype", ALL_FIXTURES)
def test_dequant_reference_fixture_blocks(name, qtype):
    raw, want = GOLD[f"{name}_raw"], GOLD[f"{name}_expected"]
    got = orc.dequantize(qtype, raw, want.size)
    assert np.array_equal(bits(got), bits(want))


def test_dequant_hand_computed_anchors():
    # Values worked out by hand from the block layouts (see the fixture script for the inputs).
    q8 = orc.dequantize(orc.Q8_0, GOLD["q8_0_raw"], 8 * 32)
    assert q8[0] == -158.0                      # -128 * 1.234375
    assert q8[7 * 32 + 31] == 18.515625         # 15 * 1.234375
    q4 = orc.dequantize(orc.Q4_K, GOLD["q4_k_raw"], 16 * 256)
    assert np.all(q4[0:32] == -22.71875)        # sc 0, m 4: -(5.6796875 * 4)
    assert np.all(q4[32:48] == -28.3984375)     # sc 1, m 5, high nibble 0
    assert np.all(q4[48:64] == -27.1640625)     # high nibble 1
    assert q4[128 + 5] == 49.375                # sub-block 4: sc 8, m 0, nibble 5
    q6 = orc.dequantize(orc.Q6_K, GOLD["q6_k_raw"], 16 * 256)
    assert q6[0] == 499872 / 2 ** 24            # (123*2^-24) * -127 * -32
    q40 = orc.dequantize(orc.Q4_0, GOLD["q4_0_raw"], 16 * 32)
    assert q40[0] == -8 * 1.234375 and q40[16] == -8 * 1.234375   # block 0: qs[0] = 0x00
    assert q40[32 + 1] == (1 - 8) * 1.234375 and q40[32 + 17] == (1 - 8) * 1.234375  # 0x11
    q41 = orc.dequantize(orc.Q4_1, GOLD["q4_1_raw"], 16 * 32)
    assert q41[5] == np.float32(5 * 1.234375) + np.float32(3 * 2.0 ** -24)
    q50 = orc.dequantize(orc.Q5_0, GOLD["q5_0_raw"], 16 * 32)
    # qh = [1, 100, 200, 250] -> u32 0xFAC86401: bit 0 set (element 0 gets +16), bit 1 clear
    assert q50[0] == (0 + 16 - 16) * 1.234375 and q50[1] == (1 - 16) * 1.234375
    # element 16 takes bit 16 (0xC8 = 0b11001000 -> bit 0 clear), element 19 takes bit 19 (set)
    assert q50[16] == (0 - 16) * 1.234375 and q50[19] == (0 + 16 - 16) * 1.234375
    q8k = orc.dequantize(orc.Q8_K, GOLD["q8_k_raw"], 16 * 256)
    assert q8k[0] == np.float32(1.234) * np.float32(-127) and q8k[255] == np.float32(1.234) * -128
    q5k = orc.dequantize(orc.Q5_K, GOLD["q5_k_raw"], 16 * 256)
    assert np.all(q5k[0:32:2] == -22.71875)     # block 0: sc 0 -> -(dmin * 4) whatever the quants


@pytest.mark.parametrize("qtype", ALL_TYPES + [orc.F16])
def test_dequant_random_bits_vs_numpy(qtype):
    nb = 10000
    raw = npref.random_blocks(qtype, nb, seed=1234 + qtype)
    want = npref.DEQUANT[qtype](raw)
    got = orc.dequantize(qtype, raw, nb * npref.BLOCK_ELEMS[qtype])
    assert np.isfinite(want).all()
    assert np.array_equal(bits(got), bits(want))


def test_dequantize_rejects_unknown_tag():
    out = np.zeros(32, dtype=np.float32)
    assert orc.lib.orc_dequantize(99, out.ctypes.data, 32, out.ctypes.data) == -1


@pytest.mark.parametrize("qtype", [orc.Q8_0, orc.Q4_K, orc.Q6_K])
def test_gemv_one_hot_returns_column(qtype):
    # out = dequant(M) . e_j must be column j of the dequantized matrix, exactly
    nrows, ncols = 8, 512
    be = npref.BLOCK_ELEMS[qtype]
    raw = npref.random_blocks(qtype, nrows * ncols // be, seed=7)
    deq = npref.DEQUANT[qtype](raw).reshape(nrows, ncols)
    for j in (0, 1, 31, 32, 255, 256, 300, 511):
        x = np.zeros(ncols, dtype=np.float32)
        x[j] = 1.0
        o32, o64 = orc.gemv_quant(qtype, raw, nrows, ncols, x)
        assert np.array_equal(o32, deq[:, j])
        assert np.array_equal(o64, deq[:, j].astype(np.float64))


def test_gemv_brute_force_and_order():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((5, 37)).astype(np.float32)
    x = rng.standard_normal(37).astype(np.float32)
    # f64 variant equals numpy's float64 product
    np.testing.assert_allclose(orc.gemv_f64(w, x), w.astype(np.float64) @ x.astype(np.float64),
                               rtol=1e-14)
    # f32 variant: sequential left-to-right sum of separately rounded products
    want = np.empty(5, dtype=np.float32)
    for i in range(5):
        acc = np.float32(x[0] * w[i, 0])
        for j in range(1, 37):
            acc = np.float32(np.float32(x[j] * w[i, j]) + acc)
        want[i] = acc
    assert np.array_equal(orc.gemv_f32(w, x), want)
    # the column-sweep twin used for CPU timing gives the same bits
    wc = np.ascontiguousarray(w.T)
    out = np.empty(5, dtype=np.float32)
    orc.lib.orc_gemv_f32_colmajor(out.ctypes.data, wc.ctypes.data, x.ctypes.data, 5, 37)
    assert np.array_equal(out, want)


def test_gemv_constant_quants_closed_form():
    # Q8_0 with every q equal: out = d * q * sum(x)
    nrows, ncols = 4, 256
    blk = np.concatenate([np.array([0x3C00], dtype=np.uint16).view(np.uint8),
                          np.full(32, 3, dtype=np.int8).view(np.uint8)])
    raw = np.tile(blk, nrows * ncols // 32)
    x = np.arange(ncols, dtype=np.float32) / 64
    _, o64 = orc.gemv_quant(orc.Q8_0, raw, nrows, ncols, x)
    np.testing.assert_allclose(o64, 3.0 * x.astype(np.float64).sum(), rtol=1e-12)

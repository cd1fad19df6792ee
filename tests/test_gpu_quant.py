"""GPU parity: half decoding and dequantization, bit-exact against the CPU oracle
and the committed golden vectors.  Mirrors the reference's `dequantization` test
(crates/wgml/src/ops/quantization.rs:37-408)."""
import os

import numpy as np
import pytest

import npref
import oracle as orc
import wgml_amd as W

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "dequant_fixtures.npz"))


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def gpu_dequant(gpu, qtype, raw, nrows, ncols):
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    out = W.GpuVector.uninit(gpu, nrows * ncols)
    W.Quantization.from_device(gpu).dequantize(out, m)
    return out.read()


def test_f16_all_bit_patterns(gpu):
    h = np.arange(65536, dtype=np.uint16)
    src = W.GpuVector.from_bytes(gpu, h)
    out = W.GpuVector.uninit(gpu, 65536)
    W.Quantization.from_device(gpu).f16_to_f32(out, src)
    got = out.read()
    want = np.array([orc.decode_f16(int(b)) for b in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got[~nan]), bits(want[~nan]))


@pytest.mark.parametrize("name,qtype,nblk", [("q8_0", W.Q8_0, 8), ("q4_k", W.Q4_K, 16),
                                            ("q6_k", W.Q6_K, 16)])
def test_dequant_reference_fixture_blocks(gpu, name, qtype, nblk):
    raw, want = GOLD[f"{name}_raw"], GOLD[f"{name}_expected"]
    be = npref.BLOCK_ELEMS[qtype]
    # as one row, and as several rows of fewer blocks (row-major block order)
    for nrows in (1, 2, nblk):
        got = gpu_dequant(gpu, qtype, raw, nrows, nblk // nrows * be)
        assert np.array_equal(bits(got), bits(want)), (name, nrows)


@pytest.mark.parametrize("qtype", [W.Q8_0, W.Q4_K, W.Q6_K])
@pytest.mark.parametrize("nrows,nblk_per_row", [(3, 1), (7, 9), (64, 43), (5, 17)])
def test_dequant_random_bits_bit_exact(gpu, qtype, nrows, nblk_per_row):
    # odd block counts per row: the reference can only keep even/paired counts quantized
    be = npref.BLOCK_ELEMS[qtype]
    raw = npref.random_blocks(qtype, nrows * nblk_per_row, seed=99 + qtype + nrows)
    want = orc.dequantize(qtype, raw, nrows * nblk_per_row * be)
    got = gpu_dequant(gpu, qtype, raw, nrows, nblk_per_row * be)
    assert np.array_equal(bits(got), bits(want))


OTHER = [("q4_0", W.Q4_0), ("q4_1", W.Q4_1), ("q5_0", W.Q5_0), ("q5_1", W.Q5_1),
         ("q5_k", W.Q5_K), ("q8_k", W.Q8_K)]


@pytest.mark.parametrize("name,qtype", OTHER)
def test_remaining_block_formats_stay_quantized(gpu, name, qtype):
    # GgufTensorData::to_gpu_matrix keeps these quantized on the GPU too (gguf.rs:172-182); the
    # matrix holds the GGUF bytes unchanged.  Reference fixture blocks, then random bits; the
    # dequantization kernel is bit-exact, the GEMV within the GEMV tolerance.
    raw, want = GOLD[f"{name}_raw"], GOLD[f"{name}_expected"]
    be = npref.BLOCK_ELEMS[qtype]
    m = W.GpuQuantMatrix(gpu, qtype, 2, 8 * be, raw)
    assert m.shape() == (qtype, 2, 8 * be) and m.gguf_bytes() == raw.size
    assert np.array_equal(bits(gpu_dequant(gpu, qtype, raw, 2, 8 * be)), bits(want))
    nrows, nblk = 5, 7
    rnd = npref.random_blocks(qtype, nrows * nblk, seed=500 + qtype)
    want = orc.dequantize(qtype, rnd, nrows * nblk * be)
    assert np.array_equal(bits(gpu_dequant(gpu, qtype, rnd, nrows, nblk * be)), bits(want))
    # host dequantizer, same values
    assert np.array_equal(bits(W.dequantize_host(qtype, rnd, want.size)), bits(want))
    # the fixture blocks through the GEMV: one-hot vectors return dequantized columns
    ncols = 8 * be
    gm = W.GemvQuant.from_device(gpu)
    ref = GOLD[f"{name}_expected"].reshape(2, ncols)
    for col in (0, 1, 15, 16, 31, ncols - 1, ncols // 2 + 3):
        x = np.zeros(ncols, np.float32)
        x[col] = 1.0
        out = W.GpuVector.uninit(gpu, 2)
        gm.dispatch(out, m, W.GpuVector.init(gpu, x))
        np.testing.assert_allclose(out.read(), ref[:, col], rtol=1e-6, atol=0)


@pytest.mark.parametrize("name,qtype", [("q8_0", W.Q8_0), ("q4_k", W.Q4_K), ("q6_k", W.Q6_K)] + OTHER)
def test_weight_bound_of_every_quantized_format(gpu, name, qtype):
    # the bound the batched product checks (computed from the block scales when the matrix is
    # created) is never below the largest dequantized weight, and not far above it: random bits
    # reach the ends of a block's range
    nrows, nblk = 24, 8
    ncols = nblk * npref.BLOCK_ELEMS[qtype]
    raw = npref.random_blocks(qtype, nrows * nblk, seed=300 + qtype)
    w = orc.dequantize(qtype, raw, nrows * ncols)
    m = W.GpuQuantMatrix(gpu, qtype, nrows, ncols, raw)
    top = float(np.abs(w).max())
    assert top <= m.weight_bound() <= 1.5 * top, (name, top, m.weight_bound())


def test_f16_matrix_expanded_at_load(gpu):
    h = np.arange(4 * 64, dtype=np.uint16) * 97 % 31744  # finite halves
    want = np.array([orc.decode_f16(int(b)) for b in h], dtype=np.float32)
    assert np.array_equal(bits(gpu_dequant(gpu, W.F16, h.view(np.uint8), 4, 64)), bits(want))
    assert np.array_equal(bits(W.dequantize_host(W.F16, h.view(np.uint8), h.size)), bits(want))


def test_f32_matrix_round_trip(gpu):
    a = W.rng_normal(5, 12 * 64)
    got = gpu_dequant(gpu, W.F32, a.view(np.uint8), 12, 64)
    assert np.array_equal(bits(got), bits(a))


def test_quantized_then_dequantized_matches_oracle(gpu):
    # real quantizer output (well-formed blocks) rather than random bits
    for qtype in (W.Q8_0, W.Q4_K, W.Q6_K):
        x = W.rng_normal(77 + qtype, 16 * 1024, 0, 0.02)
        raw = W.quantize(qtype, x)
        got = gpu_dequant(gpu, qtype, raw, 16, 1024)
        assert np.array_equal(bits(got), bits(orc.dequantize(qtype, raw, x.size)))


def test_matrix_create_errors(gpu):
    raw = np.zeros(144 * 4, dtype=np.uint8)
    with pytest.raises(W.WgmlError) as ei:  # Q2_K: a tag the reference cannot read either
        W.GpuQuantMatrix(gpu, 10, 1, 256, raw)
    assert ei.value.code == W._lib.E_UNSUPPORTED
    with pytest.raises(W.WgmlError) as ei:  # ncols not a whole number of blocks
        W.GpuQuantMatrix(gpu, W.Q4_K, 4, 200, raw)
    assert ei.value.code == W._lib.E_INVALID
    m = W.GpuQuantMatrix(gpu, W.Q4_K, 2, 512, raw)
    assert m.shape() == (W.Q4_K, 2, 512) and m.gguf_bytes() == 576
    out = W.GpuVector.uninit(gpu, 100)
    with pytest.raises(W.WgmlError):        # wrong output length
        W.Quantization.from_device(gpu).dequantize(out, m)

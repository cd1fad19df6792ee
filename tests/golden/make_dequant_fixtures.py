"""Writes tests/golden/dequant_fixtures.npz.

Inputs: the deterministic test blocks that the reference's own dequantization
test builds (crates/wgml/src/ops/quantization.rs:79-86 for Q8_0, :179-202 for
Q4_K, :205-222 for Q6_K), re-created here from their description (the reference
holds no expected numbers: its test compares its GPU kernel with its CPU twin).
Expected outputs: the vectorised numpy restatement of ggml's dequantizers in
tests/npref.py — NOT the C oracle, so that the oracle is checked against
something it did not produce.

Run from the repository root:  python tests/golden/make_dequant_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import npref  # noqa: E402


def half_bits(x: float) -> int:
    return int(np.float16(x).view(np.uint16))


def u8(v):
    return np.asarray(v, dtype=np.int64).astype(np.uint8)


def q8_0_blocks():
    # 8 blocks: scale = f16(1.234); data[k] = (i*16 - 128) + k as i8
    out = []
    for i in range(8):
        scale = np.array([half_bits(1.234)], dtype=np.uint16).view(np.uint8)
        data = (np.full(32, i * 16 - 128, dtype=np.int64) + np.arange(32)).astype(np.int8)
        out.append(np.concatenate([scale, data.view(np.uint8)]))
    return np.concatenate(out)


def q4_k_blocks():
    # 16 blocks: d = f16(1.234), dmin = f16(5.678); scales[k] = i*16 + k;
    # qs[k] = saturating_add(i*16, k)
    out = []
    for i in range(16):
        hdr = np.array([half_bits(1.234), half_bits(5.678)], dtype=np.uint16).view(np.uint8)
        scales = u8(i * 16 + np.arange(12))
        qs = u8(np.minimum(i * 16 + np.arange(128), 255))
        out.append(np.concatenate([hdr, scales, qs]))
    return np.concatenate(out)


def q6_k_blocks():
    # 16 blocks: scales[k] = (i*8 - 127) + k as i8; ql[k] = i*8 + k; qh[k] = i*8 + k;
    # d = raw bits 123 (a subnormal half)
    out = []
    for i in range(16):
        ql = u8(i * 8 + np.arange(128))
        qh = u8(i * 8 + np.arange(64))
        scales = (np.full(16, i * 8 - 127, dtype=np.int64) + np.arange(16)).astype(np.int8)
        d = np.array([123], dtype=np.uint16).view(np.uint8)
        out.append(np.concatenate([ql, qh, scales.view(np.uint8), d]))
    return np.concatenate(out)


def main():
    q8, q4, q6 = q8_0_blocks(), q4_k_blocks(), q6_k_blocks()
    assert q8.size == 8 * 34 and q4.size == 16 * 144 and q6.size == 16 * 210
    np.savez_compressed(
        os.path.join(HERE, "dequant_fixtures.npz"),
        q8_0_raw=q8, q8_0_expected=npref.dequant_q8_0(q8),
        q4_k_raw=q4, q4_k_expected=npref.dequant_q4_k(q4),
        q6_k_raw=q6, q6_k_expected=npref.dequant_q6_k(q6))
    print("wrote dequant_fixtures.npz")


if __name__ == "__main__":
    main()

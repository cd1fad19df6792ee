"""Writes tests/golden/dequant_fixtures.npz.

Inputs: the deterministic test blocks that the reference's own dequantization
test builds (crates/wgml/src/ops/quantization.rs:79-86 for Q8_0, :87-176 for Q4_0,
Q4_1, Q5_0, Q5_1, Q8_K and Q5_K, :179-202 for Q4_K, :205-222 for Q6_K), re-created here from their description (the reference
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


def small_blocks(kind):
    # ops/quantization.rs:87-135: 16 blocks, d = f16(1.234), qs[k] = i*16 + k (wrapping u8);
    # Q4_1: m = raw bits 3; Q5_x: qh = [1, 100, 200, 250]; Q5_1: m = raw bits 125
    out = []
    for i in range(16):
        d = np.array([half_bits(1.234)], dtype=np.uint16).view(np.uint8)
        qs = u8(i * 16 + np.arange(16))
        parts = [d]
        if kind == "q4_1":
            parts.append(np.array([3], dtype=np.uint16).view(np.uint8))
        if kind == "q5_1":
            parts.append(np.array([125], dtype=np.uint16).view(np.uint8))
        if kind in ("q5_0", "q5_1"):
            parts.append(u8([1, 100, 200, 250]))
        out.append(np.concatenate(parts + [qs]))
    return np.concatenate(out)


def q8_k_blocks():
    # ops/quantization.rs:137-149: d = 1.234 (f32); qs[k] = saturating_add(i*8 - 127, k as i8);
    # bsums = 0.  `k as i8` wraps for k >= 128.
    out = []
    for i in range(16):
        d = np.array([1.234], dtype=np.float32).view(np.uint8)
        k = np.arange(256).astype(np.uint8).view(np.int8).astype(np.int64)
        qs = np.clip(i * 8 - 127 + k, -128, 127).astype(np.int8)
        out.append(np.concatenate([d, qs.view(np.uint8), np.zeros(32, np.uint8)]))
    return np.concatenate(out)


def q5_k_blocks():
    # ops/quantization.rs:151-176: d = f16(1.234), dmin = f16(5.678); scales[k] = i*16 + k;
    # qs[k], qh[k] = saturating_add(i*16, k)
    out = []
    for i in range(16):
        hdr = np.array([half_bits(1.234), half_bits(5.678)], dtype=np.uint16).view(np.uint8)
        scales = u8(i * 16 + np.arange(12))
        qh = u8(np.minimum(i * 16 + np.arange(32), 255))
        qs = u8(np.minimum(i * 16 + np.arange(128), 255))
        out.append(np.concatenate([hdr, scales, qh, qs]))
    return np.concatenate(out)


def main():
    q8, q4, q6 = q8_0_blocks(), q4_k_blocks(), q6_k_blocks()
    assert q8.size == 8 * 34 and q4.size == 16 * 144 and q6.size == 16 * 210
    more = {}
    for kind, tag in (("q4_0", 2), ("q4_1", 3), ("q5_0", 6), ("q5_1", 7)):
        raw = small_blocks(kind)
        assert raw.size == 16 * npref.BLOCK_BYTES[tag]
        more[f"{kind}_raw"], more[f"{kind}_expected"] = raw, npref.DEQUANT[tag](raw)
    q8k, q5k = q8_k_blocks(), q5_k_blocks()
    assert q8k.size == 16 * 292 and q5k.size == 16 * 176
    np.savez_compressed(
        os.path.join(HERE, "dequant_fixtures.npz"),
        q8_0_raw=q8, q8_0_expected=npref.dequant_q8_0(q8),
        q4_k_raw=q4, q4_k_expected=npref.dequant_q4_k(q4),
        q6_k_raw=q6, q6_k_expected=npref.dequant_q6_k(q6),
        q8_k_raw=q8k, q8_k_expected=npref.dequant_q8_k(q8k),
        q5_k_raw=q5k, q5_k_expected=npref.dequant_q5_k(q5k), **more)
    print("wrote dequant_fixtures.npz")


if __name__ == "__main__":
    main()

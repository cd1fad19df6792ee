"""Independent numpy restatements used to pin the C oracle.

These follow ggml's published dequantizers (dequantize_row_q8_0 / q4_K / q6_K)
in vectorised form: a different code shape from oracle/wgml_oracle.c, so a
wrong index, shift or sign in either one shows up as a bit mismatch.  Every
arithmetic step is done in float32 with one rounding per operation, as the
reference's scalar Rust code does.
"""
from __future__ import annotations

import numpy as np

f32 = np.float32


def half_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float32)


def dequant_q8_0(raw: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 34)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    qs = b[:, 2:].view(np.int8).astype(np.float32)
    return (qs * d[:, None]).astype(np.float32).reshape(-1)


def _scale_min_k4(scales: np.ndarray):
    """scales: (nb, 12) uint8 -> sc, m: (nb, 8) uint8 (ggml get_scale_min_k4)."""
    s = scales.astype(np.uint8)
    sc = np.empty((s.shape[0], 8), dtype=np.uint8)
    m = np.empty_like(sc)
    sc[:, :4] = s[:, 0:4] & 63
    m[:, :4] = s[:, 4:8] & 63
    sc[:, 4:] = (s[:, 8:12] & 0x0F) | ((s[:, 0:4] >> 6) << 4)
    m[:, 4:] = (s[:, 8:12] >> 4) | ((s[:, 4:8] >> 6) << 4)
    return sc, m


def dequant_q4_k(raw: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 144)
    nb = b.shape[0]
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    dmin = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])
    sc, m = _scale_min_k4(b[:, 4:16])
    qs = b[:, 16:].reshape(nb, 4, 32)
    # sub-block 2j = low nibbles of group j, 2j+1 = high nibbles
    q = np.empty((nb, 8, 32), dtype=np.float32)
    q[:, 0::2, :] = (qs & 0x0F).astype(np.float32)
    q[:, 1::2, :] = (qs >> 4).astype(np.float32)
    dl = (d[:, None] * sc.astype(np.float32)).astype(np.float32)     # d * sc
    ml = (dmin[:, None] * m.astype(np.float32)).astype(np.float32)   # min * m
    prod = (dl[:, :, None] * q).astype(np.float32)
    return (prod - ml[:, :, None]).astype(np.float32).reshape(-1)


def dequant_q6_k(raw: np.ndarray) -> np.ndarray:
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 210)
    nb = b.shape[0]
    ql = b[:, 0:128].reshape(nb, 2, 64)
    qh = b[:, 128:192].reshape(nb, 2, 32)
    sc = b[:, 192:208].view(np.int8).reshape(nb, 2, 8).astype(np.float32)
    d = half_bits_to_f32(b[:, 208:210].copy().view(np.uint16)[:, 0])
    out = np.empty((nb, 2, 4, 32), dtype=np.float32)
    lo = [ql[:, :, 0:32] & 0x0F, ql[:, :, 32:64] & 0x0F, ql[:, :, 0:32] >> 4, ql[:, :, 32:64] >> 4]
    for k in range(4):
        hi = (qh >> (2 * k)) & 3
        q = (lo[k] | (hi << 4)).astype(np.int16) - 32          # (nb, 2, 32)
        # scale index: is = l // 16, + 2k
        s = np.repeat(sc[:, :, 2 * k:2 * k + 2], 16, axis=2)   # (nb, 2, 32)
        ds = (d[:, None, None] * s).astype(np.float32)         # d * scale
        out[:, :, k, :] = (ds * q.astype(np.float32)).astype(np.float32)
    return out.reshape(-1)


def _nibbles_5bit(b_qs: np.ndarray, qh_bytes: np.ndarray):
    """qs: (nb, 16) uint8, qh: (nb, 4) uint8 -> two (nb, 16) arrays of 5-bit values
    (elements 0..15 and 16..31 of a 32-element block; ggml dequantize_row_q5_0/q5_1)."""
    qh = qh_bytes.copy().view(np.uint32)[:, 0].astype(np.uint64)
    j = np.arange(16, dtype=np.uint64)
    hi0 = ((qh[:, None] >> j) & 1).astype(np.uint8)          # bit j
    hi1 = ((qh[:, None] >> (j + 16)) & 1).astype(np.uint8)   # bit j + 16
    return (b_qs & 0x0F) | (hi0 << 4), (b_qs >> 4) | (hi1 << 4)


def dequant_q4_0(raw):
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 18)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])[:, None]
    q = np.concatenate([b[:, 2:] & 0x0F, b[:, 2:] >> 4], axis=1).astype(np.int16) - 8
    return (q.astype(np.float32) * d).astype(np.float32).reshape(-1)


def dequant_q4_1(raw):
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 20)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])[:, None]
    m = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])[:, None]
    q = np.concatenate([b[:, 4:] & 0x0F, b[:, 4:] >> 4], axis=1).astype(np.float32)
    return ((q * d).astype(np.float32) + m).astype(np.float32).reshape(-1)


def dequant_q5_0(raw):
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 22)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])[:, None]
    lo, hi = _nibbles_5bit(b[:, 6:], b[:, 2:6])
    q = np.concatenate([lo, hi], axis=1).astype(np.int16) - 16
    return (q.astype(np.float32) * d).astype(np.float32).reshape(-1)


def dequant_q5_1(raw):
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 24)
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])[:, None]
    m = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])[:, None]
    lo, hi = _nibbles_5bit(b[:, 8:], b[:, 4:8])
    q = np.concatenate([lo, hi], axis=1).astype(np.float32)
    return ((q * d).astype(np.float32) + m).astype(np.float32).reshape(-1)


def dequant_q8_k(raw):
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 292)
    d = b[:, 0:4].copy().view(np.float32)[:, 0][:, None]
    q = b[:, 4:260].view(np.int8).astype(np.float32)
    return (d * q).astype(np.float32).reshape(-1)


def dequant_q5_k(raw):
    b = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1, 176)
    nb = b.shape[0]
    d = half_bits_to_f32(b[:, 0:2].copy().view(np.uint16)[:, 0])
    dmin = half_bits_to_f32(b[:, 2:4].copy().view(np.uint16)[:, 0])
    sc, m = _scale_min_k4(b[:, 4:16])
    qh = b[:, 16:48]                      # (nb, 32): bit s of qh[l] is the 5th bit of sub-block s
    qs = b[:, 48:].reshape(nb, 4, 32)
    q = np.empty((nb, 8, 32), dtype=np.float32)
    for s_ in range(8):
        nib = (qs[:, s_ // 2, :] & 0x0F) if s_ % 2 == 0 else (qs[:, s_ // 2, :] >> 4)
        q[:, s_, :] = (nib + (((qh >> s_) & 1) << 4)).astype(np.float32)
    dl = (d[:, None] * sc.astype(np.float32)).astype(np.float32)
    ml = (dmin[:, None] * m.astype(np.float32)).astype(np.float32)
    return ((dl[:, :, None] * q).astype(np.float32) - ml[:, :, None]).astype(np.float32).reshape(-1)


def dequant_f16(raw):
    return half_bits_to_f32(np.ascontiguousarray(raw, dtype=np.uint8).view(np.uint16))


DEQUANT = {1: dequant_f16, 2: dequant_q4_0, 3: dequant_q4_1, 6: dequant_q5_0, 7: dequant_q5_1,
           8: dequant_q8_0, 12: dequant_q4_k, 13: dequant_q5_k, 14: dequant_q6_k, 15: dequant_q8_k}
BLOCK_BYTES = {1: 2, 2: 18, 3: 20, 6: 22, 7: 24, 8: 34, 12: 144, 13: 176, 14: 210, 15: 292}
BLOCK_ELEMS = {1: 1, 2: 32, 3: 32, 6: 32, 7: 32, 8: 32, 12: 256, 13: 256, 14: 256, 15: 256}
# byte offsets of the f16 scale fields of a block (forced finite in random blocks)
_HALF_FIELDS = {1: (0,), 2: (0,), 3: (0, 2), 6: (0,), 7: (0, 2), 8: (0,), 12: (0, 2), 13: (0, 2),
                14: (208,), 15: ()}


def random_blocks(qtype: int, nblocks: int, seed: int) -> np.ndarray:
    """Random block *bits* (as wgml-bench does, ops/gemv_quant.rs:83-101) with
    the half-precision scale fields forced finite and moderate (exponent bits
    in 1..24, i.e. |d| < 1024) so that outputs are finite numbers."""
    rng = np.random.default_rng(seed)
    raw = rng.integers(0, 256, size=(nblocks, BLOCK_BYTES[qtype]), dtype=np.uint8)

    def fix_half(col: int):
        h = raw[:, col:col + 2].copy().view(np.uint16)[:, 0]
        exp = (h >> 10) & 0x1F
        exp = (exp % 24) + 1
        h = (h & 0x83FF) | (exp.astype(np.uint16) << 10)
        raw[:, col:col + 2] = h.view(np.uint8).reshape(-1, 2)

    for col in _HALF_FIELDS[qtype]:
        fix_half(col)
    if qtype == 15:  # Q8_K: d is an f32; draw it uniformly in [-4, 4)
        d = (rng.random(nblocks, dtype=np.float32) * 8 - 4).astype(np.float32)
        raw[:, 0:4] = d.view(np.uint8).reshape(-1, 4)
    return raw.reshape(-1)


# ---- simple encoders for the formats the library's quantizer does not write -------------
# (test inputs only: any valid block is a fair input, parity always compares both sides on
# identical bytes; these round to nearest with the obvious scales, nothing more)

def _f16(a):
    return np.asarray(a, dtype=np.float32).astype(np.float16)


def encode_simple(qtype: int, x) -> np.ndarray:
    """x (float32, length a multiple of the block) -> GGUF block bytes of Q4_0 / Q4_1 / Q5_0 /
    Q5_1 / Q5_K / Q8_K."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if qtype in (2, 3, 6, 7):
        xb = x.reshape(-1, 32)
        nb = xb.shape[0]
        five = qtype in (6, 7)
        levels = 31 if five else 15
        if qtype in (3, 7):  # d q + m
            mn = xb.min(axis=1)
            d = _f16((xb.max(axis=1) - mn) / levels)
            m = _f16(mn)
            df = np.where(d.astype(np.float32) == 0, 1, d.astype(np.float32))
            q = np.clip(np.rint((xb - m.astype(np.float32)[:, None]) / df[:, None]), 0, levels).astype(np.uint8)
            head = np.concatenate([d.view(np.uint8).reshape(nb, 2), m.view(np.uint8).reshape(nb, 2)], axis=1)
        else:  # d (q - 8) or d (q - 16)
            off = 16 if five else 8
            d = _f16(np.abs(xb).max(axis=1) / (off - 1))
            df = np.where(d.astype(np.float32) == 0, 1, d.astype(np.float32))
            q = np.clip(np.rint(xb / df[:, None]) + off, 0, levels).astype(np.uint8)
            head = d.view(np.uint8).reshape(nb, 2)
        qs = (q[:, :16] & 15) | ((q[:, 16:] & 15) << 4)
        parts = [head]
        if five:
            bits = (q >> 4).astype(np.uint32)
            qh = (bits << np.arange(32, dtype=np.uint32)[None, :]).sum(axis=1).astype(np.uint32)
            parts.append(qh.view(np.uint8).reshape(nb, 4))
        parts.append(qs.astype(np.uint8))
        return np.ascontiguousarray(np.concatenate(parts, axis=1)).reshape(-1)
    if qtype == 15:
        xb = x.reshape(-1, 256)
        nb = xb.shape[0]
        d = (np.abs(xb).max(axis=1) / 127).astype(np.float32)
        df = np.where(d == 0, 1, d)
        q = np.clip(np.rint(xb / df[:, None]), -127, 127).astype(np.int8)
        bsums = q.reshape(nb, 16, 16).astype(np.int16).sum(axis=2).astype(np.int16)
        return np.ascontiguousarray(np.concatenate(
            [d.view(np.uint8).reshape(nb, 4), q.view(np.uint8), bsums.view(np.uint8).reshape(nb, 32)],
            axis=1)).reshape(-1)
    if qtype == 13:
        xb = x.reshape(-1, 8, 32)
        nb = xb.shape[0]
        mn = np.maximum(0, -xb.min(axis=2))                    # (nb, 8) minima, as positive offsets
        sc = (xb.max(axis=2) + mn) / 31
        d = _f16(sc.max(axis=1) / 63)
        dmin = _f16(mn.max(axis=1) / 63)
        df = np.where(d.astype(np.float32) == 0, 1, d.astype(np.float32))[:, None]
        mf = np.where(dmin.astype(np.float32) == 0, 1, dmin.astype(np.float32))[:, None]
        ls = np.clip(np.rint(sc / df), 0, 63).astype(np.uint8)
        lm = np.clip(np.rint(mn / mf), 0, 63).astype(np.uint8)
        step = (d.astype(np.float32)[:, None] * ls.astype(np.float32))
        step = np.where(step == 0, 1, step)
        q = np.clip(np.rint((xb + (dmin.astype(np.float32)[:, None] * lm)[:, :, None]) / step[:, :, None]),
                    0, 31).astype(np.uint8)
        scales = np.zeros((nb, 12), dtype=np.uint8)
        for j in range(8):  # the packing get_scale_min_k4 reads (quantization.rs:381-389)
            if j < 4:
                scales[:, j] |= ls[:, j]
                scales[:, j + 4] |= lm[:, j]
            else:
                scales[:, j + 4] |= (ls[:, j] & 15) | ((lm[:, j] & 15) << 4)
                scales[:, j - 4] |= (ls[:, j] >> 4) << 6
                scales[:, j] |= (lm[:, j] >> 4) << 6
        qh = np.zeros((nb, 32), dtype=np.uint8)
        for s_ in range(8):
            qh |= ((q[:, s_, :] >> 4) << s_).astype(np.uint8)
        qs = np.empty((nb, 4, 32), dtype=np.uint8)
        for g in range(4):
            qs[:, g, :] = (q[:, 2 * g, :] & 15) | ((q[:, 2 * g + 1, :] & 15) << 4)
        return np.ascontiguousarray(np.concatenate(
            [d.view(np.uint8).reshape(nb, 2), dmin.view(np.uint8).reshape(nb, 2), scales, qh,
             qs.reshape(nb, 128)], axis=1)).reshape(-1)
    raise ValueError(f"no simple encoder for type {qtype}")


# ---- float64 model forwards (composition check for the oracle) ---------------

def llama_forward_f64(w, tokens, rope_variant: int = 0):
    """Straight numpy float64 Llama forward over dequantized weights; returns the
    logits after consuming `tokens` at positions 0..len-1."""
    import oracle as orc

    c = w.config
    hs, kv_dim, kv_mul = c.head_size, c.kv_dim, c.n_q_heads // c.n_kv_heads

    def deq(hm):
        return orc.dequantize(hm.qtype, hm.data, hm.nrows * hm.ncols).reshape(
            hm.nrows, hm.ncols).astype(np.float64)

    L = [{k: (deq(v) if hasattr(v, "qtype") else np.asarray(v, dtype=np.float64))
          for k, v in l.items()} for l in w.layers]
    out_w = deq(w.output)
    kc = np.zeros((c.n_layers, c.seq_len, kv_dim))
    vc = np.zeros_like(kc)

    def rms(x, g):
        return x / np.sqrt((x * x).mean() + c.rms_norm_eps) * g

    logits = None
    for pos, tok in enumerate(tokens):
        x = w.token_embd[tok].astype(np.float64)
        for l, wl in enumerate(L):
            xb = rms(x, wl["attn_norm"])
            q, k, v = wl["attn_q"] @ xb, wl["attn_k"] @ xb, wl["attn_v"] @ xb
            for name, vec in (("attn_q_bias", q), ("attn_k_bias", k), ("attn_v_bias", v)):
                if name in wl:
                    vec += wl[name]
            i = np.arange(0, c.dim, 2)
            theta = float(c.rope_base_freq) ** (-(i % hs) / hs)
            ang = pos * theta
            cs, sn = np.cos(ang), np.sin(ang)
            if rope_variant == 0:
                a, b = i, i + 1
            else:
                a = i // 2 + (i // hs) * hs // 2
                b = a + hs // 2
            qa, qb = q[a].copy(), q[b].copy()
            q[a], q[b] = cs * qa - sn * qb, sn * qa + cs * qb
            nk = kv_dim // 2
            ka, kb = k[a[:nk]].copy(), k[b[:nk]].copy()
            k[a[:nk]], k[b[:nk]] = cs[:nk] * ka - sn[:nk] * kb, sn[:nk] * ka + cs[:nk] * kb
            kc[l, pos], vc[l, pos] = k, v
            att_out = np.zeros(c.dim)
            for h in range(c.n_q_heads):
                g = h // kv_mul
                qh = q[h * hs:(h + 1) * hs]
                s = kc[l, :pos + 1, g * hs:(g + 1) * hs] @ qh / np.sqrt(hs)
                p = np.exp(s - s.max())
                p /= p.sum()
                att_out[h * hs:(h + 1) * hs] = p @ vc[l, :pos + 1, g * hs:(g + 1) * hs]
            x = x + wl["attn_output"] @ att_out
            xb = rms(x, wl["ffn_norm"])
            g_, u_ = wl["ffn_gate"] @ xb, wl["ffn_up"] @ xb
            x = x + wl["ffn_down"] @ (u_ * (g_ / (1 + np.exp(-g_))))
        logits = out_w @ rms(x, w.output_norm.astype(np.float64))
    return logits


def gpt2_forward_f64(w, tokens):
    import oracle as orc

    p = w.params
    n, hs = p.n_embd, p.n_embd // p.n_head

    def deq(hm):
        return orc.dequantize(hm.qtype, hm.data, hm.nrows * hm.ncols).reshape(
            hm.nrows, hm.ncols).astype(np.float64)

    L = [{k: (deq(v) if hasattr(v, "qtype") else np.asarray(v, dtype=np.float64))
          for k, v in l.items()} for l in w.layers]
    head = deq(w.lm_head)
    kc = np.zeros((p.n_layer, p.n_seq, n))
    vc = np.zeros_like(kc)

    def ln(x, g, b):
        mu = x.mean()
        return (x - mu) / np.sqrt(((x - mu) ** 2).mean() + 1e-5) * g + b

    logits = None
    for pos, tok in enumerate(tokens):
        x = w.wte[tok].astype(np.float64) + w.wpe[pos].astype(np.float64)
        for l, wl in enumerate(L):
            cur = ln(x, wl["ln_1_g"], wl["ln_1_b"])
            qkv = wl["attn_w"] @ cur + wl["attn_b"]
            q, kc[l, pos], vc[l, pos] = qkv[:n], qkv[n:2 * n], qkv[2 * n:]
            att = np.zeros(n)
            for h in range(p.n_head):
                sl = slice(h * hs, (h + 1) * hs)
                s = kc[l, :pos + 1, sl] @ q[sl] / np.sqrt(hs)
                pr = np.exp(s - s.max())
                pr /= pr.sum()
                att[sl] = pr @ vc[l, :pos + 1, sl]
            x = x + wl["attn_proj_w"] @ att + wl["attn_proj_b"]
            cur = ln(x, wl["ln_2_g"], wl["ln_2_b"])
            hdn = wl["mlp_fc_w"] @ cur + wl["mlp_fc_b"]
            hdn = 0.5 * hdn * (1 + np.tanh(0.7978845608028654 * hdn * (1 + 0.044715 * hdn * hdn)))
            x = x + wl["mlp_proj_w"] @ hdn + wl["mlp_proj_b"]
        logits = head @ ln(x, w.ln_f_g.astype(np.float64), w.ln_f_b.astype(np.float64))
    return logits

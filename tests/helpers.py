"""Shared test utilities: deterministic generators shaped like the reference's test helpers,
and an INDEPENDENT numpy/f64 restatement of the GGUF block decoders (written from ggml's
published dequantize_row_* loops, not from the oracle) used to pin the oracle."""
from __future__ import annotations

import numpy as np

F32, F16, BF16 = 0, 1, 2
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2K, Q3K, Q4K, Q5K, Q6K = 5, 6, 7, 8, 9, 10, 11, 12, 13, 14
IQ1_S, IQ1_M, IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S = 15, 16, 17, 18, 19, 20, 21
IQ4_NL, IQ4_XS, TQ1_0, TQ2_0, Q2_0, MXFP4, NVFP4 = 22, 23, 24, 25, 27, 28, 29
GRID_IQUANTS = (IQ1_S, IQ1_M, IQ2_XXS, IQ2_XS, IQ2_S, IQ3_XXS, IQ3_S)   # groups of 8 elements drawn from a lattice codebook
SCALE_CODE = (IQ4_NL, IQ4_XS, TQ1_0, TQ2_0, Q2_0, MXFP4, NVFP4)   # value = scale * small signed code
BLOCK = {IQ4_NL: (32, 18), IQ4_XS: (256, 136), TQ1_0: (256, 54), TQ2_0: (256, 66), Q2_0: (64, 18), MXFP4: (32, 17),
         NVFP4: (64, 36),
         IQ1_S: (256, 50), IQ1_M: (256, 56), IQ2_XXS: (256, 66), IQ2_XS: (256, 74), IQ2_S: (256, 82), IQ3_XXS: (256, 98),
         IQ3_S: (256, 110),
         Q8_0: (32, 34), Q4K: (256, 144), Q6K: (256, 210), F32: (1, 4), F16: (1, 2), BF16: (1, 2),
         Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q2K: (256, 84), Q3K: (256, 110), Q5K: (256, 176)}
# byte offsets of the f16 scale fields inside a block
F16_SLOTS = {Q4_0: (0,), Q4_1: (0, 2), Q5_0: (0,), Q5_1: (0, 2), Q8_0: (0,), Q2K: (80, 82), Q3K: (108,), Q4K: (0, 2),
             Q5K: (0, 2), Q6K: (208,), IQ4_NL: (0,), IQ4_XS: (0,), TQ1_0: (52,), TQ2_0: (64,), Q2_0: (0,),
             IQ1_S: (0,), IQ2_XXS: (0,), IQ2_XS: (0,), IQ2_S: (0,), IQ3_XXS: (0,), IQ3_S: (0,)}


# ---- generators of the reference's tests ------------------------------------------------
def lcg_bytes_blocks(seed: int, nblk: int, nbytes: int) -> np.ndarray:
    """lcg_bytes(seed ^ block_index, nbytes) for every block
    (crates/infr-testkit/src/lib.rs:49-56, :106-123), vectorised over blocks."""
    s = (np.uint32(seed) ^ np.arange(nblk, dtype=np.uint32)).astype(np.uint64)
    out = np.empty((nblk, nbytes), np.uint8)
    for i in range(nbytes):
        s = (s * np.uint64(1664525) + np.uint64(1013904223)) & np.uint64(0xFFFFFFFF)
        out[:, i] = (s >> np.uint64(16)).astype(np.uint8)
    return out


def f16_bytes(v: float) -> np.ndarray:
    return np.array([v], np.float16).view(np.uint8)


def iq1m_set_d(blk: np.ndarray, v: float) -> None:
    """IQ1_M has no d field: the f16 is cut into four nibbles that sit on top of the four u16 scale words
    (the inverse of the extraction at crates/infr-gguf/src/dequant.rs:854-856)."""
    bits = int(np.array([v], np.float16).view(np.uint16)[0])
    for i in range(4):
        blk[:, 48 + 2 * i + 1] = (blk[:, 48 + 2 * i + 1] & 0x0F) | (((bits >> (4 * i)) & 0xF) << 4)


def synth_weight(dtype: int, n_elem: int, seed: int) -> np.ndarray:
    """Valid blocks with LCG payload and sane f16 scales (testkit synth_weight + synth_scales;
    same bytes as crates/infr-metal/tests/parity.rs:426-451 for Q4_K / Q6_K)."""
    be, bb = BLOCK[dtype]
    assert n_elem % be == 0
    nblk = n_elem // be
    if dtype == Q4K:
        blk = np.empty((nblk, 144), np.uint8)
        blk[:, 4:] = lcg_bytes_blocks(seed, nblk, 140)
        blk[:, 0:2] = f16_bytes(0.05)
        blk[:, 2:4] = f16_bytes(0.10)
    elif dtype == Q6K:
        blk = np.empty((nblk, 210), np.uint8)
        blk[:, :208] = lcg_bytes_blocks(seed, nblk, 208)
        blk[:, 208:210] = f16_bytes(0.03)
    elif dtype == Q8_0:
        blk = lcg_bytes_blocks(seed, nblk, 34)
        blk[:, 0:2] = f16_bytes(0.01)
    elif dtype == MXFP4:
        # LCG nibbles, shared exponents 2^-11 .. 2^-8 (byte 117..120)
        blk = lcg_bytes_blocks(seed, nblk, bb)
        blk[:, 0] = 117 + (blk[:, 0] & 3)
    elif dtype == NVFP4:
        # LCG nibbles, the four sub-block scales with exponent field 0..3 (subnormal and normal, up to 2^-4)
        blk = lcg_bytes_blocks(seed, nblk, bb)
        blk[:, 0:4] &= 0x1F
    elif dtype == IQ1_M:
        blk = lcg_bytes_blocks(seed, nblk, bb)
        iq1m_set_d(blk, 0.03)   # the d the reference's own IQ1_M test writes (crates/infr-core/src/decode_spec.rs:554)
    elif dtype in F16_SLOTS:
        # the remaining affine formats: LCG payload everywhere, then finite scales of either sign
        blk = lcg_bytes_blocks(seed, nblk, bb)
        for k, off in enumerate(F16_SLOTS[dtype]):
            blk[:, off:off + 2] = f16_bytes(0.02 if k == 0 else -0.07)
    else:
        raise ValueError(dtype)
    return blk.reshape(-1)


def centred_weight(dtype: int, n_elem: int, seed: int, band: float = 0.02) -> np.ndarray:
    """synth_weight with the f16 scale fields chosen so that random codes decode to values of mean ~0 and
    magnitude ~band, like trained weights: the min term of the formats that have one cancels the mean of
    the scaled codes (Q4_1: m = -7.5 d; Q5_1: -15.5 d; Q2_K: dmin = 1.5 d; Q4_K, Q5_K: dmin = mean code * d)."""
    blk = synth_weight(dtype, n_elem, seed).reshape(-1, BLOCK[dtype][1])
    if dtype in (MXFP4, NVFP4):   # symmetric books, scales already of that order
        return blk.reshape(-1)
    if dtype == IQ1_M:            # ternary grid times an odd multiplier of mean 8
        iq1m_set_d(blk, band / 8)
        return blk.reshape(-1)
    # (d, second scale) per format; code ranges: q4 0..15, q5 0..31, 6-bit sub-scales mean 31.5, 4-bit 7.5
    d2 = {Q4_0: (band / 4,), Q5_0: (band / 8,), Q8_0: (band / 64,), Q4_1: (band / 4, -7.5 * band / 4),
          Q5_1: (band / 8, -15.5 * band / 8), Q2K: (band / 8, 1.5 * band / 8), Q3K: (band / 32,),
          Q4K: (band / 128, 7.5 * band / 128), Q5K: (band / 256, 15.5 * band / 256), Q6K: (band / 1024,),
          IQ4_NL: (band / 64,), IQ4_XS: (band / 1024,), TQ1_0: (band,), TQ2_0: (band,), Q2_0: (band,),
          # signed lattice magnitudes (~25, ~30, ~8, ~1) times a sub-block multiplier of mean 2, 4, 16, 8
          IQ2_XXS: (band / 64,), IQ2_XS: (band / 64,), IQ2_S: (band / 64,), IQ3_XXS: (band / 128,), IQ3_S: (band / 128,),
          IQ1_S: (band / 8,)}[dtype]
    for off, v in zip(F16_SLOTS[dtype], d2):
        blk[:, off:off + 2] = f16_bytes(v)
    return blk.reshape(-1)


def rand_f32(n: int, seed: int) -> np.ndarray:
    """crates/infr-metal/tests/parity.rs:15-25: 64-bit LCG, top 24 bits -> [-1, 1)."""
    out = np.empty(n, np.float32)
    s = seed & 0xFFFFFFFFFFFFFFFF
    for i in range(n):
        s = (s * 6364136223846793005 + 1442695040888963407) & 0xFFFFFFFFFFFFFFFF
        out[i] = np.float32(np.float32(s >> 40) / np.float32(1 << 24)) * np.float32(2.0) - np.float32(1.0)
    return out


def gen(n: int, salt: int) -> np.ndarray:
    """crates/infr-llama/tests/seam_op_parity.rs:257-261."""
    i = np.arange(n, dtype=np.int64)
    return (((i * 13 + salt) % 29).astype(np.float32) - np.float32(14.0)) * np.float32(0.05)


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    """The reference's test-local Q8_0 quantiser (crates/infr-metal/tests/parity.rs:271-287)."""
    w = np.asarray(w, np.float32).reshape(-1, 32)
    amax = np.abs(w).max(axis=1)
    d = np.where(amax > 0, amax / np.float32(127.0), np.float32(0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(d[:, None] > 0, w / d[:, None], 0).astype(np.float32)
    q = np.clip(np.sign(q) * np.floor(np.abs(q) + np.float32(0.5)), -127, 127).astype(np.int8)  # round half away
    out = np.empty((w.shape[0], 34), np.uint8)
    out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


# ---- independent decoders (ggml's dequantize_row_q8_0 / q4_K / q6_K), exact in f64 --------
def _f16(b: np.ndarray) -> np.ndarray:
    # x87 extended precision (64-bit significand): d*sc*q - dmin*m needs up to ~61 bits when the
    # two f16 scales sit at opposite ends of the f16 exponent range, so f64 could round it twice.
    return np.ascontiguousarray(b).view(np.float16).astype(np.longdouble).reshape(-1)


def ggml_dequant(dtype: int, data: np.ndarray) -> np.ndarray:
    """Returns the EXACT decoded values (x87 extended); one cast to f32 is the single rounding
    the reference's f32 expression `sc*code + mn` performs (both products are exact there)."""
    data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
    if dtype == F32:
        return data.view(np.float32).astype(np.float64)
    if dtype == F16:
        return data.view(np.float16).astype(np.float64)
    if dtype == BF16:
        return (data.view(np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    be, bb = BLOCK[dtype]
    blk = data.reshape(-1, bb)
    nb = blk.shape[0]
    if dtype == Q8_0:
        d = _f16(blk[:, 0:2])
        q = blk[:, 2:].view(np.int8).astype(np.longdouble)
        # the reference's affine form d*(q+128) + d*(-128): a cancelling sum is +0.0, never -0.0
        return ((q + 128) * d[:, None] + (d * -128)[:, None]).reshape(-1)
    if dtype == Q4K:
        d = _f16(blk[:, 0:2])
        dmin = _f16(blk[:, 2:4])
        sc_b = blk[:, 4:16].astype(np.int64)
        qs = blk[:, 16:144].astype(np.int64)
        y = np.empty((nb, 256), np.longdouble)
        for is_ in range(8):  # ggml: for j in 0..QK_K step 64 { is, is+1 } with q += 32 per step
            if is_ < 4:
                sc = sc_b[:, is_] & 63
                m = sc_b[:, is_ + 4] & 63
            else:
                sc = (sc_b[:, is_ + 4] & 0xF) | ((sc_b[:, is_ - 4] >> 6) << 4)
                m = (sc_b[:, is_ + 4] >> 4) | ((sc_b[:, is_] >> 6) << 4)
            q = qs[:, (is_ // 2) * 32:(is_ // 2) * 32 + 32]
            nib = (q & 0xF) if is_ % 2 == 0 else (q >> 4)
            y[:, is_ * 32:(is_ + 1) * 32] = (d * sc)[:, None] * nib - (dmin * m)[:, None]
        return y.reshape(-1)
    if dtype == Q6K:
        ql = blk[:, 0:128].astype(np.int64)
        qh = blk[:, 128:192].astype(np.int64)
        sc = blk[:, 192:208].view(np.int8).astype(np.int64)
        d = _f16(blk[:, 208:210])
        y = np.empty((nb, 256), np.longdouble)
        for n in range(2):  # ggml: for n in 0..QK_K step 128
            l = np.arange(32)
            is_ = l // 16
            qln, qhn, scn = ql[:, 64 * n:64 * n + 64], qh[:, 32 * n:32 * n + 32], sc[:, 8 * n:8 * n + 8]
            q1 = ((qln[:, l] & 0xF) | (((qhn[:, l] >> 0) & 3) << 4))
            q2 = ((qln[:, l + 32] & 0xF) | (((qhn[:, l] >> 2) & 3) << 4))
            q3 = ((qln[:, l] >> 4) | (((qhn[:, l] >> 4) & 3) << 4))
            q4 = ((qln[:, l + 32] >> 4) | (((qhn[:, l] >> 6) & 3) << 4))
            base = 128 * n
            # affine form of the reference, d*sc*q + d*(-32*sc) (ggml writes d*sc*(q-32)): same
            # value, but an exact cancellation is +0.0 here and would be -0.0 there
            y[:, base + l] = d[:, None] * scn[:, is_ + 0] * q1 + d[:, None] * (-32 * scn[:, is_ + 0])
            y[:, base + l + 32] = d[:, None] * scn[:, is_ + 2] * q2 + d[:, None] * (-32 * scn[:, is_ + 2])
            y[:, base + l + 64] = d[:, None] * scn[:, is_ + 4] * q3 + d[:, None] * (-32 * scn[:, is_ + 4])
            y[:, base + l + 96] = d[:, None] * scn[:, is_ + 6] * q4 + d[:, None] * (-32 * scn[:, is_ + 6])
        return y.reshape(-1)
    if dtype in (Q4_0, Q4_1, Q5_0, Q5_1):
        # ggml dequantize_row_q4_0 / q4_1 / q5_0 / q5_1: x0 = (qs[j] & 0xF | bit j of qh << 4), x1 = (qs[j] >> 4 |
        # bit j+16 of qh << 4); y[j] = x0, y[j+16] = x1 through d*(x - 8|16) or d*x + m.  Written in the reference's
        # affine form d*x + (d*-8 | d*-16 | m) so that an exact cancellation is +0.0 as there.
        five, has_m = dtype in (Q5_0, Q5_1), dtype in (Q4_1, Q5_1)
        d = _f16(blk[:, 0:2])
        o = 2
        m = None
        if has_m:
            m = _f16(blk[:, 2:4])
            o = 4
        qh = np.zeros(nb, np.int64)
        if five:
            qh = blk[:, o:o + 4].copy().view(np.uint32).reshape(-1).astype(np.int64)
            o += 4
        qs = blk[:, o:o + 16].astype(np.int64)
        j = np.arange(16)
        x0 = (qs & 0xF) | (((qh[:, None] >> j) & 1) << 4)
        x1 = (qs >> 4) | (((qh[:, None] >> (j + 16)) & 1) << 4)
        x = np.concatenate([x0, x1], axis=1).astype(np.longdouble)
        off = m if has_m else d * (-16 if five else -8)
        return (d[:, None] * x + off[:, None]).reshape(-1)
    if dtype == Q2K:
        # ggml dequantize_row_q2_K: 16-element group g takes scales[g] (low nibble scale, high nibble min) and the
        # 2-bit fields at shift 2*((g % 8) // 2) of qs[32*(g // 8) + 16*(g % 2) ..+16)
        scales = blk[:, 0:16].astype(np.int64)
        qs = blk[:, 16:80].astype(np.int64)
        d, dmin = _f16(blk[:, 80:82]), _f16(blk[:, 82:84])
        y = np.empty((nb, 256), np.longdouble)
        for g in range(16):
            q = (qs[:, 32 * (g // 8) + 16 * (g % 2):][:, :16] >> (2 * ((g % 8) // 2))) & 3
            y[:, 16 * g:16 * g + 16] = (d * (scales[:, g] & 0xF))[:, None] * q + (dmin * -(scales[:, g] >> 4))[:, None]
        return y.reshape(-1)
    if dtype == Q3K:
        # ggml dequantize_row_q3_K.  The sixteen 6-bit scales: low 4 bits are the nibbles of bytes 0..7 (low nibbles
        # first), high 2 bits are the 2-bit fields of bytes 8..11; value = (6-bit - 32).  Element = low 2 bits from qs
        # as in Q2_K, minus 4 unless bit (g // 2) of hmask[16*(g % 2) + l] is set.
        hm = blk[:, 0:32].astype(np.int64)
        qs = blk[:, 32:96].astype(np.int64)
        sr = blk[:, 96:108].astype(np.int64)
        d = _f16(blk[:, 108:110])
        y = np.empty((nb, 256), np.longdouble)
        for g in range(16):
            lo = (sr[:, g % 8] >> (4 if g >= 8 else 0)) & 0xF
            hi = (sr[:, 8 + g % 4] >> (2 * (g // 4))) & 3
            sc = (lo | (hi << 4)) - 32
            low2 = (qs[:, 32 * (g // 8) + 16 * (g % 2):][:, :16] >> (2 * ((g % 8) // 2))) & 3
            hbit = (hm[:, 16 * (g % 2):][:, :16] >> (g // 2)) & 1
            code = low2 + 4 * hbit
            y[:, 16 * g:16 * g + 16] = (d * sc)[:, None] * code + (d * (-4 * sc))[:, None]
        return y.reshape(-1)
    if dtype == Q5K:
        # ggml dequantize_row_q5_K: Q4_K plus a fifth bit: bit `is` of qh[l] for sub-block `is`
        d, dmin = _f16(blk[:, 0:2]), _f16(blk[:, 2:4])
        sc_b = blk[:, 4:16].astype(np.int64)
        qh = blk[:, 16:48].astype(np.int64)
        qs = blk[:, 48:176].astype(np.int64)
        y = np.empty((nb, 256), np.longdouble)
        for is_ in range(8):
            if is_ < 4:
                sc, m = sc_b[:, is_] & 63, sc_b[:, is_ + 4] & 63
            else:
                sc = (sc_b[:, is_ + 4] & 0xF) | ((sc_b[:, is_ - 4] >> 6) << 4)
                m = (sc_b[:, is_ + 4] >> 4) | ((sc_b[:, is_] >> 6) << 4)
            q = qs[:, (is_ // 2) * 32:(is_ // 2) * 32 + 32]
            nib = ((q & 0xF) if is_ % 2 == 0 else (q >> 4)) + 16 * ((qh >> is_) & 1)
            y[:, is_ * 32:(is_ + 1) * 32] = (d * sc)[:, None] * nib - (dmin * m)[:, None]
        return y.reshape(-1)
    if dtype in (IQ4_NL, IQ4_XS):
        # ggml dequantize_row_iq4_nl / iq4_xs: kvalues_iq4nl[nibble] * d (* (ls - 32), ls = 6-bit sub-block scale)
        kv = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.longdouble)
        d = _f16(blk[:, 0:2])
        if dtype == IQ4_NL:
            qs = blk[:, 2:18].astype(np.int64)
            return (np.concatenate([kv[qs & 0xF], kv[qs >> 4]], axis=1) * d[:, None]).reshape(-1)
        sh = blk[:, 2:4].copy().view(np.uint16).reshape(-1).astype(np.int64)
        sl = blk[:, 4:8].astype(np.int64)
        qs = blk[:, 8:136].astype(np.int64).reshape(nb, 8, 16)
        ib = np.arange(8)
        ls = ((sl[:, ib // 2] >> (4 * (ib % 2))) & 0xF) | (((sh[:, None] >> (2 * ib)) & 3) << 4)
        y = np.concatenate([kv[qs & 0xF], kv[qs >> 4]], axis=2) * (d[:, None] * (ls - 32))[:, :, None]
        return y.reshape(-1)
    if dtype in (MXFP4, NVFP4):
        # the 4-bit codes are E2M1 floats (sign, 2-bit exponent of bias 1, 1-bit mantissa), decoded arithmetically
        # here; the scale is E8M0 (2^(e - 127)) per 32 elements, or UE4M3 (4-bit exponent of bias 7, 3-bit mantissa,
        # 0x00 and the NaN code 0x7F giving 0) per 16 elements
        def e2m1(q):
            e, m = (q >> 1) & 3, q & 1
            mag = np.where(e == 0, m * 0.5, (1 + m * 0.5) * np.exp2(e - 1.0))
            return np.where(q & 8, -mag, mag).astype(np.longdouble) + 0.0   # ggml's integer table has no -0: code 8 is +0
        if dtype == MXFP4:
            scale = np.ldexp(np.longdouble(1), blk[:, 0].astype(np.int64) - 127)
            qs = blk[:, 1:17].astype(np.int64)
            return (np.concatenate([e2m1(qs & 0xF), e2m1(qs >> 4)], axis=1) * scale[:, None]).reshape(-1)
        sb = blk[:, 0:4].astype(np.int64)
        e, m = (sb >> 3) & 0xF, sb & 7
        scale = np.where(e == 0, np.ldexp(m.astype(np.longdouble), -9), np.ldexp((8 + m).astype(np.longdouble), e - 10))
        scale = np.where((sb == 0) | (sb == 0x7F), 0, scale)
        qs = blk[:, 4:36].astype(np.int64).reshape(nb, 4, 8)
        return (np.concatenate([e2m1(qs & 0xF), e2m1(qs >> 4)], axis=2) * scale[:, :, None]).reshape(-1)
    if dtype == TQ2_0:
        # ggml dequantize_row_tq2_0: two runs of 32 bytes, their four 2-bit fields field-major
        qs = blk[:, 0:64].astype(np.int64).reshape(nb, 2, 1, 32)
        q = (qs >> (2 * np.arange(4)).reshape(1, 1, 4, 1)) & 3
        return ((q - 1).reshape(nb, 256) * _f16(blk[:, 64:66])[:, None]).reshape(-1)
    if dtype == Q2_0:
        q = (blk[:, 2:18].astype(np.int64)[:, :, None] >> (2 * np.arange(4))) & 3   # fields of a byte are consecutive elements
        return ((q - 1).reshape(nb, 64) * _f16(blk[:, 0:2])[:, None]).reshape(-1)
    if dtype == TQ1_0:
        # ggml dequantize_row_tq1_0: a byte q holds five ternary digits as the fraction q / 256 in base 3, first digit
        # = floor(3 * frac(q / 256)), digit n = the same of frac(q * 3^n / 256); runs of 32, 16 and 4 bytes, digit-major
        def digits(b, n):
            q = b.astype(np.int64)[:, None, :] * (3 ** np.arange(n)).reshape(1, n, 1)
            return ((q % 256) * 3) // 256
        y = np.concatenate([digits(blk[:, 0:32], 5).reshape(nb, -1), digits(blk[:, 32:48], 5).reshape(nb, -1),
                            digits(blk[:, 48:52], 4).reshape(nb, -1)], axis=1)
        return ((y - 1) * _f16(blk[:, 52:54])[:, None]).reshape(-1)
    if dtype in GRID_IQUANTS:
        return _ggml_dequant_iquant(dtype, blk)
    raise ValueError(dtype)


# ---- lattice codebooks of the grid i-quants -------------------------------------------------
_GRID_ALPHABET = {"kIq2xxsGrid": (8, 25, 43), "kIq2xsGrid": (8, 25, 43), "kIq2sGrid": (8, 25, 43),
                  "kIq3xxsGrid": (4, 12, 20, 28, 36, 44, 52, 62), "kIq3sGrid": (1, 3, 5, 7, 9, 11, 13, 15),
                  "kIq1sGrid": (0, 1, -1)}
_GRIDS: dict = {}


def iquant_grid(name: str) -> np.ndarray:
    """Codebook `name` of moe4all_amd/csrc/iquant_grids.h widened to [entries, 8 or 4] int64 (a second reader of the
    packed table, separate from the C one the oracle and the device use)."""
    if not _GRIDS:
        import os
        import re
        path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "moe4all_amd", "csrc", "iquant_grids.h")
        for m in re.finditer(r"uint16_t (\w+)\[(\d+)\] = \{(.*?)\};", open(path).read(), re.S):
            vals = np.array([int(v, 16) for v in re.findall(r"0x[0-9a-f]+", m.group(3))], np.int64)
            assert len(vals) == int(m.group(2))
            alpha = np.array(_GRID_ALPHABET[m.group(1)], np.int64)
            bits, n = (2, 8) if len(alpha) == 3 else (3, 4)
            digits = (vals[:, None] >> (bits * np.arange(n))) & ((1 << bits) - 1)
            assert digits.max() < len(alpha)
            _GRIDS[m.group(1)] = alpha[digits]
    return _GRIDS[name]


def ksigns() -> np.ndarray:
    """ggml's ksigns_iq2xs: entry i = i with bit 7 completing an even number of one bits."""
    i = np.arange(128, dtype=np.int64)
    par = np.zeros(128, np.int64)
    for b in range(7):
        par ^= (i >> b) & 1
    return i | (par << 7)


def _signs(byte: np.ndarray) -> np.ndarray:
    """[...] sign bytes -> [..., 8] factors: bit j set means element j is negated (ggml's kmask_iq2xs[j] = 1 << j)."""
    return 1 - 2 * ((byte[..., None] >> np.arange(8)) & 1)


def _ggml_dequant_iquant(dtype: int, blk: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_iq2_xxs / iq2_xs / iq2_s / iq3_xxs / iq3_s / iq1_s / iq1_m, vectorised over blocks:
    [blocks, 8 sub-blocks of 32, 4 groups, 8 elements]."""
    nb = blk.shape[0]
    L = np.longdouble
    u8 = blk.astype(np.int64)

    def u16(a):   # [..., 2k] bytes -> [..., k] little-endian words
        return a[..., 0::2] | (a[..., 1::2] << 8)

    def u32(a):
        return a[..., 0::4] | (a[..., 1::4] << 8) | (a[..., 2::4] << 16) | (a[..., 3::4] << 24)

    l4 = np.arange(4)
    if dtype == IQ2_XXS:
        d = _f16(blk[:, 0:2])
        q = u8[:, 2:66].reshape(nb, 8, 8)
        aux1 = u32(q[:, :, 4:8])[:, :, 0]                                  # [nb, 8]
        db = d[:, None] * (L(0.5) + (aux1 >> 28)) * L(0.25)
        g = iquant_grid("kIq2xxsGrid")[q[:, :, 0:4]]                       # [nb, 8, 4, 8]
        sg = _signs(ksigns()[(aux1[:, :, None] >> (7 * l4)) & 127])
        return (db[:, :, None, None] * g * sg).reshape(-1)
    if dtype in (IQ2_XS, IQ2_S):
        d = _f16(blk[:, 0:2])
        if dtype == IQ2_XS:
            q = u16(u8[:, 2:66]).reshape(nb, 8, 4)
            g = iquant_grid("kIq2xsGrid")[q & 511]
            sg = _signs(ksigns()[q >> 9])
            sc = u8[:, 66:74]
        else:
            qs = u8[:, 2:34].reshape(nb, 8, 4)
            qh = u8[:, 66:74]
            idx = qs | ((qh[:, :, None] << (8 - 2 * l4)) & 0x300)
            g = iquant_grid("kIq2sGrid")[idx]
            sg = _signs(u8[:, 34:66].reshape(nb, 8, 4))
            sc = u8[:, 74:82]
        db = d[:, None, None] * (L(0.5) + np.stack([sc & 0xF, sc & 0xF, sc >> 4, sc >> 4], axis=2)) * L(0.25)   # [nb, 8, 4]
        return (db[:, :, :, None] * g * sg).reshape(-1)
    if dtype == IQ3_XXS:
        d = _f16(blk[:, 0:2])
        q = u8[:, 2:66].reshape(nb, 8, 4, 2)
        aux = u32(u8[:, 66:98])                                            # [nb, 8]
        db = d[:, None] * (L(0.5) + (aux >> 28)) * L(0.5)
        g = iquant_grid("kIq3xxsGrid")[q].reshape(nb, 8, 4, 8)             # the two 4-element entries side by side
        sg = _signs(ksigns()[(aux[:, :, None] >> (7 * l4)) & 127])
        return (db[:, :, None, None] * g * sg).reshape(-1)
    if dtype == IQ3_S:
        d = _f16(blk[:, 0:2])
        q = u8[:, 2:66].reshape(nb, 8, 4, 2)
        qh = u8[:, 66:74]
        hi = np.stack([(qh[:, :, None] << (8 - 2 * l4)) & 256, (qh[:, :, None] << (7 - 2 * l4)) & 256], axis=3)
        g = iquant_grid("kIq3sGrid")[q | hi].reshape(nb, 8, 4, 8)
        sg = _signs(u8[:, 74:106].reshape(nb, 8, 4))
        sc = u8[:, 106:110]
        nib = np.stack([sc & 0xF, sc >> 4], axis=2).reshape(nb, 8)
        db = d[:, None] * (1 + 2 * nib)
        return (db[:, :, None, None] * g * sg).reshape(-1)
    if dtype == IQ1_S:
        d = _f16(blk[:, 0:2])
        qs = u8[:, 2:34].reshape(nb, 8, 4)
        qh = u16(u8[:, 34:50])                                             # [nb, 8]
        dl = d[:, None] * (2 * ((qh >> 12) & 7) + 1)
        delta = np.where(qh & 0x8000, L(-0.125), L(0.125))
        g = iquant_grid("kIq1sGrid")[qs | (((qh[:, :, None] >> (3 * l4)) & 7) << 8)]
        return (dl[:, :, None, None] * (g + delta[:, :, None, None])).reshape(-1)
    if dtype == IQ1_M:
        sc = u16(u8[:, 48:56])                                             # [nb, 4]
        dbits = (sc[:, 0] >> 12) | ((sc[:, 1] >> 8) & 0x00F0) | ((sc[:, 2] >> 4) & 0x0F00) | (sc[:, 3] & 0xF000)
        d = dbits.astype(np.uint16).view(np.float16).astype(L)
        ib = np.arange(8)
        s3 = np.stack([(sc[:, ib // 2] >> (6 * (ib % 2))) & 7, (sc[:, ib // 2] >> (6 * (ib % 2) + 3)) & 7], axis=2)   # [nb, 8, 2]
        dl = (d[:, None, None] * (2 * s3 + 1))[:, :, [0, 0, 1, 1]]          # [nb, 8, 4]
        qs = u8[:, 0:32].reshape(nb, 8, 4)
        qh = u8[:, 32:48].reshape(nb, 8, 2)[:, :, [0, 0, 1, 1]]
        odd = (l4 & 1).astype(bool)
        idx = qs | np.where(odd, (qh << 4) & 0x700, (qh << 8) & 0x700)
        delta = np.where(qh & np.where(odd, 0x80, 0x08), L(-0.125), L(0.125))
        g = iquant_grid("kIq1sGrid")[idx]
        return (dl[:, :, :, None] * (g + delta[:, :, :, None])).reshape(-1)
    raise ValueError(dtype)


def tq1_0_pack(trits: np.ndarray) -> np.ndarray:
    """ggml quantize_row_tq1_0_ref's byte: five digits t0..t4 in {0, 1, 2}, most significant first, stored as
    ceil(value * 256 / 243) so that multiplying by 3^n brings digit n to the top."""
    t = np.asarray(trits, np.int64).reshape(-1, 5)
    v = t @ np.array([81, 27, 9, 3, 1])
    return ((v * 256 + 242) // 243).astype(np.uint8)


# ---- independent f64 model of Op::MoeFfn (shape of moe_ref / moe_v4_ref) -----------------
def moe_ffn_f64(x, router_w, gate_w, up_w, down_w, *, ne, n_expert, n_used, n_ff, scale=1.0, gating="softmax",
                norm_w=True, bias=None, n_groups=0, n_groups_used=0, weight_before=False, down_scale=None,
                clamp=None, act="silu", hash_ids=None):
    """x [rows, ne]; weights already decoded to float arrays (router [E,ne], gate/up [E,nff,ne],
    down [E,ne,nff]).  Plain f64 everywhere; follows the f32/f64 references in
    crates/infr-llama/tests/seam_op_parity.rs:2245-2343 and :5635-5696."""
    x = np.asarray(x, np.float64).reshape(-1, ne)
    R = np.asarray(router_w, np.float64).reshape(n_expert, ne)
    G = np.asarray(gate_w, np.float64).reshape(n_expert, n_ff, ne)
    U = np.asarray(up_w, np.float64).reshape(n_expert, n_ff, ne)
    D = np.asarray(down_w, np.float64).reshape(n_expert, ne, n_ff)
    out = np.zeros_like(x)
    sel_idx = []
    for r in range(x.shape[0]):
        logits = R @ x[r]
        if gating == "softmax":
            p = np.exp(logits - logits.max())
            p /= p.sum()
        elif gating == "sigmoid":
            p = 1.0 / (1.0 + np.exp(-logits))
        else:
            sp = np.where(logits > 20.0, logits, np.log1p(np.exp(np.minimum(logits, 700))))
            p = np.sqrt(sp)
        if hash_ids is not None:
            idx = [int(v) for v in np.asarray(hash_ids).reshape(-1, n_used)[r]]
        else:
            sel = p + (np.asarray(bias, np.float64) if bias is not None else 0.0)
            if n_groups > 1 and n_groups_used > 0:
                per = n_expert // n_groups
                gs = [np.sort(sel[g * per:(g + 1) * per])[-2:].sum() for g in range(n_groups)]
                keep = sorted(range(n_groups), key=lambda g: (-gs[g], g))[:n_groups_used]
                for g in range(n_groups):
                    if g not in keep:
                        sel[g * per:(g + 1) * per] = -np.inf
            idx = sorted(range(n_expert), key=lambda e: (-sel[e], e))[:n_used]
        w = p[idx] / max(p[idx].sum(), 1e-20) * scale if norm_w else p[idx] * scale
        sel_idx.append(idx)
        for k, e in enumerate(idx):
            wp = w[k] if weight_before else 1.0
            g = wp * (G[e] @ x[r])
            u = wp * (U[e] @ x[r])
            if clamp is not None:
                g = np.minimum(g, clamp)
                u = np.clip(u, -clamp, clamp)
            if act == "silu":
                a = g / (1.0 + np.exp(-g))
            elif act == "gelu":
                a = 0.5 * g * (1.0 + np.tanh(0.7978846 * (g + 0.044715 * g ** 3)))
            else:
                a = 1.0 / (1.0 + np.exp(-g))
            y = D[e] @ (a * u)
            if down_scale is not None:
                y = y * down_scale[e]
            out[r] += (1.0 if weight_before else w[k]) * y
    return out, np.array(sel_idx, np.int32)


def rel_l2(a, b) -> float:
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def elem_rel_err(got, want) -> float:
    """The per-element measure of the reference's device parity tests:
    |c - m| / max(|c|, 1)  (crates/infr-metal/tests/parity.rs:158-163)."""
    got, want = np.asarray(got, np.float64).ravel(), np.asarray(want, np.float64).ravel()
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1.0))) if got.size else 0.0


def max_abs(a, b) -> float:
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return float(np.max(np.abs(a - b))) if a.size else 0.0


# ---- the reference-specified cases behind tests/golden/*.npz --------------------------------
def pattern(n, mul, add):
    return ((np.arange(n, dtype=np.int64) * mul + add) & 0xFF).astype(np.uint8)


def dequant_cases():
    out = {}
    b = pattern(288, 37, 11)
    for blk in range(2):
        b[blk * 144:blk * 144 + 2] = f16_bytes(0.375)
        b[blk * 144 + 2:blk * 144 + 4] = f16_bytes(-0.125)
    out["q4k_ref_pattern"] = (Q4K, b)
    b = pattern(420, 53, 7)
    for blk in range(2):
        b[blk * 210 + 208:blk * 210 + 210] = f16_bytes(0.05)
    out["q6k_ref_pattern"] = (Q6K, b)
    for name, dt, bb in (("q8_0", Q8_0, 34), ("q4k", Q4K, 144), ("q6k", Q6K, 210)):
        out[f"{name}_all_formats_pattern"] = (dt, pattern(2 * bb, 29, 3))
    out["q8_0_lcg"] = (Q8_0, synth_weight(Q8_0, 32 * 24, 5))
    out["q4k_lcg"] = (Q4K, synth_weight(Q4K, 256 * 6, 80))
    out["q6k_lcg"] = (Q6K, synth_weight(Q6K, 256 * 6, 90))
    # the other affine formats: the same (i*29+3)&0xFF pattern (dequant.rs:1206-1230; its f16 fields happen to be
    # finite for each of them), LCG blocks, and the single blocks of the reference's known-answer tests
    for name, dt in (("q4_0", Q4_0), ("q4_1", Q4_1), ("q5_0", Q5_0), ("q5_1", Q5_1), ("q2k", Q2K), ("q3k", Q3K), ("q5k", Q5K)):
        out[f"{name}_all_formats_pattern"] = (dt, pattern(2 * BLOCK[dt][1], 29, 3))
        out[f"{name}_lcg"] = (dt, synth_weight(dt, BLOCK[dt][0] * 8, 100 + dt))
    for name, dt in (("iq4_nl", IQ4_NL), ("iq4_xs", IQ4_XS), ("tq1_0", TQ1_0), ("tq2_0", TQ2_0), ("q2_0", Q2_0),
                     ("mxfp4", MXFP4), ("nvfp4", NVFP4)):
        b = pattern(2 * BLOCK[dt][1], 29, 3)
        if dt == MXFP4:   # keep the shared exponents of the pattern inside f32 after the multiply by 12
            b[0::17] = 64 + (b[0::17] >> 1)
        out[f"{name}_pattern"] = (dt, b)
        out[f"{name}_lcg"] = (dt, synth_weight(dt, BLOCK[dt][0] * 8, 100 + dt))
    # the grid i-quants: the (i*29+3)&0xFF pattern over two blocks (IQ1_M: with the d nibbles of its own test) and
    # LCG blocks, which reach every codebook with arbitrary indices, sign bytes and multipliers
    for name, dt in (("iq1_s", IQ1_S), ("iq1_m", IQ1_M), ("iq2_xxs", IQ2_XXS), ("iq2_xs", IQ2_XS), ("iq2_s", IQ2_S),
                     ("iq3_xxs", IQ3_XXS), ("iq3_s", IQ3_S)):
        b = pattern(2 * BLOCK[dt][1], 29, 3)
        if dt == IQ1_M:
            iq1m_set_d(b.reshape(2, -1), 0.03)
        out[f"{name}_pattern"] = (dt, b)
        out[f"{name}_lcg"] = (dt, synth_weight(dt, 256 * 8, 100 + dt))
    for name, (dt, b, _) in known_answer_blocks().items():
        out[name] = (dt, b)
    return out


def known_answer_blocks():
    """The single blocks of the reference's own decoder tests with the values those tests assert
    (crates/infr-gguf/src/dequant.rs:1619-1846): name -> (dtype, bytes, {element index: value})."""
    out = {}
    b = np.zeros(84, np.uint8)          # q2k_single_block: scales 0x23, qs 0x55, d = 1, dmin = 2
    b[0] = b[1] = 0x23
    b[16:80] = 0x55
    b[80:82], b[82:84] = f16_bytes(1.0), f16_bytes(2.0)
    out["q2k_single_block"] = (Q2K, b, {i: -1.0 for i in range(32)})
    b = np.zeros(110, np.uint8)         # q3k_single_block: everything 0, d = 1 -> 128 everywhere
    b[108:110] = f16_bytes(1.0)
    out["q3k_single_block"] = (Q3K, b, {i: 128.0 for i in range(256)})
    b = np.full(18, 0x88, np.uint8)     # q4_0_single_block: d = 2, qs[0] = 0x89
    b[0:2] = f16_bytes(2.0)
    b[2] = 0x89
    out["q4_0_single_block"] = (Q4_0, b, {0: 2.0, 16: 0.0, 1: 0.0})
    b = np.zeros(20, np.uint8)          # q4_1_single_block: d = 1, m = 0.5, qs[0] = 0x30
    b[0:2], b[2:4] = f16_bytes(1.0), f16_bytes(0.5)
    b[4] = 0x30
    out["q4_1_single_block"] = (Q4_1, b, {0: 0.5, 16: 3.5})
    b = np.zeros(22, np.uint8)          # q5_0_single_block: d = 1, qh bit 0, qs[0] = 0x0F
    b[0:2] = f16_bytes(1.0)
    b[2] = 0x01
    b[6] = 0x0F
    out["q5_0_single_block"] = (Q5_0, b, {0: 15.0, 16: -16.0})
    b = np.zeros(24, np.uint8)          # q5_1_single_block: d = 2, m = -1, qs[0] = 0x1F
    b[0:2], b[2:4] = f16_bytes(2.0), f16_bytes(-1.0)
    b[8] = 0x1F
    out["q5_1_single_block"] = (Q5_1, b, {0: 29.0, 16: 1.0})
    # the scale-times-code formats (dequant.rs:1228-1432)
    b = np.zeros(18, np.uint8)          # iq4nl_single_block: d = 1, qs[0] = 0x80
    b[0:2] = f16_bytes(1.0)
    b[2] = 0x80
    out["iq4nl_single_block"] = (IQ4_NL, b, {0: -127.0, 16: 1.0})
    b = np.zeros(136, np.uint8)         # iq4xs_single_block: d = 1, everything else 0 -> -32 * -127
    b[0:2] = f16_bytes(1.0)
    out["iq4xs_single_block"] = (IQ4_XS, b, {i: 4064.0 for i in range(256)})
    b = np.zeros(17, np.uint8)          # mxfp4_single_block: e = 128, qs[0] = 0x21
    b[0], b[1] = 128, 0x21
    out["mxfp4_single_block"] = (MXFP4, b, {0: 1.0, 16: 2.0, **{i: 0.0 for i in range(1, 16)}})
    out["nvfp4_single_block"] = (NVFP4, np.zeros(36, np.uint8), {i: 0.0 for i in range(64)})
    b = np.zeros(54, np.uint8)          # tq1_0_single_block: d = 1
    b[52:54] = f16_bytes(1.0)
    out["tq1_0_single_block"] = (TQ1_0, b, {i: -1.0 for i in range(256)})
    b = np.zeros(66, np.uint8)          # tq2_0_single_block: d = 1
    b[64:66] = f16_bytes(1.0)
    out["tq2_0_single_block"] = (TQ2_0, b, {i: -1.0 for i in range(256)})
    b = np.zeros(18, np.uint8)          # q2_0_single_block: d = 0.5, qs[0] = 0b11100100
    b[0:2] = f16_bytes(0.5)
    b[2] = 0b11100100
    out["q2_0_single_block"] = (Q2_0, b, {0: -0.5, 1: 0.0, 2: 0.5, 3: 1.0, **{i: -0.5 for i in range(4, 64)}})
    # the grid i-quants (dequant.rs:1290-1308, :1355-1363, :1495-1617): all-zero payload, d = 1 -> entry 0 of the codebook,
    # no sign set, smallest multiplier
    for name, dt, v in (("iq2xxs", IQ2_XXS, 1.0), ("iq2xs", IQ2_XS, 1.0), ("iq2s", IQ2_S, 1.0), ("iq3xxs", IQ3_XXS, 1.0),
                        ("iq3s", IQ3_S, 1.0), ("iq1s", IQ1_S, -0.875)):
        b = np.zeros(BLOCK[dt][1], np.uint8)
        b[0:2] = f16_bytes(1.0)
        out[f"{name}_single_block"] = (dt, b, {i: v for i in range(256)})
    out["iq1m_single_block"] = (IQ1_M, np.zeros(56, np.uint8), {i: 0.0 for i in range(256)})
    return out


def moe_cases():
    cases = {}
    # seam_op_parity.rs moe_sqrt_softplus_parity
    ne, E, K, nff = 32, 6, 2, 32
    lead = np.array([24.0, 1.0, 0.75, 0.5, -1.5, -1.0], np.float32)
    router = np.zeros((E, ne), np.float32)
    router[:, 0] = lead
    cases["sqrt_softplus"] = dict(ne=ne, n_expert=E, n_used=K, n_ff=nff, gating=2, x=np.ones(ne, np.float32),
                                  router=router.reshape(-1), gate=gen(E * nff * ne, 12), up=gen(E * nff * ne, 13),
                                  down=gen(E * ne * nff, 14), dtype=F32, expect_idx=[0, 1])
    # seam_op_parity.rs moe_groups_bias_parity
    E = 8
    lead = np.array([3.0, 2.5, 2.0, 1.5, 1.0, 0.9, 0.8, 0.7], np.float32)
    router = np.zeros((E, ne), np.float32)
    router[:, 0] = lead
    cases["groups_bias"] = dict(ne=ne, n_expert=E, n_used=K, n_ff=nff, gating=1, x=np.ones(ne, np.float32),
                                router=router.reshape(-1), gate=gen(E * nff * ne, 15), up=gen(E * nff * ne, 16),
                                down=gen(E * ne * nff, 17), dtype=F32,
                                bias=np.array([0, 0, 0, 0, .6, .6, .6, .6], np.float32), n_groups=2, n_groups_used=1,
                                expect_idx=[4, 5])
    # metal parity.rs moe_ffn_parity (f32, softmax)
    ne, E, K, nff = 64, 8, 2, 128
    cases["metal_f32"] = dict(ne=ne, n_expert=E, n_used=K, n_ff=nff, gating=0, x=rand_f32(ne, 60),
                              router=rand_f32(E * ne, 61), gate=rand_f32(E * nff * ne, 62),
                              up=rand_f32(E * nff * ne, 63), down=rand_f32(E * ne * nff, 64), dtype=F32)
    # metal parity.rs moe_quant_test (Q4_K seed 80, Q6_K seed 90)
    ne, E, K, nff = 256, 8, 3, 256
    for name, dt, seed in (("metal_q4k", Q4K, 80), ("metal_q6k", Q6K, 90)):
        cases[name] = dict(ne=ne, n_expert=E, n_used=K, n_ff=nff, gating=0, x=rand_f32(ne, seed),
                           router=rand_f32(E * ne, seed + 1), gate=synth_weight(dt, E * nff * ne, seed + 2),
                           up=synth_weight(dt, E * nff * ne, seed + 3), down=synth_weight(dt, E * ne * nff, seed + 4),
                           dtype=dt)
    return cases



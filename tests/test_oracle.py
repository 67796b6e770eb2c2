"""Pins the CPU oracle (oracle/infr_oracle.c) WITHOUT running the reference (Rust, not
buildable here): against the committed golden fixtures, against an independent extended-precision
decoder written from ggml's published loops, against closed forms / brute force, and against the
facts the reference's own tests state (selected experts, tolerances)."""
import os
from fractions import Fraction

import numpy as np
import pytest

import helpers as H
import oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


# ------------------------------------------------------------------ geometry / f16 / k4
def test_block_geometry_matches_ggml_formulas():
    # crates/infr-core/src/decode_spec.rs:455-504 restates ggml: Q8_0 2+32, Q4_K 2+2+12+128, Q6_K 128+64+16+2
    assert O.block_geometry(O.Q8_0) == (32, 2 + 32)
    assert O.block_geometry(O.Q4K) == (256, 2 + 2 + 12 + 128)
    assert O.block_geometry(O.Q6K) == (256, 128 + 64 + 16 + 2)
    assert O.block_geometry(O.Q4_0) == (32, 2 + 16) and O.block_geometry(O.Q4_1) == (32, 2 + 2 + 16)
    assert O.block_geometry(O.Q5_0) == (32, 2 + 4 + 16) and O.block_geometry(O.Q5_1) == (32, 2 + 2 + 4 + 16)
    assert O.block_geometry(O.Q2K) == (256, 16 + 64 + 2 + 2) and O.block_geometry(O.Q3K) == (256, 32 + 64 + 12 + 2)
    assert O.block_geometry(O.Q5K) == (256, 2 + 2 + 12 + 32 + 128)
    # decode_spec.rs:468-474, QK_K = 256
    assert O.block_geometry(O.IQ1_S) == (256, 2 + 256 // 8 + 256 // 32 * 2) and O.block_geometry(O.IQ1_M) == (256, 256 // 8 + 256 // 16 + 256 // 32)
    assert O.block_geometry(O.IQ2_XXS) == (256, 2 + 256 // 8 * 2) and O.block_geometry(O.IQ2_XS) == (256, 2 + 256 // 8 * 2 + 256 // 32)
    assert O.block_geometry(O.IQ2_S) == (256, 2 + 256 // 4 + 256 // 16) and O.block_geometry(O.IQ3_XXS) == (256, 2 + 3 * (256 // 8))
    assert O.block_geometry(O.IQ3_S) == (256, 2 + 13 * (256 // 32) + 256 // 64)
    assert O.bytes_for(O.Q4K, 768 * 2048) == 884736
    assert O.bytes_for(O.Q6K, 2048 * 768) == 1290240
    assert O.bytes_for(O.Q8_0, 768 * 2048) == 1671168
    with pytest.raises(ValueError):
        O.bytes_for(O.Q4K, 100)


def test_f16_to_f32_all_65536_values():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([O.f16_to_f32(int(v)) for v in h], np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_k4_inverts_ggml_scale_packing_exhaustively():
    """get_scale_min_k4 must invert the packing ggml's quantiser writes
    (scales[j]=ls, scales[j+4]=lm for j<4; else scales[j+4]=(ls&0xF)|((lm&0xF)<<4),
    scales[j-4]|=(ls>>4)<<6, scales[j]|=(lm>>4)<<6) for every 6-bit (ls, lm) at every j."""
    rng = np.random.default_rng(0)
    for j in range(8):
        for ls in range(64):
            for lm in range(0, 64, 3):
                other = rng.integers(0, 64, size=(8, 2))
                other[j] = (ls, lm)
                s = np.zeros(12, np.uint8)
                for jj in range(8):
                    a, b = int(other[jj][0]), int(other[jj][1])
                    if jj < 4:
                        s[jj] |= a
                        s[jj + 4] |= b
                    else:
                        s[jj + 4] = (a & 0xF) | ((b & 0xF) << 4)
                        s[jj - 4] |= (a >> 4) << 6
                        s[jj] |= (b >> 4) << 6
                for jj in range(8):
                    assert O.k4(jj, s) == (int(other[jj][0]), int(other[jj][1]))


# ------------------------------------------------------------------ dequant
def test_dequant_matches_golden_fixture_bit_for_bit():
    g = np.load(os.path.join(GOLD, "dequant.npz"))
    names = sorted({k.rsplit(".", 1)[0] for k in g.files})
    assert len(names) == 8 + 14 + 6 + 14 + 7 + 14 + 7
    for n in names:
        got = O.dequant(int(g[n + ".dtype"]), g[n + ".bytes"])
        assert np.array_equal(got.view(np.uint32), g[n + ".bits"]), n


def test_dequant_fixture_inputs_are_the_reference_test_patterns():
    g = np.load(os.path.join(GOLD, "dequant.npz"))
    for n, (dt, b) in H.dequant_cases().items():
        assert np.array_equal(g[n + ".bytes"], b) and int(g[n + ".dtype"]) == dt


def test_dequant_gives_the_values_the_reference_tests_assert():
    """The single blocks of crates/infr-gguf/src/dequant.rs:1619-1846 and the values asserted there."""
    for name, (dt, b, want) in H.known_answer_blocks().items():
        y = O.dequant(dt, b)
        for i, v in want.items():
            assert y[i] == np.float32(v), (name, i, y[i], v)


@pytest.mark.parametrize("dt,seed", [(O.Q8_0, 1), (O.Q4K, 2), (O.Q6K, 3), (O.Q4_0, 4), (O.Q4_1, 5), (O.Q5_0, 6), (O.Q5_1, 7),
                                     (O.Q2K, 8), (O.Q3K, 9), (O.Q5K, 10), (O.IQ4_NL, 11), (O.IQ4_XS, 12), (O.TQ1_0, 13),
                                     (O.TQ2_0, 14), (O.Q2_0, 15), (O.MXFP4, 16), (O.NVFP4, 17), (O.IQ1_S, 18), (O.IQ1_M, 19),
                                     (O.IQ2_XXS, 20), (O.IQ2_XS, 21), (O.IQ2_S, 22), (O.IQ3_XXS, 23), (O.IQ3_S, 24)])
def test_dequant_matches_independent_decoder_on_random_blocks(dt, seed):
    be, bb = O.block_geometry(dt)
    b = H.synth_weight(dt, be * 64, seed)
    want = H.ggml_dequant(dt, b).astype(np.float32)
    assert np.array_equal(O.dequant(dt, b).view(np.uint32), want.view(np.uint32))


def test_iquant_codebooks_are_the_reference_tables():
    """The packed codebooks, widened to one signed byte per element by the C reader (oracle, device) and by the separate
    Python reader, hash to the digests taken from crates/infr-core/src/iquant_grids.rs when the tables were packed
    (tests/golden/iquant_grids.json); the sign table is the parity rule, the mask table 1 << j."""
    import hashlib
    import json
    dig = json.load(open(os.path.join(GOLD, "iquant_grids.json")))
    names = ("kIq2xxsGrid", "kIq2xsGrid", "kIq2sGrid", "kIq3xxsGrid", "kIq3sGrid", "kIq1sGrid")
    for which, name in enumerate(names):
        g = O.grid(which)
        assert g.shape == (dig[name]["entries"], dig[name]["entry_bytes"]) == (O.GRID_SIZES[which], 8 if which in (0, 1, 2, 5) else 4)
        assert np.array_equal(g, H.iquant_grid(name)), name
        assert hashlib.sha256(g.astype(np.int8).tobytes()).hexdigest() == dig[name]["sha256"], name
    assert hashlib.sha256(bytes(O.ksigns())).hexdigest() == dig["KSIGNS_IQ2XS"]["sha256"]
    assert np.array_equal(O.ksigns(), H.ksigns())
    assert hashlib.sha256(bytes(1 << j for j in range(8))).hexdigest() == dig["KMASK_IQ2XS"]["sha256"]


def test_iquant_codebooks_have_the_structure_ggml_documents():
    """IQ2 and IQ3 codebooks are sorted lists of distinct lattice points (read as little-endian integers); every IQ2 point
    has odd coordinates of the form (8, 25, 43) ~ (1, 3, 5) * 8.5, every IQ3_S coordinate is odd, IQ1 is ternary."""
    for which in range(5):
        g = O.grid(which).astype(np.int64)
        as_int = (g << (8 * np.arange(g.shape[1]))).sum(axis=1)
        assert (np.diff(as_int) > 0).all(), which
    assert set(np.unique(O.grid(0))) == set(np.unique(O.grid(1))) == set(np.unique(O.grid(2))) == {8, 25, 43}
    assert set(np.unique(O.grid(3))) == {4, 12, 20, 28, 36, 44, 52, 62}
    assert set(np.unique(O.grid(4))) == set(range(1, 16, 2))
    g1 = O.grid(5)
    assert set(np.unique(g1)) == {-1, 0, 1} and len({tuple(r) for r in g1}) == 2048
    assert (g1[0] == -1).all()     # the entry the reference's IQ1_S test decodes (dequant.rs:1286)
    assert (O.grid(0)[0] == 8).all() and (O.grid(3)[0] == 4).all() and (O.grid(4)[0] == 1).all()   # :1490, :1575, :1598


def test_iquant_fields_land_where_the_published_layout_puts_them():
    """One block per format built field by field (not from random bytes): a chosen codebook index, sign pattern and
    multiplier for one group must come out at that group's eight positions and nowhere else."""
    def base(dt):
        b = np.zeros(H.BLOCK[dt][1], np.uint8)
        if dt == H.IQ1_M:
            H.iq1m_set_d(b.reshape(1, -1), 1.0)
        else:
            b[0:2] = H.f16_bytes(1.0)
        return b
    zero = {dt: O.dequant(dt, base(dt)) for dt in H.GRID_IQUANTS}
    ks = H.ksigns()
    # IQ2_XXS: sub-block 3, group 2 -> index 0xA7, sign index 0x55, multiplier 9
    b = base(H.IQ2_XXS)
    aux0, aux1 = 0xA7 << 16, (0x55 << 14) | (9 << 28)
    b[2 + 24:2 + 32] = np.frombuffer(np.array([aux0, aux1], "<u4").tobytes(), np.uint8)
    y = O.dequant(H.IQ2_XXS, b)
    g = H.iquant_grid("kIq2xxsGrid")
    sg = 1 - 2 * ((int(ks[0x55]) >> np.arange(8)) & 1)
    assert np.array_equal(y[96 + 16:96 + 24], (np.float32(9.5 * 0.25) * g[0xA7] * sg).astype(np.float32))
    assert np.array_equal(y[96:96 + 16], np.full(16, 9.5 * 0.25 * 8, np.float32))        # same multiplier, entry 0
    assert np.array_equal(np.delete(y, np.arange(96, 128)), np.delete(zero[H.IQ2_XXS], np.arange(96, 128)))
    # IQ2_XS: sub-block 5, group 3 -> 9-bit index 0x1B3, sign index 0x2A; high nibble of scale byte 5 = 6
    b = base(H.IQ2_XS)
    b[2 + 2 * 23:2 + 2 * 24] = np.frombuffer(np.array([0x1B3 | (0x2A << 9)], "<u2").tobytes(), np.uint8)
    b[66 + 5] = 6 << 4
    y = O.dequant(H.IQ2_XS, b)
    sg = 1 - 2 * ((int(ks[0x2A]) >> np.arange(8)) & 1)
    assert np.array_equal(y[160 + 24:160 + 32], (np.float32(6.5 * 0.25) * H.iquant_grid("kIq2xsGrid")[0x1B3] * sg).astype(np.float32))
    assert np.array_equal(y[160:160 + 16], zero[H.IQ2_XS][:16])                            # low nibble untouched
    # IQ2_S: sub-block 1, group 2 -> index 0x2C5 (high bits 2 from qh), sign byte 0x81, low nibble of scale 1 = 3 (not used
    # by group 2), high nibble 12
    b = base(H.IQ2_S)
    b[2 + 4 + 2] = 0xC5
    b[66 + 1] = 2 << 4
    b[34 + 4 + 2] = 0x81
    b[74 + 1] = 3 | (12 << 4)
    y = O.dequant(H.IQ2_S, b)
    sg = np.array([-1, 1, 1, 1, 1, 1, 1, -1])
    assert np.array_equal(y[32 + 16:32 + 24], (np.float32(12.5 * 0.25) * H.iquant_grid("kIq2sGrid")[0x2C5] * sg).astype(np.float32))
    assert np.array_equal(y[32:32 + 16], np.full(16, 3.5 * 0.25 * 8, np.float32))
    # IQ3_XXS: sub-block 6, group 1 -> entries 0x9E then 0x31, sign index 0x13, multiplier 4
    b = base(H.IQ3_XXS)
    b[2 + 48 + 2], b[2 + 48 + 3] = 0x9E, 0x31
    b[66 + 24:66 + 28] = np.frombuffer(np.array([(0x13 << 7) | (4 << 28)], "<u4").tobytes(), np.uint8)
    y = O.dequant(H.IQ3_XXS, b)
    g = H.iquant_grid("kIq3xxsGrid")
    sg = 1 - 2 * ((int(ks[0x13]) >> np.arange(8)) & 1)
    assert np.array_equal(y[192 + 8:192 + 16], (np.float32(4.5 * 0.5) * np.concatenate([g[0x9E], g[0x31]]) * sg).astype(np.float32))
    # IQ3_S: sub-block 3 (odd: high nibble of scale byte 1), group 2 -> entries 0x1F0 and 0x0F0: ninth bits are bits 4, 5 of qh
    b = base(H.IQ3_S)
    b[2 + 24 + 4], b[2 + 24 + 5] = 0xF0, 0xF0
    b[66 + 3] = 1 << 4
    b[74 + 12 + 2] = 0x0F
    b[106 + 1] = 7 << 4
    y = O.dequant(H.IQ3_S, b)
    g = H.iquant_grid("kIq3sGrid")
    assert np.array_equal(y[96 + 16:96 + 24], (np.float32(15.0) * np.concatenate([-g[0x1F0], g[0x0F0]])).astype(np.float32))
    assert np.array_equal(y[64:96], zero[H.IQ3_S][64:96])                                   # sub-block 2 keeps the low nibble (0)
    # IQ1_S: sub-block 4, group 3 -> index 0x5A | 6 << 8, multiplier 2 * 5 + 1, negative shift
    b = base(H.IQ1_S)
    b[2 + 16 + 3] = 0x5A
    b[34 + 8:34 + 10] = np.frombuffer(np.array([(6 << 9) | (5 << 12) | 0x8000], "<u2").tobytes(), np.uint8)
    y = O.dequant(H.IQ1_S, b)
    g = H.iquant_grid("kIq1sGrid")
    assert np.array_equal(y[128 + 24:128 + 32], (np.float32(11.0) * (g[0x65A] - 0.125)).astype(np.float32))
    assert np.array_equal(y[128:128 + 24], np.full(24, 11.0 * (-1 - 0.125), np.float32))
    # IQ1_M: sub-block 5 (second six bits of scale word 2), group 1 (high nibble of qh[10]) and group 2 (low nibble of qh[11])
    b = base(H.IQ1_M)
    b[20 + 1], b[20 + 2] = 0x33, 0x44
    b[32 + 10], b[32 + 11] = (0x8 | 5) << 4, 3
    w = int(np.frombuffer(b[52:54].tobytes(), "<u2")[0]) | (2 << 6) | (6 << 9)
    b[52:54] = np.frombuffer(np.array([w], "<u2").tobytes(), np.uint8)
    y = O.dequant(H.IQ1_M, b)
    assert np.array_equal(y[160 + 8:160 + 16], (np.float32(5.0) * (g[0x533] - 0.125)).astype(np.float32))
    assert np.array_equal(y[160 + 16:160 + 24], (np.float32(13.0) * (g[0x344] + 0.125)).astype(np.float32))
    assert np.array_equal(y[160:160 + 8], np.full(8, 5.0 * (-1 + 0.125), np.float32))
    assert np.array_equal(np.delete(y, np.arange(160, 192)), np.delete(zero[H.IQ1_M], np.arange(160, 192)))


def test_fp4_scales_match_their_arithmetic_definition_for_every_byte():
    """E8M0 (MXFP4) and UE4M3 (NVFP4) scale bytes 0..255 against 2^(e - 127) and (8 + m) 2^(e - 10); element 0 carries
    the code 1 (E2M1 0.5), element 16 / 8 the code 2 (E2M1 1.0)."""
    b = np.zeros((256, 17), np.uint8)
    b[:, 0], b[:, 1] = np.arange(256), 0x21
    y = O.dequant(O.MXFP4, b.reshape(-1)).reshape(256, 32)
    with np.errstate(over="ignore"):   # byte 255 (NaN in the E8M0 definition) decodes to 2^127, the code 2 overflows on it
        assert np.array_equal(y[:, 16], np.ldexp(np.float32(1), np.arange(256) - 127))
    assert np.array_equal(y[:255, 0], y[:255, 16] / 2) and y[255, 0] == np.float32(2.0) ** 127
    assert np.array_equal(y, H.ggml_dequant(H.MXFP4, b.reshape(-1)).astype(np.float32).reshape(256, 32))
    b = np.zeros((256, 36), np.uint8)
    b[:, 0], b[:, 4] = np.arange(256), 0x21
    y = O.dequant(O.NVFP4, b.reshape(-1)).reshape(256, 64)
    x = np.arange(256)
    want = np.where((x >> 3) & 15, (8 + (x & 7)) * np.exp2(((x >> 3) & 15) - 10.0), (x & 7) * 2.0 ** -9)
    want[[0, 0x7F]] = 0
    assert np.array_equal(y[:, 8], want.astype(np.float32)) and not y[:, 16:].any()
    assert np.array_equal(y, H.ggml_dequant(H.NVFP4, b.reshape(-1)).astype(np.float32).reshape(256, 64))


def test_tq1_0_decodes_what_the_published_packing_stores():
    """All 243 five-digit ternary numbers packed as ggml's quantiser packs them (ceil(v * 256 / 243)) come back
    digit by digit, in the three byte runs of a block (32, 16 and 4 bytes; the last holds four digits per byte)."""
    import itertools
    trits = np.array(list(itertools.product(range(3), repeat=5)))
    packed = H.tq1_0_pack(trits)
    for start in range(0, 243, 16):
        chunk, t = packed[start:start + 16], trits[start:start + 16]
        n = len(chunk)
        blk = np.zeros(54, np.uint8)
        blk[52:54] = H.f16_bytes(2.0)
        blk[:n], blk[32:32 + n], blk[48:48 + min(n, 4)] = chunk, chunk, chunk[:4]
        y = O.dequant(O.TQ1_0, blk) / 2 + 1
        assert np.array_equal(y[:160].reshape(5, 32)[:, :n].T, t)
        assert np.array_equal(y[160:240].reshape(5, 16)[:, :n].T, t)
        assert np.array_equal(y[240:].reshape(4, 4)[:, :min(n, 4)].T, t[:4, :4])


def test_dequant_hand_computed_values():
    # Q8_0: d = 0.5, q = -128..-97: y = d*q exactly
    blk = np.zeros(34, np.uint8)
    blk[0:2] = H.f16_bytes(0.5)
    blk[2:] = np.arange(-128, -96).astype(np.int8).view(np.uint8)
    assert np.array_equal(O.dequant(O.Q8_0, blk), np.arange(-128, -96, dtype=np.float32) * 0.5)
    # Q4_K: one block, d=1, dmin=1, sub-block 0: sc=3,m=2 -> y = 3*q - 2; sub-block 5 (j>=4): sc=33, m=50
    blk = np.zeros(144, np.uint8)
    blk[0:2] = H.f16_bytes(1.0)
    blk[2:4] = H.f16_bytes(1.0)
    s = blk[4:16]
    s[0] = 3
    s[4] = 2
    s[5 + 4] = (33 & 0xF) | ((50 & 0xF) << 4)
    s[5 - 4] |= (33 >> 4) << 6
    s[5] |= (50 >> 4) << 6
    blk[16 + 0] = 0x0F           # element 0 (low nibble of qs[0]) = 15, element 32 (high nibble) = 0
    blk[16 + 64 + 7] = 0xA0      # qs[71]: j=2 -> elements 128+7 (low)=0 and 160+7 (high, sub-block 5)=10
    y = O.dequant(O.Q4K, blk)
    assert y[0] == 3 * 15 - 2 and y[1] == -2.0
    assert y[160 + 7] == 33 * 10 - 50 and y[160] == -50.0
    # Q6_K: d=2, scale[9] = -3, element 128+16+3 (half 1, l=19, group 0 -> scale index 8+1): q = ql lo | qh bits0-1
    blk = np.zeros(210, np.uint8)
    blk[208:210] = H.f16_bytes(2.0)
    blk[192 + 9] = np.array([-3], np.int8).view(np.uint8)[0]
    blk[64 + 19] = 0x05          # ql[64+19] low nibble 5
    blk[128 + 32 + 19] = 0x02    # qh[32+19] bits 0-1 = 2 -> q = 5 | (2<<4) = 37
    y = O.dequant(O.Q6K, blk)
    assert y[128 + 19] == 2.0 * -3 * (37 - 32)
    assert y[128 + 16] == 2.0 * -3 * (0 - 32)


def test_dequant_float_dtypes():
    v = np.array([1.5, -2.25, 65504.0, 6e-8], np.float32)
    assert np.array_equal(O.dequant(O.F16, v.astype(np.float16)), v.astype(np.float16).astype(np.float32))
    bf = (v.view(np.uint32) >> 16).astype(np.uint16)
    assert np.array_equal(O.dequant(O.BF16, bf), (bf.astype(np.uint32) << 16).view(np.float32))
    assert np.array_equal(O.dequant(O.F32, v), v)
    assert np.array_equal(O.dequant(O.I32, np.array([-7, 3], np.int32)), np.array([-7.0, 3.0], np.float32))


# ------------------------------------------------------------------ dot
def _round_f32(fr: Fraction) -> np.float32:
    """Exact round-to-nearest-even of a rational to f32."""
    if fr == 0:
        return np.float32(0.0)
    f = np.float32(float(fr))  # float(Fraction) is correctly rounded to f64; fix the second rounding
    cands = {f, np.nextafter(f, np.float32(np.inf)), np.nextafter(f, np.float32(-np.inf))}
    best = None
    for c in cands:
        if not np.isfinite(c):
            continue
        err = abs(Fraction(float(c)) - fr)
        key = (err, int(np.float32(c).view(np.uint32)) & 1)
        if best is None or key < best[0]:
            best = (key, c)
    return np.float32(best[1])


def _dot_exact_model(a, b):
    """kernels.rs:6568-6583 evaluated with exact rational arithmetic and one rounding per FMA / add."""
    n = len(a)
    acc = [np.float32(0)] * 8
    for c in range(n // 8):
        for j in range(8):
            i = 8 * c + j
            acc[j] = _round_f32(Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(acc[j])))
    s = np.float32(0)
    for j in range(8):
        s = _round_f32(Fraction(float(s)) + Fraction(float(acc[j])))
    for i in range(n // 8 * 8, n):
        s = _round_f32(Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(s)))
    return s


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 15, 16, 17, 63, 64, 65, 200])
def test_dot_lane_order_and_fma_bit_exact(n):
    rng = np.random.default_rng(n)
    # wide dynamic range so a different association or an unfused multiply changes the bits
    a = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 4, n)).astype(np.float32)
    b = (rng.standard_normal(n) * 10.0 ** rng.integers(-3, 4, n)).astype(np.float32)
    got = O.dot(a, b)
    want = _dot_exact_model(a, b)
    assert got.view(np.uint32) == want.view(np.uint32)


def test_dot_distinguishes_plausible_wrong_orders():
    # The 8-lane order must differ from a sequential sum and from a pairwise/tree lane reduction
    # on this input, otherwise the test above could not catch those mistakes.
    rng = np.random.default_rng(7)
    a = (rng.standard_normal(64) * 10.0 ** rng.integers(-4, 5, 64)).astype(np.float32)
    b = rng.standard_normal(64).astype(np.float32)
    seq = np.float32(0)
    for i in range(64):
        seq = _round_f32(Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(seq)))
    assert O.dot(a, b).view(np.uint32) != seq.view(np.uint32)
    assert abs(float(O.dot(a, b)) - float(np.dot(a.astype(np.float64), b.astype(np.float64)))) < 1e-2 * np.abs(a * b).sum()


# ------------------------------------------------------------------ activations
def test_act_fn_closed_forms():
    for g in (-30.0, -3.0, -0.5, 0.0, 0.5, 3.0, 30.0):
        silu = g / (1.0 + np.exp(-g))
        assert abs(float(O.act(O.ACT_SILU, g)) - silu) <= 2e-7 * max(1.0, abs(silu))
        sig = 1.0 / (1.0 + np.exp(-g))
        assert abs(float(O.act(O.ACT_SIGMOID, g)) - sig) <= 2e-7
        gelu = 0.5 * g * (1.0 + np.tanh(0.7978846 * (g + 0.044715 * g ** 3)))
        assert abs(float(O.act(O.ACT_GELU, g)) - gelu) <= 4e-7 * max(1.0, abs(gelu))
    assert float(O.act(O.ACT_SILU, 0.0)) == 0.0
    # clamp: act(min(gate, l)) * clamp(up, -l, l)  (graph.rs:953-971)
    assert O.gated_act(O.ACT_SILU, 5.0, 9.0, clamp=2.0) == np.float32(O.act(O.ACT_SILU, 2.0) * np.float32(2.0))
    assert O.gated_act(O.ACT_SILU, -5.0, -9.0, clamp=2.0) == np.float32(O.act(O.ACT_SILU, -5.0) * np.float32(-2.0))
    assert O.gated_act(O.ACT_SILU, 1.0, 3.0) == np.float32(O.act(O.ACT_SILU, 1.0) * np.float32(3.0))


# ------------------------------------------------------------------ routing
def test_route_softmax_topk_renorm():
    rng = np.random.default_rng(3)
    lg = rng.standard_normal(128).astype(np.float32)
    probs, idx, w = O.route_row(lg, 8)
    p64 = np.exp(lg.astype(np.float64) - lg.max())
    p64 /= p64.sum()
    assert np.allclose(probs, p64, rtol=2e-6, atol=0)
    assert list(idx) == list(np.argsort(-p64, kind="stable")[:8])
    assert np.allclose(w, p64[idx] / p64[idx].sum(), rtol=3e-6)
    assert abs(float(w.sum()) - 1.0) < 1e-6
    # not renormalised, scaled
    _, idx2, w2 = O.route_row(lg, 8, norm_w=False, scale=2.5)
    assert list(idx2) == list(idx) and np.allclose(w2, p64[idx] * 2.5, rtol=3e-6)


def test_route_ties_keep_ascending_expert_id():
    lg = np.zeros(16, np.float32)
    lg[[11, 3, 7]] = 1.0  # three equal maxima, then all-equal rest
    _, idx, w = O.route_row(lg, 5)
    assert list(idx) == [3, 7, 11, 0, 1]
    assert np.allclose(w[:3], w[0]) and np.allclose(w[3:], w[3])


def test_route_groups_bias_selects_what_the_reference_test_states():
    # seam_op_parity.rs:2495-2504: sigmoid gating, +0.6 bias on group 1 -> group 1 wins, experts 4 and 5,
    # while the weights come from the UNBIASED probabilities.
    lg = np.array([3.0, 2.5, 2.0, 1.5, 1.0, 0.9, 0.8, 0.7], np.float32)
    bias = np.array([0, 0, 0, 0, .6, .6, .6, .6], np.float32)
    probs, idx, w = O.route_row(lg, 2, gating=O.GATE_SIGMOID, exp_probs_b=bias, n_groups=2, n_groups_used=1)
    assert list(idx) == [4, 5]
    sig = 1 / (1 + np.exp(-lg.astype(np.float64)))
    assert np.allclose(w, sig[[4, 5]] / sig[[4, 5]].sum(), rtol=1e-6)
    # group scores from the comment: 1.877 vs 1.442 unbiased, 2.642 biased
    assert abs(np.sort(sig[:4])[-2:].sum() - 1.877) < 1e-3 and abs(np.sort(sig[4:])[-2:].sum() + 1.2 - 2.642) < 1e-3
    _, idx_nobias, _ = O.route_row(lg, 2, gating=O.GATE_SIGMOID, n_groups=2, n_groups_used=1)
    assert list(idx_nobias) == [0, 1]


def test_route_sqrt_softplus_and_hash_ids():
    lg = np.array([24.0, 1.0, 0.75, 0.5, -1.5, -1.0], np.float32)  # seam_op_parity.rs:2393-2396
    probs, idx, w = O.route_row(lg, 2, gating=O.GATE_SQRT_SOFTPLUS)
    assert list(idx) == [0, 1]
    assert probs[0] == np.float32(np.sqrt(np.float32(24.0)))  # v > 20 shortcut: sp = v
    assert abs(float(probs[1]) - np.sqrt(np.log1p(np.exp(1.0)))) < 1e-6
    # hash routing: ids in table order, weights = renormalised probs at those ids (graph.rs:1318-1351)
    p2, idx2, w2 = O.route_row(lg, 2, hash_ids=[5, 2])
    assert list(idx2) == [5, 2] and np.allclose(w2, p2[[5, 2]] / p2[[5, 2]].sum(), rtol=1e-6)
    with pytest.raises(ValueError):
        O.route_row(lg, 2, hash_ids=[6, 0])


# ------------------------------------------------------------------ Op::MoeFfn
def _run_case(c, **kw):
    return O.moe_ffn(c["x"], c["router"], c["gate"], c["up"], c["down"], ne=c["ne"], n_expert=c["n_expert"],
                     n_used=c["n_used"], n_ff_exp=c["n_ff"], gate_dtype=c["dtype"], gating=c["gating"],
                     exp_probs_b=c.get("bias"), n_expert_groups=c.get("n_groups", 0),
                     n_expert_groups_used=c.get("n_groups_used", 0), **kw)


def test_moe_ffn_matches_golden_cases_of_the_reference_tests():
    g = np.load(os.path.join(GOLD, "moe_small.npz"))
    cases = H.moe_cases()
    assert sorted(cases) == sorted({k.split(".")[0] for k in g.files})
    for name, c in cases.items():
        r = _run_case(c)
        assert np.array_equal(r["idx"], g[name + ".idx"]), name
        # seam_op_parity.rs asserts max-abs 1e-4 on its f32 cases; metal parity.rs asserts
        # |c-m|/max(|c|,1) <= 1e-3 on its (large-magnitude) synthetic quantised cases
        if name in ("sqrt_softplus", "groups_bias"):
            assert H.max_abs(r["dst"], g[name + ".want"]) < 1e-4, name
        assert H.elem_rel_err(r["dst"], g[name + ".want"]) < 1e-3, name
        assert H.rel_l2(r["dst"], g[name + ".want"]) < 1e-5, name


@pytest.mark.parametrize("gdt,ddt", [(O.Q4K, O.Q6K), (O.Q8_0, O.Q8_0), (O.Q6K, O.Q4K)])
@pytest.mark.parametrize("rows", [1, 5])
def test_moe_ffn_quantised_multirow_vs_f64_model(gdt, ddt, rows):
    ne, E, K, nff = 256, 16, 4, 512
    rng = np.random.default_rng(rows * 100 + gdt)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    gate, up = H.synth_weight(gdt, E * nff * ne, 11), H.synth_weight(gdt, E * nff * ne, 12)
    down = H.synth_weight(ddt, E * ne * nff, 13)
    r = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt,
                  down_dtype=ddt, scale=1.3)
    want, idx = H.moe_ffn_f64(x, router, H.ggml_dequant(gdt, gate), H.ggml_dequant(gdt, up),
                              H.ggml_dequant(ddt, down), ne=ne, n_expert=E, n_used=K, n_ff=nff, scale=1.3)
    assert np.array_equal(r["idx"], idx)
    assert H.rel_l2(r["dst"], want) < 2e-6
    # thread count must not change a single bit (every output is owned by one task)
    r1 = O.moe_ffn(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt,
                   down_dtype=ddt, scale=1.3, n_threads=1)
    assert np.array_equal(r1["dst"].view(np.uint32), r["dst"].view(np.uint32))


def test_moe_ffn_variants_vs_f64_model():
    ne, E, K, nff = 64, 8, 3, 96
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, ne)).astype(np.float32)
    router = rng.standard_normal((E, ne)).astype(np.float32) * 0.3
    gate = rng.standard_normal((E, nff, ne)).astype(np.float32) * 0.2
    up = rng.standard_normal((E, nff, ne)).astype(np.float32) * 0.2
    down = rng.standard_normal((E, ne, nff)).astype(np.float32) * 0.2
    ds = rng.uniform(0.5, 1.5, E).astype(np.float32)
    common = dict(ne=ne, n_expert=E, n_used=K, n_ff_exp=nff)
    # weight_before (llama4), sigmoid gating, no renorm
    r = O.moe_ffn(x, router, gate, up, down, gating=O.GATE_SIGMOID, norm_w=False, weight_before=True, **common)
    want, _ = H.moe_ffn_f64(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff=nff, gating="sigmoid",
                            norm_w=False, weight_before=True)
    assert H.rel_l2(r["dst"], want) < 2e-6
    # down_scale + clamp + gelu
    r = O.moe_ffn(x, router, gate, up, down, down_scale=ds, swiglu_clamp=0.7, act=O.ACT_GELU, **common)
    want, _ = H.moe_ffn_f64(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff=nff, down_scale=ds,
                            clamp=0.7, act="gelu")
    assert H.rel_l2(r["dst"], want) < 2e-6
    # fused gate_up: gate rows first, up rows second per expert (graph.rs:1279-1285)
    fused = np.concatenate([gate, up], axis=1)
    rf = O.moe_ffn(x, router, fused, None, down, fused_gate_up=True, **common)
    rs = O.moe_ffn(x, router, gate, up, down, **common)
    assert np.array_equal(rf["dst"].view(np.uint32), rs["dst"].view(np.uint32))
    # hash routing
    ids = np.array([[1, 5, 2], [0, 7, 3], [4, 4, 6]], np.int32)
    r = O.moe_ffn(x, router, gate, up, down, expert_ids=ids.astype(np.float32), **common)
    want, _ = H.moe_ffn_f64(x, router, gate, up, down, ne=ne, n_expert=E, n_used=K, n_ff=nff, hash_ids=ids)
    assert np.array_equal(r["idx"], ids) and H.rel_l2(r["dst"], want) < 2e-6
    # refused combinations (lib.rs:3613-3629)
    with pytest.raises(ValueError):
        O.moe_ffn(x, router, gate, up, down, swiglu_clamp=1.0, weight_before=True, **common)
    with pytest.raises(ValueError):
        O.moe_ffn(x, router, gate, up, down, expert_ids=ids.astype(np.float32), exp_probs_b=np.zeros(E), **common)


def test_bucketing_order_and_inverse_map():
    ne, E, K, nff, rows = 32, 12, 3, 32, 40
    rng = np.random.default_rng(9)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = rng.standard_normal((E, ne)).astype(np.float32)
    w = (rng.standard_normal(E * nff * ne) * 0.1).astype(np.float32)
    r = O.moe_ffn(x, router, w, w, (rng.standard_normal(E * ne * nff) * 0.1).astype(np.float32), ne=ne, n_expert=E,
                  n_used=K, n_ff_exp=nff)
    idx = r["idx"]
    # brute force of lib.rs:3887-3906: experts ascending, rows ascending inside an expert
    pairs = sorted((int(idx[rr, k]), rr, k) for rr in range(rows) for k in range(K))
    assert list(r["pair_row"]) == [p[1] for p in pairs]
    experts = sorted({p[0] for p in pairs})
    assert list(r["bucket_expert"]) == experts and r["n_buckets"] == len(experts)
    counts = [sum(1 for p in pairs if p[0] == e) for e in experts]
    assert list(r["bucket_count"]) == counts and int(np.sum(counts)) == rows * K
    assert list(r["bucket_p0"]) == list(np.cumsum([0] + counts[:-1]))
    for flat, (e, rr, k) in enumerate(pairs):
        assert r["slot_pair"][rr, k] == flat
    assert sorted(r["slot_pair"].ravel()) == list(range(rows * K))  # a permutation


def test_moe_ffn_empty_rows():
    r = O.moe_ffn(np.zeros((0, 32), np.float32), np.zeros(4 * 32, np.float32), np.zeros(4 * 32 * 32, np.float32),
                  np.zeros(4 * 32 * 32, np.float32), np.zeros(4 * 32 * 32, np.float32), ne=32, n_expert=4, n_used=2,
                  n_ff_exp=32)
    assert r["dst"].shape == (0, 32) and r["n_buckets"] == 0


# ------------------------------------------------------------------ neighbours
@pytest.mark.parametrize("dt", [O.Q4K, O.Q6K, O.Q8_0, O.F32, O.F16])
def test_linear_reference_mode_vs_f64(dt):
    in_f, out_f, m = 512, 24, 3
    rng = np.random.default_rng(dt)
    x = rng.standard_normal((m, in_f)).astype(np.float32)
    if dt in (O.F32, O.F16):
        w = (rng.standard_normal(out_f * in_f) * 0.1).astype(np.float32 if dt == O.F32 else np.float16)
    else:
        w = H.synth_weight(dt, out_f * in_f, 21)
    got = O.linear(x, w, dt, in_f, out_f)
    W = np.asarray(H.ggml_dequant(dt, w), np.float64).reshape(out_f, in_f)
    want = x.astype(np.float64) @ W.T
    # decode_parity.rs:93-102 holds reference mode to 1e-5 of the f64 GEMV
    assert H.rel_l2(got, want) < 1e-5
    # w_off selects a row band of a concatenated weight (graph.rs:208-211)
    got2 = O.linear(x, w, dt, in_f, 8, w_off=8 * in_f)
    assert np.array_equal(got2.view(np.uint32), np.ascontiguousarray(got[:, 8:16]).view(np.uint32))


def test_elementwise_neighbours():
    rng = np.random.default_rng(2)
    a, b = rng.standard_normal((3, 40)).astype(np.float32), rng.standard_normal((3, 40)).astype(np.float32)
    assert np.array_equal(O.add(a, b), a + b)
    ga = O.gated_act_rows(a, b)
    assert np.allclose(ga, a / (1 + np.exp(-a.astype(np.float64))) * b, rtol=1e-6, atol=1e-7)
    gate = np.array([0.3, -1.2, 4.0], np.float32)
    got = O.moe_shared_expert_add(a, b, gate)
    want = a + (1 / (1 + np.exp(-gate.astype(np.float64))))[:, None] * b
    assert np.allclose(got, want, rtol=1e-6, atol=1e-7)


def test_rms_norm_closed_forms_and_f64():
    """Op::RmsNorm (crates/infr-cpu/src/lib.rs:1046-1069).  Pinned by what the definition fixes: a
    constant row of c with unit weight gives c / sqrt(c^2 + eps) in every column; with eps = 0 the
    mean square of out / weight is 1; rows do not mix; the weight multiplies per column; and the whole
    thing agrees with an f64 evaluation.  The Add form accumulates onto dst (lib.rs:1070-1093)."""
    dim = 96
    c = np.float32(3.0)
    out = O.rms_norm(np.full((2, dim), c, np.float32), np.ones(dim, np.float32), 1e-2)
    assert np.allclose(out, c / np.sqrt(np.float64(c) ** 2 + 1e-2), rtol=2e-7, atol=0)
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((4, dim)) * 5).astype(np.float32)
    w = (1 + 0.3 * rng.standard_normal(dim)).astype(np.float32)
    out = O.rms_norm(x, w, 0.0)
    assert np.allclose(np.mean((out.astype(np.float64) / w) ** 2, axis=1), 1.0, rtol=1e-5)
    x64 = x.astype(np.float64)
    eps = 1e-5
    want = x64 / np.sqrt(np.mean(x64 * x64, axis=1, keepdims=True) + eps) * w
    got = O.rms_norm(x, w, eps)
    assert H.rel_l2(got, want) < 2e-7
    # rows are independent: a row alone gives the bits it gives inside the batch
    assert np.array_equal(O.rms_norm(x[2:3], w, eps).view(np.uint32), got[2:3].view(np.uint32))
    # a column's weight reaches that column only
    w2 = w.copy()
    w2[7] *= 2
    got2 = O.rms_norm(x, w2, eps)
    assert np.array_equal(np.delete(got2, 7, axis=1), np.delete(got, 7, axis=1)) and np.allclose(got2[:, 7], 2 * got[:, 7])
    base = rng.standard_normal((4, dim)).astype(np.float32)
    assert np.array_equal(O.rms_norm(x, w, eps, add_to=base), base + got)
    assert O.rms_norm(np.zeros((0, dim), np.float32), w, eps).shape == (0, dim)


# ------------------------------------------------------------------ production int8 path (timed baseline only)
def test_quantize_q8_follows_the_definition():
    """crates/infr-cpu/src/quant.rs:27-63: d = amax / 127 per 256, round half AWAY from zero, clamp to +-127,
    sums per 32; an all-zero block gives d = 0 and zero codes."""
    x = np.zeros(512, np.float32)
    x[:256] = np.linspace(-2.0, 2.0, 256, dtype=np.float32)
    x[3] = 2.0 * 0.5 / 127      # exactly half a step: rounds away from zero, to 1 (round-half-even would give 0)
    x[4] = -2.0 * 2.5 / 127     # -2.5 steps -> -3
    qs, d, bs = O.quantize_q8(x)
    assert d[0] == np.float32(2.0) / np.float32(127.0) and d[1] == 0.0
    assert qs[0] == -127 and qs[255] == 127 and qs[3] == 1 and qs[4] == -3
    assert not qs[256:].any() and np.abs(qs).max() == 127
    assert np.array_equal(bs, qs.astype(np.int32).reshape(-1, 32).sum(axis=1))
    idv = np.float32(1.0) / d[0]
    want = np.clip(np.sign(x[:256]) * np.floor(np.abs(x[:256] * idv) + np.float32(0.5)), -127, 127)
    assert np.array_equal(qs[:256], want.astype(np.int8))


@pytest.mark.parametrize("dt,in_f,d,dmin", [(O.Q4K, 768, 0.05, 0.015), (O.Q6K, 768, 0.04, None), (O.Q8_0, 512, 0.03, None)])
def test_int8_dot_matches_the_dequantised_dot(dt, in_f, d, dmin):
    """The reference's own check of its int8 kernels (crates/infr-cpu/src/kernels.rs:6782-6826): the integer dot
    equals dot(dequant(weight row), dequant(q8 activations)) to 1e-3 of max(|want|, 1)."""
    rng = np.random.default_rng(dt)
    be, bb = O.block_geometry(dt)
    w = rng.integers(0, 256, in_f // be * bb, dtype=np.uint8).reshape(-1, bb)
    slots = H.F16_SLOTS[dt]
    w[:, slots[0]:slots[0] + 2] = H.f16_bytes(d)
    if dmin is not None:
        w[:, slots[1]:slots[1] + 2] = H.f16_bytes(dmin)
    w = w.reshape(-1)
    x = (rng.standard_normal(in_f) * 1.5).astype(np.float32)
    q8 = O.quantize_q8(x)
    xq = (q8[0].astype(np.float32).reshape(-1, 256) * q8[1][:, None]).reshape(-1)
    want = float(np.dot(H.ggml_dequant(dt, w).astype(np.float64), xq.astype(np.float64)))
    got = float(O.vec_dot_q8(dt, w, q8))
    assert abs(got - want) / max(abs(want), 1.0) < 1e-3
    # and the activation rounding itself is the only other error: 1/254 of the block's amax per element
    assert np.abs(xq - x).max() <= np.abs(x).max() / 254 * 1.0001


@pytest.mark.parametrize("gdt,ddt", [(O.Q4K, O.Q6K), (O.Q8_0, O.Q8_0)])
def test_production_mode_stays_close_to_reference_mode(gdt, ddt):
    """Batch numerics of the CPU backend (int8 activations): same routing, outputs within the activation
    quantisation error of the f32 reference; a single row is not affected (int8_ok needs two rows, lib.rs:3679)."""
    ne, E, K, nff, rows = 512, 8, 2, 256, 6
    rng = np.random.default_rng(9)
    x = rng.standard_normal((rows, ne)).astype(np.float32)
    router = (rng.standard_normal((E, ne)) * 0.1).astype(np.float32)
    gate, up = H.centred_weight(gdt, E * nff * ne, 1), H.centred_weight(gdt, E * nff * ne, 2)
    down = H.centred_weight(ddt, E * ne * nff, 3)
    kw = dict(ne=ne, n_expert=E, n_used=K, n_ff_exp=nff, gate_dtype=gdt, down_dtype=ddt)
    ref = O.moe_ffn(x, router, gate, up, down, **kw)
    prod = O.moe_ffn(x, router, gate, up, down, production=True, **kw)
    assert np.array_equal(ref["idx"], prod["idx"]) and np.array_equal(ref["w"].view(np.uint32), prod["w"].view(np.uint32))
    err = H.rel_l2(prod["dst"], ref["dst"])
    assert 1e-6 < err < 3e-2, err
    one_ref = O.moe_ffn(x[:1], router, gate, up, down, **kw)
    one_prod = O.moe_ffn(x[:1], router, gate, up, down, production=True, **kw)
    assert np.array_equal(one_ref["dst"].view(np.uint32), one_prod["dst"].view(np.uint32))

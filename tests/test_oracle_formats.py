"""Pins the oracle's conversions and block decoders: golden vectors of the reference's own tests
(tests/data/kquant_golden.bin, gguf-py values), exhaustive conversions against hardware / closed forms, the NVFP4G
closed form, and, where built, the reference's own objects. Encoders (this build's own: parity unpinned) are held
to round-trip error and block validity only."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "kquant_golden.bin")


def golden_records():
    b = open(GOLDEN, "rb").read()
    o = 0
    while o < len(b):
        t, nb, bb, el = struct.unpack_from("<4I", b, o)
        o += 16
        raw = np.frombuffer(b, np.uint8, nb * bb, o)
        o += nb * bb
        vals = np.frombuffer(b, np.float32, nb * el, o)
        o += nb * el * 4
        yield t, nb, bb, el, raw, vals


def test_golden_file_holds_the_path_types():
    types = [r[0] for r in golden_records()]
    assert types == [10, 11, 12, 13, 21, 23, 20]


@pytest.mark.parametrize("wtype", [12, 21, 23, 20])
def test_decoders_match_golden_bit_for_bit(oracle, wtype):
    for t, nb, bb, el, raw, vals in golden_records():
        if t != wtype:
            continue
        assert oracle.BLOCK[t] == (el, bb)
        got = oracle.dequantize(t, raw, nb * el)
        assert np.array_equal(got.view(np.uint32), vals.view(np.uint32))
        return
    pytest.fail("type not in the golden file")


def test_half_to_float_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.half_to_float(int(v)) for v in h], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.isnan(got[nan]).all()


def test_float_to_half_against_hardware(oracle):
    rng = np.random.default_rng(1)
    cases = np.concatenate([
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),        # every half, exactly
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.uniform(-9, 6, 20000).astype(np.float32),
        np.array([65504.0, 65519.99, 65520.0, 1e9, 5.96e-8, 2.98e-8, 2.9802322e-8, 2.99e-8, 6.1e-5, 0.0, -0.0], np.float32),
    ])
    cases = cases[~np.isnan(cases)]
    # halfway cases between neighbouring halves (ties to even)
    hs = np.arange(0, 0x7BFF, dtype=np.uint16)
    mid = (hs.view(np.float16).astype(np.float64) + (hs + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2
    cases = np.concatenate([cases, mid.astype(np.float32)])
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16).view(np.uint16)
    got = np.array([oracle.float_to_half(float(v)) for v in cases], np.uint16)
    assert np.array_equal(got, want)


def test_e4m3_closed_form(oracle):
    for b in range(256):
        e, m = (b >> 3) & 15, b & 7
        v = oracle.e4m3_to_float(b)
        if e == 15 and m == 7:
            assert np.isnan(v)
            continue
        want = (m / 8 * 2.0 ** -6) if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
        assert v == (-want if b & 0x80 else want)
    assert oracle.e4m3_to_float(0x7E) == 448.0


def test_float_to_e4m3_is_nearest_even(oracle):
    codes = [b for b in range(127)]  # positive finite codes, ascending in value
    vals = np.array([oracle.e4m3_to_float(b) for b in codes])
    assert (np.diff(vals) > 0).all()
    for b in codes:
        assert oracle.float_to_e4m3(vals[b]) == b
        assert oracle.float_to_e4m3(-vals[b]) == (b | 0x80)
    rng = np.random.default_rng(2)
    for v in np.concatenate([rng.uniform(0, 460, 4000), rng.uniform(0, 0.05, 2000), (vals[:-1] + vals[1:]) / 2]):
        v = float(np.float32(v))
        got = oracle.float_to_e4m3(v)
        d = np.abs(vals - min(v, 448.0))
        best = np.flatnonzero(d == d.min())
        if len(best) == 2:  # exact tie: even mantissa code
            want = best[0] if best[0] % 2 == 0 else best[1]
        else:
            want = best[0]
        assert got == want, (v, got, want)


def test_nvfp4g_closed_form(oracle):
    rng = np.random.default_rng(3)
    e2m1 = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], np.float32)
    nb = 12
    raw = rng.integers(0, 256, (nb, 76), dtype=np.uint8)
    raw[:, 4:12] &= 0x7E                      # finite, positive scales
    g = rng.uniform(1e-3, 2e-2, nb).astype(np.float32)
    raw[:, 0:4] = g.view(np.uint8).reshape(nb, 4)
    got = oracle.dequantize(oracle.NVFP4G, raw, nb * 128).reshape(nb, 128)
    for b in range(nb):
        for grp in range(8):
            d = np.float32(oracle.e4m3_to_float(raw[b, 4 + grp])) * g[b]
            q = raw[b, 12 + 8 * grp:20 + 8 * grp]
            want = np.empty(16, np.float32)
            want[0::2] = e2m1[q & 15] * d     # low nibble = even weight
            want[1::2] = e2m1[q >> 4] * d
            assert np.array_equal(got[b, 16 * grp:16 * grp + 16], want)


def test_iq4xs_independent_decode(oracle):
    """Second, independently written IQ4_XS decode (vectorised numpy over the raw layout)."""
    rng = np.random.default_rng(4)
    kv = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float32)
    nb = 40
    raw = rng.integers(0, 256, (nb, 136), dtype=np.uint8)
    raw[:, 0:2] = np.float16(rng.uniform(1e-3, 5e-2, nb)).view(np.uint8).reshape(nb, 2)
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32)[:, 0]
    sh = raw[:, 2:4].copy().view(np.uint16)[:, 0].astype(np.int32)
    ib = np.arange(8)
    lo = (raw[:, 4:8].astype(np.int32)[:, ib // 2] >> (4 * (ib % 2))) & 15
    ls = lo | (((sh[:, None] >> (2 * ib)) & 3) << 4)
    dl = d[:, None] * (ls - 32).astype(np.float32)
    qs = raw[:, 8:].reshape(nb, 8, 16)
    want = np.concatenate([dl[:, :, None] * kv[qs & 15], dl[:, :, None] * kv[qs >> 4]], axis=2).reshape(nb, 256)
    got = oracle.dequantize(oracle.IQ4_XS, raw, nb * 256).reshape(nb, 256)
    assert np.array_equal(got, want.astype(np.float32))


def test_q8_0_closed_form(oracle):
    """Q8_0 (dequant.cpp:555-562): 34 bytes = fp16 d, 32 int8; value d * q, every code from -128 to 127."""
    rng = np.random.default_rng(5)
    nb = 16
    raw = np.empty((nb, 34), np.uint8)
    d = np.float16(rng.uniform(1e-3, 5e-2, nb) * rng.choice([-1, 1], nb))
    raw[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    q = rng.integers(-128, 128, (nb, 32)).astype(np.int8)
    q[0] = np.arange(-128, -96)
    q[1] = np.arange(96, 128)
    raw[:, 2:] = q.view(np.uint8)
    got = oracle.dequantize(oracle.Q8_0, raw, nb * 32).reshape(nb, 32)
    assert np.array_equal(got, d.astype(np.float32)[:, None] * q.astype(np.float32))
    # the encoder's round trip: within half a step of d = amax / 127
    x = rng.standard_normal((8, 32)).astype(np.float32)
    back = oracle.dequantize(oracle.Q8_0, oracle.quantize(oracle.Q8_0, x), x.size).reshape(8, 32)
    assert (np.abs(back - x) <= np.abs(x).max(axis=1, keepdims=True) / 127 * 0.51 + 1e-6).all()


@pytest.mark.parametrize("wtype,bits", [(13, 5), (14, 6)])
def test_q5k_q6k_independent_decode_and_round_trip(oracle, wtype, bits):
    """Q5_K / Q6_K: the codes are plain integers, so a block built from known codes and scales must decode to the closed
    form (scale * code - min, scale * (code - 32)); the encoders' round trip stays within a step."""
    rng = np.random.default_rng(wtype)
    if wtype == 13:
        b = np.zeros(176, np.uint8)
        b[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
        b[2:4] = np.array([np.float16(0.25)]).view(np.uint8)
        b[4:8] = [3, 5, 7, 9]            # scales of sub-blocks 0..3 (6-bit), mins follow
        b[8:12] = [1, 2, 3, 4]
        code = rng.integers(0, 32, 256)
        for i in range(4):               # the first four sub-blocks: scale b[4 + i], min b[8 + i]
            for l in range(32):
                c = int(code[32 * i + l])
                b[48 + 32 * (i // 2) + l] |= (c & 15) << (4 * (i & 1))
                b[16 + l] |= (c >> 4) << i
        got = oracle.dequantize(13, b, 256)
        for i in range(4):
            want = np.float32(0.5) * np.float32(b[4 + i]) * code[32 * i:32 * i + 32].astype(np.float32) - np.float32(0.25) * np.float32(b[8 + i])
            assert np.array_equal(got[32 * i:32 * i + 32], want.astype(np.float32))
    else:
        b = np.zeros(210, np.uint8)
        b[208:210] = np.array([np.float16(0.125)]).view(np.uint8)
        sc = rng.integers(-20, 21, 16).astype(np.int8)
        b[192:208] = sc.view(np.uint8)
        code = rng.integers(0, 64, 256)
        for n in range(2):
            for l in range(32):
                c = [int(code[128 * n + 32 * j + l]) for j in range(4)]
                b[64 * n + l] = (c[0] & 15) | ((c[2] & 15) << 4)
                b[64 * n + 32 + l] = (c[1] & 15) | ((c[3] & 15) << 4)
                b[128 + 32 * n + l] = (c[0] >> 4) | ((c[1] >> 4) << 2) | ((c[2] >> 4) << 4) | ((c[3] >> 4) << 6)
        got = oracle.dequantize(14, b, 256)
        want = np.float32(0.125) * np.repeat(sc, 16).astype(np.float32) * (code - 32).astype(np.float32)
        assert np.array_equal(got, want.astype(np.float32))
    x = (rng.standard_normal((4, 256)) * 0.05).astype(np.float32)
    back = oracle.dequantize(wtype, oracle.quantize(wtype, x), x.size).reshape(4, 256)
    assert np.abs(back - x).max() < np.abs(x).max() / (2 ** bits - 1) * 1.6


def test_iq3xxs_closed_form(oracle):
    """IQ3_XXS (dequant.cpp:157-174): lattice index 0 is the point (4, 4, 4, 4); the scale nibble s gives d (0.5 + s) / 2;
    the seven stored sign bits are completed by a parity bit, so one stored minus sign makes the eighth weight negative too."""
    b = np.zeros(98, np.uint8)
    b[0:2] = np.array([np.float16(0.25)]).view(np.uint8)
    words = np.zeros(8, np.uint32)
    words[0] = 3 << 28                        # sub-block 0: scale nibble 3, no minus signs
    words[1] = (1 << 28) | 0b0000001          # sub-block 1: first group has weight 0 negative -> parity makes weight 7 negative
    words[2] = (15 << 28) | (0b0000011 << 7)  # sub-block 2: second group, weights 0 and 1 negative, parity even
    b[66:98] = words.view(np.uint8)
    got = oracle.dequantize(oracle.IQ3_XXS, b, 256)
    assert np.array_equal(got[0:32], np.full(32, 0.25 * 3.5 * 0.5 * 4, np.float32))
    want1 = np.full(32, 0.25 * 1.5 * 0.5 * 4, np.float32)
    want1[[0, 7]] *= -1
    assert np.array_equal(got[32:64], want1)
    want2 = np.full(32, 0.25 * 15.5 * 0.5 * 4, np.float32)
    want2[[8, 9]] *= -1
    assert np.array_equal(got[64:96], want2)
    # every lattice point has magnitudes from the eight levels, and the table's points are distinct
    idx = np.zeros(98, np.uint8)
    idx[0:2] = np.array([np.float16(1.0)]).view(np.uint8)
    pts = set()
    for base in range(0, 256, 64):
        idx[2:66] = np.arange(base, base + 64, dtype=np.uint8)
        v = oracle.dequantize(oracle.IQ3_XXS, idx, 256) * 4        # d (0.5 + 0) / 2 = 0.25
        assert set(np.unique(v).tolist()) <= {4.0, 12.0, 20.0, 28.0, 36.0, 44.0, 52.0, 62.0}
        pts |= {tuple(r) for r in v.reshape(64, 4).tolist()}
    assert len(pts) == 256


def test_iq2s_closed_form(oracle):
    """IQ2_S (dequant.cpp:271-287): lattice index 0 is the point of eight 8s; the low scale nibble serves the first 16 weights
    of a sub-block, the high one the other 16; a sign byte's bit j negates weight j of its group; qh adds 256 per two bits."""
    b = np.zeros(82, np.uint8)
    b[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    b[74] = 0x53                 # sub-block 0: nibble 3 for weights 0..15, 5 for 16..31
    b[34] = 0b10000001           # group 0: weights 0 and 7 negative
    got = oracle.dequantize(oracle.IQ2_S, b, 256)
    want = np.concatenate([np.full(16, 0.5 * 3.5 * 0.25 * 8), np.full(16, 0.5 * 5.5 * 0.25 * 8)]).astype(np.float32)
    want[[0, 7]] *= -1
    assert np.array_equal(got[:32], want)
    assert np.array_equal(got[32:], np.full(224, 0.5 * 0.5 * 0.25 * 8, np.float32))
    # the index reaches all 1024 points through qh; they are distinct and their magnitudes are the three levels
    pts = set()
    blk = np.zeros(82, np.uint8)
    blk[0:2] = np.array([np.float16(1.0)]).view(np.uint8)
    for hi in range(4):
        blk[66:74] = hi * 0x55                       # the same two high bits for the four groups of every sub-block
        for base in range(0, 256, 32):
            blk[2:34] = np.arange(base, base + 32, dtype=np.uint8)
            v = oracle.dequantize(oracle.IQ2_S, blk, 256) * 8          # d (0.5 + 0) / 4 = 0.125
            assert set(np.unique(v).tolist()) <= {8.0, 25.0, 43.0}
            pts |= {tuple(r) for r in v.reshape(32, 8).tolist()}
    assert len(pts) == 1024


def test_q4_0_closed_form(oracle):
    """Q4_0 (dequant.cpp:480-491): byte j of a block holds weight j (low nibble) and weight j + 16 (high), value (q - 8) d."""
    b = np.zeros(18, np.uint8)
    b[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    b[2:18] = np.arange(16, dtype=np.uint8) | ((15 - np.arange(16, dtype=np.uint8)) << 4)
    got = oracle.dequantize(oracle.Q4_0, b, 32)
    want = np.concatenate([np.arange(16) - 8, 7 - np.arange(16)]).astype(np.float32) * 0.5
    assert np.array_equal(got, want)


def test_q3k_closed_form(oracle):
    """Q3_K (dequant.cpp:66-76, 118-131): weight 128 n + 32 j + w takes two bits of qs[32 n + w] at 2 j and its third bit from
    hmask[w] at 4 n + j (set: +0, clear: -4); scale 8 n + 2 j + (w >= 16) of sixteen 6-bit scales, each taken minus 32."""
    rng = np.random.default_rng(3)
    hm = rng.integers(0, 256, 32, dtype=np.uint8)
    qs = rng.integers(0, 256, 64, dtype=np.uint8)
    sc6 = rng.integers(0, 64, 16)
    packed = np.zeros(12, np.uint8)
    for i in range(16):           # the layout the reference unpacks: low nibbles in bytes 0..7, upper two bits in bytes 8..11
        packed[i % 8] |= (sc6[i] & 15) << (4 * (i // 8))
        packed[8 + i % 4] |= (sc6[i] >> 4) << (2 * (i // 4))
    b = np.concatenate([hm, qs, packed, np.array([np.float16(0.25)]).view(np.uint8)])
    got = oracle.dequantize(oracle.Q3_K, b, 256)
    e = np.arange(256)
    n, j, w = e // 128, (e % 128) // 32, e % 32
    q = ((qs[32 * n + w] >> (2 * j)) & 3).astype(np.int32) - 4 * (1 - ((hm[w] >> (4 * n + j)) & 1).astype(np.int32))
    want = (np.float32(0.25) * (sc6[8 * n + 2 * j + (w >= 16)] - 32).astype(np.float32)) * q.astype(np.float32)
    assert np.array_equal(got, want.astype(np.float32))
    assert q.min() == -4 and q.max() == 3


def test_q2k_closed_form(oracle):
    """Q2_K (dequant.cpp:289-310): weight 128 n + 32 j + w takes two bits of qs[32 n + w] at 2 j; byte 8 n + 2 j + (w >= 16) of
    the sixteen holds its scale (low nibble) and minimum (high): (d scale) q - dmin minimum."""
    rng = np.random.default_rng(4)
    sc = rng.integers(0, 256, 16, dtype=np.uint8)
    qs = rng.integers(0, 256, 64, dtype=np.uint8)
    b = np.concatenate([sc, qs, np.array([np.float16(0.25), np.float16(0.5)]).view(np.uint8)])
    got = oracle.dequantize(oracle.Q2_K, b, 256)
    e = np.arange(256)
    n, j, w = e // 128, (e % 128) // 32, e % 32
    s = sc[8 * n + 2 * j + (w >= 16)]
    q = (qs[32 * n + w] >> (2 * j)) & 3
    want = (np.float32(0.25) * (s & 15).astype(np.float32)) * q.astype(np.float32) - np.float32(0.5) * (s >> 4).astype(np.float32)
    assert np.array_equal(got, want.astype(np.float32))


def test_iq1s_closed_form(oracle):
    """IQ1_S (dequant.cpp:311-326): values -1, 0, 1 shifted by +-1/8 (bit 15 of the sub-block's qh: minus), times d (2 s + 1)
    with s in bits 12..14; the lattice index is the qs byte plus three bits of qh per group of eight weights."""
    blk = np.zeros(50, np.uint8)
    blk[0:2] = np.array([np.float16(1.0)]).view(np.uint8)
    qh = np.zeros(8, np.uint16)
    qh[1] = (5 << 12) | 0x8000
    pts = set()
    for hi in range(8):
        qh[0] = hi | hi << 3 | hi << 6 | hi << 9
        blk[34:50] = qh.view(np.uint8)
        for base in range(0, 256, 4):
            blk[2:6] = np.arange(base, base + 4, dtype=np.uint8)
            v = oracle.dequantize(oracle.IQ1_S, blk, 256)
            assert set(np.unique(v[:32]).tolist()) <= {-0.875, 0.125, 1.125}
            pts |= {tuple(r) for r in v[:32].reshape(4, 8).tolist()}
    assert len(pts) == 2048
    first = oracle.dequantize(oracle.IQ1_S, blk, 256)
    g0 = first[64:72] - np.float32(0.125)                     # lattice point 0 (sub-block 2: index 0, scale 1, plus shift)
    assert set(np.unique(g0).tolist()) <= {-1.0, 0.0, 1.0}
    assert np.array_equal(first[32:40], np.float32(11.0) * (g0 - np.float32(0.125)))


@pytest.mark.parametrize("wtype,points", [(16, 256), (17, 512)])
def test_iq2xxs_iq2xs_closed_form(oracle, wtype, points):
    """IQ2_XXS (dequant.cpp:233-249) and IQ2_XS (252-268): lattice index 0 is the point of eight 8s; d (0.5 + s) / 4 with s
    the word's top nibble (IQ2_XXS) or a nibble per 16 weights (IQ2_XS); seven stored sign bits completed by a parity bit."""
    el, bb = oracle.BLOCK[wtype]
    b = np.zeros(bb, np.uint8)
    b[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    if wtype == 16:
        w = np.zeros(16, np.uint32)
        w[1] = (3 << 28) | 0b0000001             # sub-block 0: scale 3, group 0 weight 0 negative -> weight 7 too
        w[3] = (5 << 28) | (0b0000011 << 14)     # sub-block 1: scale 5, group 2 weights 0 and 1 negative
        b[2:66] = w.view(np.uint8)
        want0 = np.full(32, 0.5 * 3.5 * 0.25 * 8, np.float32)
        want1 = np.full(32, 0.5 * 5.5 * 0.25 * 8, np.float32)
    else:
        q = np.zeros(32, np.uint16)
        q[0] = 0b0000001 << 9
        q[6] = 0b0000011 << 9
        b[2:66] = q.view(np.uint8)
        b[66], b[67] = 0x73, 0x95                # sub-block 0: nibbles 3 | 7, sub-block 1: 5 | 9
        want0 = np.concatenate([np.full(16, 0.5 * 3.5 * 0.25 * 8), np.full(16, 0.5 * 7.5 * 0.25 * 8)]).astype(np.float32)
        want1 = np.concatenate([np.full(16, 0.5 * 5.5 * 0.25 * 8), np.full(16, 0.5 * 9.5 * 0.25 * 8)]).astype(np.float32)
    want0[[0, 7]] *= -1
    want1[[16, 17]] *= -1
    got = oracle.dequantize(wtype, b, 256)
    assert np.array_equal(got[0:32], want0) and np.array_equal(got[32:64], want1)
    assert np.array_equal(got[64:], np.full(192, 0.5 * 0.5 * 0.25 * 8, np.float32))
    # every point of the lattice is reached, the points are distinct and their magnitudes are the three levels
    blk = np.zeros(bb, np.uint8)
    blk[0:2] = np.array([np.float16(1.0)]).view(np.uint8)
    pts = set()
    for base in range(0, points, 32):
        if wtype == 16:
            idx = np.zeros((8, 8), np.uint8)
            idx[:, 0:4] = np.arange(base, base + 32, dtype=np.uint8).reshape(8, 4)
            blk[2:66] = idx.reshape(-1)
        else:
            blk[2:66] = np.arange(base, base + 32, dtype=np.uint16).view(np.uint8)
        v = oracle.dequantize(wtype, blk, 256) * 8
        assert set(np.unique(v).tolist()) <= {8.0, 25.0, 43.0}
        pts |= {tuple(r) for r in v.reshape(32, 8).tolist()}
    assert len(pts) == points


@pytest.mark.parametrize("wtype", [2, 8, 10, 11, 12, 13, 14, 16, 17, 18, 19, 20, 21, 22, 23, 323])
def test_decoders_match_reference_objects(oracle, ref, wtype):
    rng = np.random.default_rng(wtype)
    el, bb = oracle.BLOCK[wtype]
    nb = 64
    raw = rng.integers(0, 256, (nb, bb), dtype=np.uint8)
    halves = {2: [0], 10: [80, 82], 19: [0], 11: [108], 16: [0], 17: [0], 8: [0], 12: [0, 2], 13: [0, 2], 14: [208], 18: [0], 20: [0], 21: [0], 22: [0], 23: [0]}.get(wtype, [])
    for off in halves:
        raw[:, off:off + 2] = np.float16(rng.uniform(1e-3, 5e-2, nb) * rng.choice([-1, 1], nb)).view(np.uint8).reshape(nb, 2)
    if wtype == 323:
        raw[:, 0:4] = rng.uniform(1e-3, 2e-2, nb).astype(np.float32).view(np.uint8).reshape(nb, 4)
    got = oracle.dequantize(wtype, raw, nb * el)
    want = np.empty(nb * el, np.float32)
    assert ref.ref_dequantize(wtype, raw.ctypes.data_as(C.c_void_p), want.ctypes.data_as(C.c_void_p), nb * el) == 0
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # NaNs (E4M3 0x7F scales) compare by bits


def test_conversions_match_reference_objects(oracle, ref):
    for h in range(0, 65536, 7):
        a, b = oracle.half_to_float(h), ref.ref_half_to_float(h)
        assert (np.isnan(a) and np.isnan(b)) or a == b
    rng = np.random.default_rng(5)
    for v in rng.standard_normal(5000).astype(np.float32) * 10.0 ** rng.uniform(-9, 6, 5000).astype(np.float32):
        assert oracle.float_to_half(float(v)) == ref.ref_float_to_half(float(v))
    for b in range(256):
        a, r = oracle.e4m3_to_float(b), ref.ref_e4m3_to_float(b)
        assert (np.isnan(a) and np.isnan(r)) or a == r


# relative round-trip error (rms(decode(encode(w)) - w) / rms(w)) each encoder must stay under on N(0, 0.02) weights
ROUND_TRIP = {12: 0.09, 20: 0.09, 23: 0.09, 21: 0.20, 323: 0.12}


@pytest.mark.parametrize("wtype", sorted(ROUND_TRIP))
def test_encoders_round_trip(oracle, wtype):
    rng = np.random.default_rng(100 + wtype)
    w = (rng.standard_normal((16, 1024)) * 0.02).astype(np.float32)
    raw = oracle.quantize(wtype, w)
    el, bb = oracle.BLOCK[wtype]
    assert raw.size == w.size // el * bb
    back = oracle.dequantize(wtype, raw, w.size).reshape(w.shape)
    assert np.isfinite(back).all()
    rel = np.sqrt(np.mean((back - w) ** 2) / np.mean(w ** 2))
    assert rel < ROUND_TRIP[wtype], rel
    # zeros encode to blocks that decode to zeros
    z = oracle.dequantize(wtype, oracle.quantize(wtype, np.zeros((1, 1024), np.float32)), 1024)
    assert not z.any()

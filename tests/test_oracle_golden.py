"""Pins the CPU oracle: golden vectors the reference's own tests hold, closed forms, invariants and
brute force — each chosen so that a dropped term, a wrong index or a transposed nibble fails."""
import json
import os

import numpy as np
import pytest

Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11

# the reference's own regression digests (crates/ojas-formats/tests/quant_formats.rs:36-48), kept as a fixture
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "quant_format_digests.json")) as _f:
    _GOLDEN = json.load(_f)["digests"]
DIGESTS = {int(ty): int(row["digest"], 16) for ty, row in _GOLDEN.items()}
COUNTS = {int(ty): row["values"] for ty, row in _GOLDEN.items()}
# crates/ojas-core/src/iq_tables.rs:881-884
KVALUES_IQ4NL = np.array([-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113], np.float64)


IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29
GRID_TYPES = [IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M]


@pytest.mark.parametrize("ty", [Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS] + GRID_TYPES)
def test_dequant_digest_matches_reference(orc, pkg, ty):
    wpb = pkg.synth.BLOCK_SHAPE[ty][1]
    raw = orc.synth_blocks(ty, 40)
    bits = orc.dequant_to_f16(raw, ty, 40 * wpb)
    assert bits.size == 40 * wpb == COUNTS[ty]        # 10240 values; 1280 for the 32-weight IQ4_NL block
    assert orc.digest_f16(bits) == DIGESTS[ty]


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS, Q4_0, Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, 139] + GRID_TYPES)
def test_synth_blocks_two_implementations_agree(orc, pkg, ty):
    assert np.array_equal(orc.synth_blocks(ty, 9), pkg.synth.synth_blocks(ty, 9))


def test_f16_to_f32_exhaustive(orc):
    L = orc.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.ojo_f16_to_f32(int(b)) for b in bits], np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f32_to_f16_round_to_nearest_even(orc):
    L = orc.lib()
    rng = np.random.default_rng(1)
    # every f16 value, every midpoint between neighbours, and random f32 across all exponents
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    rnd = (rng.standard_normal(20000) * np.exp2(rng.integers(-30, 18, 20000))).astype(np.float32)
    tiny = (rng.standard_normal(5000) * 2.0 ** -24).astype(np.float32)
    special = np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, np.inf, -np.inf, 2.0 ** -25,
                        2.0 ** -25 * 1.0000001, 2.0 ** -24, 6.1e-5], np.float32)
    xs = np.concatenate([h.astype(np.float32), mids, -mids, rnd, tiny, special])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([L.ojo_f32_to_f16(float(v)) for v in xs], np.uint16)
    assert np.array_equal(got, want)


def test_bf16_rounding(orc, pkg):
    L = orc.lib()
    xs = np.random.default_rng(2).standard_normal(4000).astype(np.float32)
    got = np.array([L.ojo_f32_to_bf16(float(v)) for v in xs], np.uint16)
    assert np.array_equal(got, pkg.synth.to_bf16_bits(xs))
    # ties go to even: 1 + 2^-8 is exactly between two bf16 values
    assert L.ojo_f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    assert L.ojo_f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82


def test_q80_table_closed_form(orc, pkg):
    """crates/ojas-formats/tests/rows.rs:13-18: d = 0.25 (r+1), q_j = j - 16 + r — all exact."""
    raw, want = pkg.synth.q80_rows_table()
    got = orc.dequant_to_f16(raw, Q8_0, 96).view(np.float16).astype(np.float32).reshape(3, 32)
    assert np.array_equal(got, want)


def _q4k_block(d, dmin, sc, mn, qs, pkg):
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.array([d], np.float16).view(np.uint8)
    blk[2:4] = np.array([dmin], np.float16).view(np.uint8)
    blk[4:16] = pkg.synth.pack_scales_k4(np.array([sc]), np.array([mn]))[0]
    blk[16:] = qs
    return blk


def test_q4k_closed_forms(orc, pkg):
    # all-zero quants => w = -dmin * m_j, constant per sub-block, in sub-block order
    mn = np.arange(8) * 7 + 3
    blk = _q4k_block(0.5, 0.25, np.full(8, 9), mn, np.zeros(128, np.uint8), pkg)
    w = orc.dequant_to_f16(blk, Q4_K, 256).view(np.float16).astype(np.float32).reshape(8, 32)
    assert np.array_equal(w, np.repeat((-0.25 * mn).astype(np.float32)[:, None], 32, 1))
    # sc = 1, m = 0 => w = d * nibble; low nibbles feed sub-block 2c, high nibbles 2c+1
    qs = np.random.default_rng(3).integers(0, 256, 128, dtype=np.uint8)
    blk = _q4k_block(2.0, 1.0, np.ones(8), np.zeros(8), qs, pkg)
    w = orc.dequant_to_f16(blk, Q4_K, 256).view(np.float16).astype(np.float32).reshape(4, 2, 32)
    q = qs.reshape(4, 32)
    assert np.array_equal(w[:, 0], 2.0 * (q & 15))
    assert np.array_equal(w[:, 1], 2.0 * (q >> 4))
    # scales with the top bits set exercise the j >= 4 packing
    sc = np.array([1, 2, 3, 4, 63, 48, 33, 17])
    blk = _q4k_block(1.0, 1.0, sc, sc[::-1].copy(), np.full(128, 0x11, np.uint8), pkg)
    w = orc.dequant_to_f16(blk, Q4_K, 256).view(np.float16).astype(np.float32).reshape(8, 32)
    assert np.array_equal(w[:, 0], (sc - sc[::-1]).astype(np.float32))


def test_q6k_closed_forms(orc):
    blk = np.zeros(210, np.uint8)
    blk[208:210] = np.array([1.0], np.float16).view(np.uint8)
    blk[192:208] = np.arange(1, 17, dtype=np.int8).view(np.uint8)
    # code 32 (ql nibble 0, qh bits = 2) decodes to 0
    blk[0:128] = 0
    blk[128:192] = 0xAA
    assert not orc.dequant_to_f16(blk, Q6_K, 256).any()
    # code 33 => w = d * sc[sub]; sub-scales apply per 16 weights in element order
    blk[0:128] = 0x11
    w = orc.dequant_to_f16(blk, Q6_K, 256).view(np.float16).astype(np.float32)
    assert np.array_equal(w, np.repeat(np.arange(1, 17, dtype=np.float32), 16))
    # a single byte of ql / qh lands where the layout says
    blk[0:192] = 0
    blk[5] = 0xF0           # ql[5] high nibble -> weight 64+5 of the first half
    blk[128 + 32 + 7] = 0x0C  # qh[7] of the second half, bits 2..3 -> weight 128+32+7
    w = orc.dequant_to_f64(blk, Q6_K, 256)
    base = -32.0 * np.repeat(np.arange(1, 17, dtype=np.float64), 16)
    delta = w - base
    assert delta[64 + 5] == 15 * 5.0 and delta[128 + 32 + 7] == 48 * 11.0
    assert np.count_nonzero(delta) == 2


@pytest.mark.parametrize("ty", [Q8_0, Q4_K, Q5_K, Q6_K])
def test_dequant_f64_rounds_to_the_f16_decoder(orc, pkg, ty):
    raw = orc.synth_blocks(ty, 12)
    n = 12 * pkg.synth.BLOCK_SHAPE[ty][1]
    exact = orc.dequant_to_f64(raw, ty, n)
    f16 = orc.dequant_to_f16(raw, ty, n).view(np.float16).astype(np.float64)
    # the f16 decoder rounds twice (f32 then f16): within one f16 ulp of the exact value
    assert np.all(np.abs(f16 - exact) <= np.maximum(np.abs(exact) * 2.0 ** -10, 2.0 ** -24))


def test_quant_q8k_invariants(orc):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(1024).astype(np.float32)
    x[256:512] = 0.0                      # all-zero segment => scale 1, q 0
    s, q, b = orc.quant_q8k(x)
    assert s[1] == 1.0 and not q[256:512].any()
    for sb in (0, 2, 3):
        seg = x[sb * 256:(sb + 1) * 256]
        assert s[sb] == np.float32(np.max(np.abs(seg))) / np.float32(127.0)
        assert np.max(np.abs(q[sb * 256:(sb + 1) * 256])) == 127
        assert np.all(np.abs(seg - s[sb] * q[sb * 256:(sb + 1) * 256]) <= s[sb] * 0.5000001)
    assert np.array_equal(b, q.astype(np.int32).reshape(-1, 32).sum(1))
    # ties round away from zero: amax = 127 makes scale 1, so x = +-2.5 must give +-3
    x = np.zeros(256, np.float32)
    x[0], x[1], x[2], x[3] = 127.0, 2.5, -2.5, 0.49999997
    _, q, _ = orc.quant_q8k(x)
    assert list(q[:4]) == [127, 3, -3, 0]
    # ragged tail: K = 300 quantizes the 44-element tail on its own scale, pads with zero
    x = rng.standard_normal(300).astype(np.float32)
    s, q, b = orc.quant_q8k(x)
    assert s.size == 2 and q.size == 512 and not q[300:].any()
    assert s[1] == np.float32(np.max(np.abs(x[256:]))) / np.float32(127.0)
    # non-finite inputs, as Rust's `fold(max)`, `clamp` and `as i8` treat them (cpu_math.rs:552-557): a NaN does not
    # enter the maximum and quantizes to 0; an infinity makes the scale infinite, 1/scale zero, and every code of its
    # segment 0 (finite * 0 = 0, inf * 0 = NaN -> 0)
    x = rng.standard_normal(512).astype(np.float32)
    x[5], x[300], x[301] = np.nan, np.inf, -np.inf
    s, q, b = orc.quant_q8k(x)
    finite = np.delete(x[:256], 5)
    assert s[0] == np.float32(np.max(np.abs(finite))) / np.float32(127.0) and q[5] == 0
    assert np.max(np.abs(q[:256])) == 127
    assert np.isinf(s[1]) and not q[256:].any() and not b[8:].any()


def test_dot_q80_matches_f64_dot(orc, pkg):
    n, k = 7, 320
    raw = pkg.synth.q80_weights(n, k, "t", "q80")
    x = pkg.synth.normal_f32(k, "t", "x")
    w = orc.dequant_to_f64(raw, Q8_0, n * k).reshape(n, k)
    want = w @ x.astype(np.float64)
    got = np.array([orc.dot_q80(raw[r * 340:(r + 1) * 340], x) for r in range(n)])
    assert np.max(np.abs(got - want)) <= 1e-6 * np.max(np.abs(want))
    # brute force on one block, in the reference's order: sum = d * (sequential f32 acc)
    blk = raw[:34]
    acc = np.float32(0)
    for j in range(32):
        acc = np.float32(acc + np.float32(np.int8(blk[2 + j])) * x[j])
    d = blk[0:2].view(np.float16).astype(np.float32)[0]
    assert orc.dot_q80(blk, x[:32]) == np.float32(d * acc)


@pytest.mark.parametrize("ty", [Q4_0, Q4_1, Q5_0, Q5_1])
def test_legacy_block_closed_forms(orc, pkg, ty):
    """The 32-weight blocks against their definitions in numpy (the reference's tests hold no digest for
    them): w = d (q - 8), d q + m, d (q5 - 16), d q5 + m; low nibbles are weights 0..15, high nibbles
    16..31; the fifth bit of weight j is bit j of the little-endian qh field; and the f16 decoder equals
    the f32 expression of the reference (a product, then where the format has one a sum, each rounded)."""
    bb = pkg.synth.BLOCK_SHAPE[ty][0]
    raw = orc.synth_blocks(ty, 50).reshape(50, bb).copy()
    g = np.random.default_rng(ty)
    raw[:, 2:4] = (g.standard_normal(50) * 0.3).astype(np.float16).view(np.uint8).reshape(50, 2)   # m (or qh / qs bytes)
    five, affine = ty in (Q5_0, Q5_1), ty in (Q4_1, Q5_1)
    hdr = 4 if affine else 2
    d = raw[:, 0:2].copy().view(np.float16).astype(np.float32)[:, 0]
    m = raw[:, 2:4].copy().view(np.float16).astype(np.float32)[:, 0] if affine else np.zeros(50, np.float32)
    qh = raw[:, hdr:hdr + 4].copy().view(np.uint32)[:, 0] if five else np.zeros(50, np.uint32)
    qs = raw[:, hdr + (4 if five else 0):]
    j = np.arange(16)
    lo = (qs & 0xF).astype(np.uint32) | (((qh[:, None] >> j) & 1) << 4)
    hi = (qs >> 4).astype(np.uint32) | (((qh[:, None] >> (j + 16)) & 1) << 4)
    q = np.concatenate([lo, hi], axis=1).astype(np.float32)
    if affine:
        want32 = (d[:, None] * q).astype(np.float32) + m[:, None]
    else:
        want32 = d[:, None] * (q - np.float32(16.0 if five else 8.0))
    with np.errstate(over="ignore"):
        want16 = want32.astype(np.float32).astype(np.float16).view(np.uint16)
    got16 = orc.dequant_to_f16(raw.reshape(-1), ty, 50 * 32).reshape(50, 32)
    assert np.array_equal(got16, want16)
    got64 = orc.dequant_to_f64(raw.reshape(-1), ty, 50 * 32).reshape(50, 32)
    exact = d.astype(np.float64)[:, None] * (q.astype(np.float64) - (0.0 if affine else (16.0 if five else 8.0))) + m.astype(np.float64)[:, None]
    assert np.array_equal(got64, exact)


@pytest.mark.parametrize("ty", [Q2_K, Q3_K])
def test_two_bit_plane_blocks_against_numpy(orc, pkg, ty):
    """Q2_K and Q3_K decoded weight by weight in numpy from the block definitions: weight i of a super-block
    sits in code byte 32 (i // 128) + i % 32 at bits 2 ((i // 32) % 4), its scale is number i // 16; Q2_K:
    (d sc) q - dmin m with sc, m the nibbles of a scale byte; Q3_K: a third bit in hmask[i % 32] at bit i // 32
    (clear = subtract 4), 6-bit scales biased by 32 whose low nibbles fill bytes 0..7 (low, then high nibble)
    and whose high bit pairs fill bytes 8..11.  The f64 decoder must be exact, the f16 one the f32 expression
    of the reference rounded once more; special blocks: all mask bits set / clear, every scale value."""
    nb = 64
    raw = orc.synth_blocks(ty, nb).reshape(nb, -1).copy()
    if ty == Q3_K:
        raw[0, :32], raw[1, :32] = 0xFF, 0x00
        sc = (np.arange(16) * 4 + 1) % 64     # block 2: scale i = (4 i + 1) % 64, written with the packing rule
        packed = np.zeros(12, np.uint8)
        for i, v in enumerate(sc):
            packed[i % 8] |= (v & 0xF) << (4 * (i // 8))
            packed[8 + i % 4] |= (v >> 4) << (2 * (i // 4))
        raw[2, 96:108] = packed
    i = np.arange(256)
    half, plane, l, grp = i // 128, (i // 32) % 4, i % 32, i // 16
    if ty == Q2_K:
        d = raw[:, 80:82].copy().view(np.float16).astype(np.float64)
        dmin = raw[:, 82:84].copy().view(np.float16).astype(np.float64)
        q = (raw[:, 16 + 32 * half + l] >> (2 * plane)) & 3
        scb = raw[:, grp]
        exact = d * (scb & 0xF) * q - dmin * (scb >> 4)
        dl = (d.astype(np.float32) * (scb & 0xF).astype(np.float32)).astype(np.float32)
        ml = (dmin.astype(np.float32) * (scb >> 4).astype(np.float32)).astype(np.float32)
        f32 = (dl * q.astype(np.float32)).astype(np.float32) - ml
    else:
        d = raw[:, 108:110].copy().view(np.float16).astype(np.float64)
        q = ((raw[:, 32 + 32 * half + l] >> (2 * plane)) & 3).astype(np.int64)
        hbit = (raw[:, l] >> (i // 32)) & 1
        code = q - 4 * (1 - hbit.astype(np.int64))
        sraw = raw[:, 96:108]
        lo = np.where(grp < 8, sraw[:, grp % 8] & 0xF, sraw[:, grp % 8] >> 4)
        hi = (sraw[:, 8 + grp % 4] >> (2 * (grp // 4))) & 3
        s6 = (lo | (hi << 4)).astype(np.int64) - 32
        assert np.array_equal(s6[2, ::16] + 32, (np.arange(16) * 4 + 1) % 64)
        exact = d * s6 * code
        f32 = (d.astype(np.float32) * s6.astype(np.float32)).astype(np.float32) * code.astype(np.float32)
    got64 = orc.dequant_to_f64(raw.reshape(-1), ty, nb * 256).reshape(nb, 256)
    assert np.array_equal(got64, exact)
    with np.errstate(over="ignore"):
        want16 = f32.astype(np.float32).astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.dequant_to_f16(raw.reshape(-1), ty, nb * 256).reshape(nb, 256), want16)


def test_iq4_closed_forms(orc):
    """A block whose every index is c decodes to d * codebook[c] (IQ4_NL) and d * (ls - 32) * codebook[c]
    (IQ4_XS); low nibbles fill the first 16 weights of a 32-group, high nibbles the next 16; the 6-bit
    sub-scale is 4 low bits from scales_l (nibble per sub-block) and 2 high bits from scales_h."""
    d = np.array([0.5], np.float16).view(np.uint8)
    for c in range(16):
        blk = np.concatenate([d, np.full(16, c | ((15 - c) << 4), np.uint8)])
        w = orc.dequant_to_f64(blk, IQ4_NL, 32)
        assert np.all(w[:16] == 0.5 * KVALUES_IQ4NL[c]) and np.all(w[16:] == 0.5 * KVALUES_IQ4NL[15 - c])
    for ib in range(8):
        for ls in (0, 31, 32, 47, 63):
            blk = np.zeros(136, np.uint8)
            blk[0:2] = d
            sh = (ls >> 4) << (2 * ib)
            blk[2], blk[3] = sh & 0xFF, sh >> 8
            blk[4 + ib // 2] = (ls & 0xF) << (4 * (ib % 2))
            blk[8:] = 0x9C                     # low nibble 12 -> 53, high nibble 9 -> 13
            w = orc.dequant_to_f64(blk, IQ4_XS, 256).reshape(8, 32)
            for jb in range(8):
                scale = 0.5 * ((ls if jb == ib else 0) - 32)
                assert np.all(w[jb, :16] == scale * 53) and np.all(w[jb, 16:] == scale * 13), (ib, ls, jb)


@pytest.mark.parametrize("ty", [IQ4_NL, IQ4_XS])
def test_iq4_dot_matches_f64_dot(orc, pkg, ty):
    """dot_iq4nl / dot_iq4xs against the dequantized row in double (the reference's own check,
    crates/ojas-cpu/src/cpu_math.rs:1206-1285), one-hot activations (element order), matvec_kq routing."""
    n, k = 5, 1024
    bb, wpb = pkg.synth.BLOCK_SHAPE[ty]
    rb = k // wpb * bb
    raw = orc.synth_blocks(ty, n * k // wpb)
    x = pkg.synth.normal_f32(k, "t", "xiq", ty)
    w = orc.dequant_to_f64(raw, ty, n * k).reshape(n, k)
    want = w @ x.astype(np.float64)
    got = np.array([orc.dot_iq(ty, raw[r * rb:(r + 1) * rb], x) for r in range(n)])
    assert np.max(np.abs(got - want)) <= 2e-6 * np.max(np.abs(want))
    assert np.array_equal(orc.matvec_kq(raw, ty, n, k, x, threads=3), got.astype(np.float32))
    for i in [0, 1, 15, 16, 17, 31, 32, 47, 48, 255, 256, 272, 1023]:
        e = np.zeros(k, np.float32)
        e[i] = 1.0
        assert orc.dot_iq(ty, raw[:rb], e) == np.float32(w[0, i]), (ty, i)


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K])
def test_kquant_dot_equals_dequant_dot_on_quantized_activations(orc, pkg, ty):
    """dot_<fmt>(row, quant_q8k(x)) == sum dequant(row) * (scale * q), evaluated in double."""
    n, k = 6, 1024
    bb = pkg.synth.BLOCK_SHAPE[ty][0]
    raw = orc.synth_blocks(ty, n * k // 256)
    x = pkg.synth.normal_f32(k, "t", "xk", ty)
    act = orc.quant_q8k(x)
    xq = (np.repeat(act[0].astype(np.float64), 256) * act[1].astype(np.float64))
    w = orc.dequant_to_f64(raw, ty, n * k).reshape(n, k)
    want = w @ xq
    rb = k // 256 * bb
    got = np.array([orc.dot_kq(ty, raw[r * rb:(r + 1) * rb], k, act) for r in range(n)])
    assert np.max(np.abs(got - want)) <= 2e-6 * np.max(np.abs(want))
    y = orc.matvec_kq(raw, ty, n, k, x, threads=3)
    assert np.array_equal(y, got.astype(np.float32))


@pytest.mark.parametrize("ty", [Q4_K, Q5_K, Q6_K])
def test_kquant_dot_one_hot_selects_the_weight(orc, pkg, ty):
    """x = e_i quantizes to scale 1/127, q_i = 127, so the dot returns w_i: pins element order."""
    k = 512
    bb = pkg.synth.BLOCK_SHAPE[ty][0]
    raw = orc.synth_blocks(ty, 2)
    w = orc.dequant_to_f64(raw, ty, k)
    for i in [0, 1, 15, 16, 31, 32, 33, 63, 64, 100, 127, 128, 129, 200, 255, 256, 300, 511]:
        x = np.zeros(k, np.float32)
        x[i] = 1.0
        got = orc.dot_kq(ty, raw[:2 * bb], k, orc.quant_q8k(x))
        assert abs(got - w[i]) <= 1e-6 * max(abs(w[i]), 1e-3), (ty, i)


def test_dot_q4k_brute_force_association(orc, pkg):
    """One super-block, restated term by term in f32 in the reference's order."""
    raw = orc.synth_blocks(Q4_K, 1)
    x = pkg.synth.normal_f32(256, "bf")
    s, q, b = orc.quant_q8k(x)
    d, dmin = raw[0:4].view(np.float16).astype(np.float32)
    sc = raw[4:16]
    f = np.float32
    sumd = f(0)
    summ = f(0)
    for c in range(4):
        qq = raw[16 + 32 * c:48 + 32 * c]
        def sm(j):
            if j < 4:
                return sc[j] & 63, sc[j + 4] & 63
            return (sc[j + 4] & 15) | ((sc[j - 4] >> 6) << 4), (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)
        s1, m1 = sm(2 * c)
        s2, m2 = sm(2 * c + 1)
        il = int(np.dot((qq & 15).astype(np.int32), q[64 * c:64 * c + 32].astype(np.int32)))
        ih = int(np.dot((qq >> 4).astype(np.int32), q[64 * c + 32:64 * c + 64].astype(np.int32)))
        sumd = f(sumd + f(f(s1) * f(il)))
        sumd = f(sumd + f(f(s2) * f(ih)))
        summ = f(summ + f(f(f(m1) * f(b[2 * c])) + f(f(m2) * f(b[2 * c + 1]))))
    want = f(s[0] * f(f(d * sumd) - f(dmin * summ)))
    assert orc.dot_kq(Q4_K, raw, 256, (s, q, b)) == want


def test_relayout_q4k_q4l(orc):
    n, k = 3, 512
    raw = orc.synth_blocks(Q4_K, n * k // 256)
    nib, qa, qb = orc.relayout_q4k_q4l(raw, k, n)
    lo, hi = nib & 15, nib >> 4
    codes = np.stack([lo, hi], 1).reshape(n, k)          # element 2i low nibble, 2i+1 high
    a = np.repeat(qa.view(np.float16).astype(np.float64), 32).reshape(n, k)
    b = np.repeat(qb.view(np.float16).astype(np.float64), 32).reshape(n, k)
    w = orc.dequant_to_f64(raw, Q4_K, n * k).reshape(n, k)
    # qa, qb carry one f16 rounding each
    assert np.all(np.abs(a * codes + b - w) <= 2.0 ** -10 * (np.abs(a) * 15 + np.abs(b)) + 1e-12)
    # and the codes are exactly the nibbles in element order (d = 1/sc trick: compare to exact codes)
    exact = np.empty((n, k), np.int64)
    blocks = raw.reshape(-1, 144)
    for i, blk in enumerate(blocks):
        q = blk[16:].reshape(4, 32)
        exact.reshape(-1, 256)[i] = np.stack([q & 15, q >> 4], 1).reshape(256)
    assert np.array_equal(codes, exact)


def test_q4l_kernel_weights_round_once(orc):
    """ojo_q4l_weights_f16 = binary16(qa*q + qb) with ONE rounding (the half fma of
    crates/ojas-cuda/src/kernels/gemm_q.rs:112-121), checked against numpy's correctly rounded
    float64 -> float16 conversion of the exact value; a conversion through f32 first would
    double-round and fail this on ties."""
    n, k = 16, 1024
    raw = orc.synth_blocks(Q4_K, n * k // 256)
    nib, qa, qb = orc.relayout_q4k_q4l(raw, k, n)
    codes = np.stack([nib & 15, nib >> 4], 1).reshape(n, k).astype(np.float64)
    a = np.repeat(qa.view(np.float16).astype(np.float64), 32).reshape(n, k)
    b = np.repeat(qb.view(np.float16).astype(np.float64), 32).reshape(n, k)
    with np.errstate(over="ignore", invalid="ignore"):
        want = (a * codes + b).astype(np.float16).reshape(-1)
    got = orc.q4l_weights_f16(raw, k, n).view(np.float16)
    ok = np.isfinite(want)
    assert ok.sum() > 0.9 * want.size
    assert np.array_equal(got.view(np.uint16)[ok], want.view(np.uint16)[ok])
    # and against the dequantized tensor: one extra f16 rounding of each scale, nothing more
    w = orc.dequant_to_f64(raw, Q4_K, n * k)
    assert np.all(np.abs(got.astype(np.float64)[ok] - w[ok]) <= 2.0 ** -9 * (np.abs(a.reshape(-1)[ok]) * 15 + np.abs(b.reshape(-1)[ok])) + 1e-12)


def test_moe_topk_matches_closed_form(orc, pkg):
    """crates/ojas-cuda/tests/conformance.rs:380-408: E=64, K=8, tvec(64, 51)."""
    lg = pkg.synth.tvec(64, 51)
    idx, wgt = orc.moe_topk(lg[None, :], 8)
    ex = np.exp(lg.astype(np.float64) - lg.max())
    p = ex / ex.sum()
    order = sorted(range(64), key=lambda i: (-p[i], i))[:8]
    assert list(idx[0]) == order
    assert np.max(np.abs(wgt[0] - p[order] / p[order].sum())) < 1e-6
    assert abs(float(wgt[0].sum()) - 1.0) < 1e-6
    # ties resolve to the lowest index
    idx, _ = orc.moe_topk(np.zeros((1, 16), np.float32), 4)
    assert list(idx[0]) == [0, 1, 2, 3]


def test_other_routers_match_closed_forms(orc, pkg):
    """nonorm: the raw softmax probabilities of the top-k (crates/ojas-metal/src/kernels/moe.rs:130-150); v3: sigmoid
    scores, chosen by score + bias, weights from the unbiased scores, renormalised and scaled
    (crates/ojas-metal/src/kernels/moe.rs:531-551, crates/ojas-cpu/src/cpu_glm.rs:526-548)."""
    lg = pkg.synth.tvec(64, 51)
    ex = np.exp(lg.astype(np.float64) - lg.max())
    p = ex / ex.sum()
    order = sorted(range(64), key=lambda i: (-p[i], i))[:6]
    idx, wgt = orc.moe_topk_nonorm(lg[None, :], 6)
    assert list(idx[0]) == order
    assert np.max(np.abs(wgt[0] - p[order])) < 1e-6
    assert float(wgt[0].sum()) < 1.0           # not renormalised
    # v3: a bias that reverses the order changes who is chosen and leaves the weights unbiased
    sg = 1.0 / (1.0 + np.exp(-lg.astype(np.float64)))
    bias = (-2.0 * sg).astype(np.float32)      # choice = sg - 2 sg (as f32) : smallest sigmoid wins
    ch = sg.astype(np.float32).astype(np.float64) + bias
    order = sorted(range(64), key=lambda i: (-ch[i], i))[:8]
    for norm, rs in ((True, 1.0), (True, 2.5), (False, 1.0), (False, 0.5)):
        idx, wgt = orc.moe_topk_v3(lg[None, :], bias, 8, rs, norm)
        assert list(idx[0]) == order
        want = sg[order] / (sg[order].sum() if norm else 1.0) * rs
        assert np.max(np.abs(wgt[0] - want)) < 1e-6 * max(1.0, rs)
    # zero bias: plain top-k of the sigmoid = top-k of the logits; ties take the lowest index
    idx, wgt = orc.moe_topk_v3(lg[None, :], np.zeros(64, np.float32), 8, 1.0, True)
    assert list(idx[0]) == sorted(range(64), key=lambda i: (-lg[i], i))[:8]
    assert abs(float(wgt[0].sum()) - 1.0) < 1e-6
    idx, wgt = orc.moe_topk_v3(np.zeros((1, 16), np.float32), np.zeros(16, np.float32), 4, 1.0, False)
    assert list(idx[0]) == [0, 1, 2, 3] and np.all(wgt[0] == 0.5)
    idx, _ = orc.moe_topk_nonorm(np.zeros((1, 16), np.float32), 4)
    assert list(idx[0]) == [0, 1, 2, 3]


def test_q8_1_quantizer_and_integer_dot_restatements(orc, pkg):
    """`quantize_q8_1` (crates/ojas-cuda/src/kernels/gemv.rs:33-52) against its closed form, and the block_q8_0 integer
    dot (crates/ojas-cuda/src/kernels/gemv_q8.rs:178-193) against exact integer arithmetic in f64 and, by the reference's
    own test (crates/ojas-cuda/tests/conformance.rs:563-605: K = 1024, N = 128, x = tvec(K, 81), its block generator),
    within 1e-2 of the output peak of the dequantized dot."""
    k, n = 1024, 128
    x = pkg.synth.tvec(k, 81)
    q8, d8, d8sum = orc.quantize_q8_1(x)
    xb = x.reshape(-1, 32)
    d = (np.abs(xb).max(1) / np.float32(127.0)).astype(np.float32)
    assert np.array_equal(d8, d)
    inv = (np.float32(1.0) / d).astype(np.float32)
    want_q = np.clip(np.rint(xb * inv[:, None]), -127, 127).astype(np.int8)
    assert np.array_equal(q8.reshape(-1, 32), want_q)
    assert np.array_equal(d8sum, d * want_q.sum(1).astype(np.float32))
    assert np.abs(q8.reshape(-1, 32)).max(1).min() == 127          # every block reaches the end of the range
    # an all-zero block: scale 0, codes 0 (id = 0, not 1 / 0)
    z = x.copy(); z[64:96] = 0.0
    qz, dz, sz = orc.quantize_q8_1(z)
    assert dz[2] == 0.0 and sz[2] == 0.0 and not qz[64:96].any()
    w, plain = pkg.synth.q80_rows_mod5(n, k, 82)
    got = orc.gemv_q80_dp4a(w, q8, d8, n, k)
    blocks = w.reshape(n, k // 32, 34)
    dw = blocks[:, :, :2].copy().view(np.float16).astype(np.float64)[:, :, 0]
    wq = blocks[:, :, 2:].view(np.int8).astype(np.int64)
    idot = (wq * q8.reshape(1, -1, 32).astype(np.int64)).sum(2)
    exact = (dw * d8.astype(np.float64)[None, :] * idot).sum(1)
    assert np.max(np.abs(got - exact)) <= 1e-6 * np.max(np.abs(exact))
    reader = (plain.astype(np.float64) * x.astype(np.float64)).sum(1)
    assert np.max(np.abs(got - reader)) / np.max(np.abs(reader)) < 1e-2
    # a transposed operand or a dropped block would not survive this: one nonzero block, one nonzero code
    w1 = np.zeros((1, k // 32, 34), np.uint8)
    w1[0, 5, :2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    w1[0, 5, 2 + 9] = np.uint8(np.int8(-3))
    assert orc.gemv_q80_dp4a(w1.reshape(-1), q8, d8, 1, k)[0] == np.float32(0.5) * d8[5] * np.float32(-3 * int(q8[5 * 32 + 9]))


def test_matmul_q8_row_int8_path(orc):
    rng = np.random.default_rng(7)
    n, k, m = 9, 64, 3
    w = rng.standard_normal((n, k)).astype(np.float16)
    wq, ws = orc.q8_rows_from_f16(w.view(np.uint16), n, k)
    amax = np.abs(w.astype(np.float32)).max(1)
    assert np.array_equal(ws, amax / np.float32(127.0))
    assert np.all(np.abs(wq.reshape(n, k)).max(1) == 127)
    xs = rng.standard_normal((m, k)).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    ys = orc.matmul_q8(wq, ws, n, k, xs, bias)
    for t in range(m):
        q, s = orc.quant_row_i8(xs[t])
        acc = wq.reshape(n, k).astype(np.int64) @ q.astype(np.int64)
        want = bias + acc.astype(np.float32) * ws * np.float32(s)
        assert np.array_equal(ys[t], want.astype(np.float32))


def test_moe_ffn_is_the_composition(orc, pkg):
    E, d, nff, ksel, T = 4, 256, 256, 2, 3
    gate = pkg.synth.q4k_weights(E * nff, d, "m", "g")
    up = pkg.synth.q4k_weights(E * nff, d, "m", "u")
    down = pkg.synth.q4k_weights(E * d, nff, "m", "d")
    x = pkg.synth.normal_f32(T * d, "m", "x").reshape(T, d)
    idx, wgt = orc.moe_topk(pkg.synth.normal_f32(T * E, "m", "lg").reshape(T, E), ksel)
    y = orc.moe_ffn(x, idx, wgt, gate, up, Q4_K, down, Q4_K, E, nff, mode=0)
    gb = nff * d // 256 * 144
    want = np.zeros((T, d), np.float32)
    for t in range(T):
        for j in range(ksel):
            e = int(idx[t, j])
            g = orc.matvec_kq(gate[e * gb:(e + 1) * gb], Q4_K, nff, d, x[t])
            u = orc.matvec_kq(up[e * gb:(e + 1) * gb], Q4_K, nff, d, x[t])
            with np.errstate(over="ignore"):
                act = (g / (np.float32(1) + np.exp(-g, dtype=np.float32))) * u
            dv = orc.matvec_kq(down[e * gb:(e + 1) * gb], Q4_K, d, nff, act.astype(np.float32))
            want[t] += wgt[t, j] * dv
    assert np.max(np.abs(y - want)) <= 2e-6 * np.max(np.abs(want))


def test_rmsnorm_and_activations_closed_forms(orc):
    """rmsnorm (crates/ojas-cpu/src/cpu_math.rs:456-460) and the FFN activations (:486, :497-501)
    against their textbook forms in float64."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal(777).astype(np.float32) * 2.5
    w = (1.0 + 0.2 * rng.standard_normal(777)).astype(np.float32)
    got = orc.rmsnorm(x, w, 1e-5)
    want = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5) * w
    assert np.max(np.abs(got - want)) <= 5e-7 * np.max(np.abs(want))
    assert np.allclose(orc.rmsnorm(np.full(64, 3.0, np.float32), np.ones(64, np.float32), 0.0), 1.0, atol=1e-7)
    g = np.array([-20.0, -3.0, -0.5, 0.0, 0.5, 3.0, 20.0], np.float32)
    g64 = g.astype(np.float64)
    assert np.allclose(orc.ffn_act(g, 0), g64 / (1.0 + np.exp(-g64)), rtol=1e-6, atol=1e-12)
    gelu = 0.5 * g64 * (1.0 + np.tanh(0.7978845608028654 * g64 * (1.0 + 0.044715 * g64 * g64)))
    assert np.allclose(orc.ffn_act(g, 1), gelu, rtol=2e-6, atol=1e-7)


# ------------------------------------------------------------------ grid-codebook formats
def _fnv(data: bytes) -> int:
    h = 0xCBF29CE484222325
    for b in data:
        h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def test_iq_codebooks_expand_to_the_published_tables(orc):
    """The packed codebooks, expanded, hash to the digests taken from the published tables when the header was written
    (tests/golden/iq_grid_digests.json), and hold the entries quoted here from crates/ojas-core/src/iq_tables.rs."""
    with open(os.path.join(os.path.dirname(__file__), "golden", "iq_grid_digests.json")) as f:
        want = json.load(f)["tables"]
    known = {  # (table, entry) -> value, little-endian
        (0, 1): 0x080808080808082B, (0, 2): 0x0808080808081919, (0, 131): 0x082B2B2B19081908, (0, 255): 0x2B2B2B1908081908,
        (1, 259): 0x190808080819082B, (1, 511): 0x2B2B2B2B2B2B2B2B, (2, 515): 0x190808191908192B, (2, 1023): 0x2B2B2B2B2B2B2B2B,
        (3, 0): 0x04040404, (3, 1): 0x04040414, (3, 131): 0x14242C1C, (3, 255): 0x3E341C04,
        (4, 0): 0x01010101, (4, 2): 0x01010105, (4, 259): 0x05090903, (4, 511): 0x0F0F0101,
        (5, 0): 0xFFFFFFFFFFFFFFFF, (5, 1): 0xFFFFFFFFFFFFFF01, (5, 2): 0xFFFFFFFFFFFF0000, (5, 1027): 0xFF01, (5, 2047): 0x0101010101010101,
    }
    for which, name in enumerate(["iq2xxs", "iq2xs", "iq2s", "iq3xxs", "iq3s", "iq1s"]):
        raw = orc.iq_grid_bytes(which)
        row = want[name]
        assert raw.size == row["entries"] * row["entry_bytes"]
        assert _fnv(raw.tobytes()) == int(row["fnv1a64"], 16), name
        table = raw.reshape(row["entries"], row["entry_bytes"])
        for (w, i), v in known.items():
            if w == which:
                assert int.from_bytes(table[i].tobytes(), "little") == v, (name, i)


def _f16(v):
    return np.array([v], np.float16).view(np.uint8)


def test_grid_format_closed_forms(orc):
    """Hand-built blocks: which bits are the grid index, the signs, the sub-block scale, the delta; all products exact."""
    d = 0.5
    # IQ2_XXS: group 3 of sub-block 5 -> entry 1 (43, 8 x 7); sign index 1 = 0b10000001 (even parity): weights 0 and 7 negative
    blk = np.zeros(66, np.uint8)
    blk[0:2] = _f16(d)
    a1 = (9 << 28) | (1 << 21)
    blk[2 + 8 * 5 + 3] = 1
    blk[2 + 8 * 5 + 4:2 + 8 * 5 + 8] = np.frombuffer(int(a1).to_bytes(4, "little"), np.uint8)
    w = orc.dequant_to_f64(blk, IQ2_XXS, 256).reshape(8, 4, 8)
    db = d * 9.5 * 0.25
    assert np.array_equal(w[5, 3], db * np.array([-43, 8, 8, 8, 8, 8, 8, -8.0]))
    assert np.all(w[5, :3] == db * 8) and np.all(w[4] == d * 0.5 * 0.25 * 8)
    # IQ2_XS: 9-bit index 259 (low byte 0x2b ... ) with sign index 2 -> bits 1 and 7; scale nibbles: low for groups 0-1, high for 2-3
    blk = np.zeros(74, np.uint8)
    blk[0:2] = _f16(d)
    q = 259 | (2 << 9)
    blk[2 + 2 * (4 * 6 + 2):2 + 2 * (4 * 6 + 2) + 2] = [q & 0xFF, q >> 8]
    blk[66 + 6] = 0xA3
    w = orc.dequant_to_f64(blk, IQ2_XS, 256).reshape(8, 4, 8)
    e259 = np.array([0x2B, 0x08, 0x19, 0x08, 0x08, 0x08, 0x08, 0x19], np.float64)
    sg = np.array([1, -1, 1, 1, 1, 1, 1, -1.0])
    assert np.array_equal(w[6, 2], d * 10.5 * 0.25 * e259 * sg)
    assert np.all(w[6, 0] == d * 3.5 * 0.25 * 8) and np.all(w[6, 3] == d * 10.5 * 0.25 * 8)
    # IQ2_S: index = qs | (two bits of qh per group) << 8; raw sign byte
    blk = np.zeros(82, np.uint8)
    blk[0:2] = _f16(d)
    blk[2 + 4 * 2 + 1] = 515 & 0xFF
    blk[66 + 2] = (515 >> 8) << 2                     # group l = 1 reads qh bits 2..3
    blk[2 + 32 + 4 * 2 + 1] = 0x05                    # weights 0 and 2 negative
    blk[74 + 2] = 0x07                                # groups 0-1: (0.5 + 7) / 4
    w = orc.dequant_to_f64(blk, IQ2_S, 256).reshape(8, 4, 8)
    e515 = np.array([0x2B, 0x19, 0x08, 0x19, 0x19, 0x08, 0x08, 0x19], np.float64)
    assert np.array_equal(w[2, 1], d * 7.5 * 0.25 * e515 * np.array([-1, 1, -1, 1, 1, 1, 1, 1.0]))
    assert np.all(w[2, 2] == d * 0.5 * 0.25 * 8)
    # IQ3_XXS: two 4-entry indices per group of 8, scale and signs in the trailing 32 bytes
    blk = np.zeros(98, np.uint8)
    blk[0:2] = _f16(d)
    blk[2 + 8 * 1 + 2 * 2] = 131
    blk[2 + 8 * 1 + 2 * 2 + 1] = 255
    a = (4 << 28) | (1 << 14)                           # group 2: sign index 1 -> weights 0 and 7
    blk[66 + 4:66 + 8] = np.frombuffer(int(a).to_bytes(4, "little"), np.uint8)
    w = orc.dequant_to_f64(blk, IQ3_XXS, 256).reshape(8, 4, 8)
    assert np.array_equal(w[1, 2], d * 4.5 * 0.5 * np.array([-0x1C, 0x2C, 0x24, 0x14, 0x04, 0x1C, 0x34, -0x3E], np.float64))
    assert np.all(w[1, 0] == d * 4.5 * 0.5 * 4)
    # IQ3_S: ninth index bit from qh, raw sign bytes, scale 1 + 2 s per 64 weights half by half
    blk = np.zeros(110, np.uint8)
    blk[0:2] = _f16(d)
    blk[2 + 8 * 3 + 2 * 1] = 259 & 0xFF                # sub-block 3, group 1, first index = 259
    blk[66 + 3] = 1 << 2                               # its ninth bit: (h << (8 - 2 l)) & 256 with l = 1
    blk[2 + 8 * 3 + 2 * 1 + 1] = 2                     # second index = 2
    blk[74 + 4 * 3 + 1] = 0x90                         # weights 4 and 7 negative
    blk[106 + 1] = 0x60                                # sub-block 3 = high nibble of scales[1]
    w = orc.dequant_to_f64(blk, IQ3_S, 256).reshape(8, 4, 8)
    assert np.array_equal(w[3, 1], d * 13 * np.array([0x03, 0x09, 0x09, 0x05, -0x05, 0x01, 0x01, -0x01], np.float64))
    assert np.all(w[2] == d * 1)
    # IQ1_S: index = qs | 3 bits of qh << 8, scale 2 s + 1 from bits 12..14, bit 15 flips the delta
    blk = np.zeros(50, np.uint8)
    blk[0:2] = _f16(d)
    blk[2 + 4 * 4 + 2] = 1027 & 0xFF
    qh = (5 << 12) | 0x8000 | ((1027 >> 8) << 6)
    blk[34 + 2 * 4:34 + 2 * 4 + 2] = [qh & 0xFF, qh >> 8]
    w = orc.dequant_to_f64(blk, IQ1_S, 256).reshape(8, 4, 8)
    assert np.array_equal(w[4, 2], d * 11 * (np.array([1, -1, 0, 0, 0, 0, 0, 0.0]) - 0.125))
    assert np.all(w[4, 0] == d * 11 * (-1 - 0.125)) and np.all(w[3] == d * (-1 + 0.125))
    # IQ1_M: d from the top nibbles of the four scale words; two 3-bit scales per sub-block; delta bits 3 and 7 of qh
    blk = np.zeros(56, np.uint8)
    dbits = int(np.array([d], np.float16).view(np.uint16)[0])
    sc = [((dbits >> (4 * i)) & 0xF) << 12 for i in range(4)]
    sc[1] |= (3 << 6) | (6 << 9)                        # sub-block 3 = second half of word 1: scales 3 and 6
    for i in range(4):
        blk[48 + 2 * i:50 + 2 * i] = [sc[i] & 0xFF, sc[i] >> 8]
    blk[4 * 3 + 3] = 1027 & 0xFF                        # group 3: index 1027, high bits from qh[2 * 3 + 1] bits 4..6
    blk[32 + 2 * 3 + 1] = ((1027 >> 8) << 4) | 0x80     # and its delta negative
    w = orc.dequant_to_f64(blk, IQ1_M, 256).reshape(8, 4, 8)
    assert np.array_equal(w[3, 3], d * 13 * (np.array([1, -1, 0, 0, 0, 0, 0, 0.0]) - 0.125))
    assert np.all(w[3, 0] == d * 7 * (-1 + 0.125)) and np.all(w[3, 2] == d * 13 * (-1 + 0.125))
    assert np.all(w[0] == d * 1 * (-1 + 0.125))


@pytest.mark.parametrize("ty", GRID_TYPES)
def test_grid_format_f16_is_the_rounded_exact_value(orc, ty):
    """dequant_to_f16 of random blocks == the exact products (double) rounded once: every factor chain of these formats
    (an f16 d, small odd or half-integer scales, magnitudes below 64) is exact in f32."""
    raw = orc.synth_blocks(ty, 12)
    exact = orc.dequant_to_f64(raw, ty, 12 * 256)
    assert np.array_equal(orc.dequant_to_f16(raw, ty, 12 * 256), exact.astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("ty", [IQ2_XXS, IQ3_XXS, IQ3_S, IQ2_S])
def test_grid_format_f32_dots(orc, pkg, ty):
    """dot_iq2xxs / dot_iq3xxs / dot_iq2s / dot_iq3s against the exactly decoded row in double, one-hot activations
    (element order), and matvec_kq's routing: f32 activations for IQ3_S / IQ2_S, quant_q8k for the two XXS types."""
    n, k = 5, 1024
    rb = k // 256 * pkg.synth.BLOCK_SHAPE[ty][0]
    raw = orc.synth_blocks(ty, n * k // 256)
    x = pkg.synth.normal_f32(k, "t", "xgrid", ty)
    w = orc.dequant_to_f64(raw, ty, n * k).reshape(n, k)
    want = w @ x.astype(np.float64)
    got = np.array([orc.dot_iq(ty, raw[r * rb:(r + 1) * rb], x) for r in range(n)])
    assert np.max(np.abs(got - want)) <= 2e-6 * np.max(np.abs(want))
    for i in [0, 1, 7, 8, 31, 32, 100, 255, 256, 1023]:
        e = np.zeros(k, np.float32)
        e[i] = 1.0
        assert orc.dot_iq(ty, raw[:rb], e) == np.float32(w[0, i]), (ty, i)
    mv = orc.matvec_kq(raw, ty, n, k, x, threads=3)
    if ty in (IQ3_S, IQ2_S):
        assert np.array_equal(mv, got.astype(np.float32))
    else:
        act = orc.quant_q8k(x)
        s, q, _ = act
        ident = np.array([sum(float(s[b]) * (w[r, b * 256:(b + 1) * 256] @ q[b * 256:(b + 1) * 256].astype(np.float64))
                              for b in range(k // 256)) for r in range(n)])
        q8 = np.array([orc.dot_iq_q8k(ty, raw[r * rb:(r + 1) * rb], k, act) for r in range(n)])
        assert np.max(np.abs(q8 - ident)) <= 2e-6 * np.max(np.abs(ident))
        assert np.array_equal(mv, q8.astype(np.float32))
        assert np.max(np.abs(q8 - want)) <= 2e-2 * np.max(np.abs(want))      # activation quantization only


def test_mxfp4_hand_computed_blocks(orc):
    """The reference's own known answers for its 17-byte MXFP4 block (crates/ojas-core/src/quant_src.rs:1376-1420,
    crates/ojas-formats/src/mxfp4.rs:127-160): a codebook sweep at scale 1, code 5 / 13 at scale 2^2, code 2 at 2^-1, and
    the e8m0 table (127 -> 1, 128 -> 2, 126 -> 0.5, 120 -> 2^-7, 0 -> 0); weight 2j is the low nibble of qs[j]."""
    MXFP4 = 139
    a = np.zeros(17, np.uint8)
    a[0] = 127
    a[1:9] = [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]
    wa = orc.dequant_to_f64(a, MXFP4, 32)
    want = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])
    assert np.array_equal(wa[:16], want) and np.array_equal(np.signbit(wa[:16]), np.signbit(want)) and np.all(wa[16:] == 0.0)
    b = np.full(17, 0xD5, np.uint8)
    b[0] = 129
    wb = orc.dequant_to_f64(b, MXFP4, 32)
    assert np.all(wb[0::2] == 12.0) and np.all(wb[1::2] == -12.0)
    c = np.zeros(17, np.uint8)
    c[0], c[1] = 126, 0x22
    wc = orc.dequant_to_f64(c, MXFP4, 32)
    assert wc[0] == 0.5 and wc[1] == 0.5 and np.all(wc[2:] == 0.0)
    for e, v in [(127, 1.0), (128, 2.0), (129, 4.0), (126, 0.5), (120, 2.0 ** -7), (0, 0.0)]:
        blk = np.full(17, 0x22, np.uint8)
        blk[0] = e
        assert np.all(orc.dequant_to_f64(blk, MXFP4, 32) == v), e
    # the f16 decoder is the same value rounded once
    raw = orc.synth_blocks(MXFP4, 64)
    assert np.array_equal(orc.dequant_to_f16(raw, MXFP4, 64 * 32), orc.dequant_to_f64(raw, MXFP4, 64 * 32).astype(np.float16).view(np.uint16))


def test_row_int8_gemv_and_per_token_quantizer_restatements(orc, pkg):
    """`gemv_q8` (crates/ojas-cuda/src/kernels/gemv_q8.rs:31-55) on the generators of the reference's own test
    (crates/ojas-cuda/tests/conformance.rs:248-286: K = 512, N = 256, seeds 11 / 12) against a numpy f64 product, all-ones
    rows and one-hot activations; `quantize_q8_pertoken` (gemv.rs:57-74) against its invariants."""
    k, n = 512, 256
    x = pkg.synth.tvec(k, 11)
    w, scale = pkg.synth.q8_rows(n, k, 12)
    assert w.dtype == np.int8 and np.abs(w.astype(np.int32)).max() <= 127 and 0.01 <= scale.min() and scale.max() <= 0.011
    # the generator itself, value by value on a few entries (Rust: (tvec(1, seed + i)[0] * 127).round())
    for i in (0, 1, 777, n * k - 1):
        v = float(pkg.synth.tvec(1, 12 + i)[0]) * 127.0
        assert int(w.ravel()[i]) == int(np.sign(v) * np.floor(abs(v) + 0.5))
    y = orc.gemv_q8_rows(w, scale, x)
    want = (w.astype(np.float64) @ x.astype(np.float64)).astype(np.float32) * scale
    assert np.array_equal(y, want)
    # the reference's oracle sums in f32, term by term: the two agree far inside its 1e-4 bound
    acc = np.zeros(n, np.float32)
    for i in range(k):
        acc += w[:, i].astype(np.float32) * x[i]
    assert np.max(np.abs(acc * scale - y) / np.maximum(np.abs(y), 1e-6)) < 1e-4
    ones = np.ones((3, k), np.int8)
    assert np.allclose(orc.gemv_q8_rows(ones, np.float32([1, 2, 0.5]), x), np.float32([1, 2, 0.5]) * x.astype(np.float64).sum(), rtol=1e-6)
    e = np.zeros(k, np.float32)
    e[37] = 2.0
    assert np.array_equal(orc.gemv_q8_rows(w, scale, e), (2.0 * w[:, 37].astype(np.float32)) * scale)
    # the per-token quantizer
    xs = pkg.synth.normal_f32(5 * 640, "oracle", "pertoken").reshape(5, 640)
    xs[3] = 0.0
    xs[4, 0] = 127.0                      # d = 1: the codes are rint(x)
    xs[4, 1:5] = [0.5, 1.5, -2.5, 126.5]  # ties go to the even neighbour
    xs[4, 5:] = np.clip(xs[4, 5:], -100, 100)
    q, d = orc.quantize_q8_pertoken(xs)
    assert np.array_equal(d, (np.abs(xs).max(1) / np.float32(127.0)).astype(np.float32))
    assert d[3] == 0.0 and not q[3].any()
    assert list(q[4, :5]) == [127, 0, 2, -2, 126]
    for t in (0, 1, 2):
        assert np.abs(q[t].astype(np.int32)).max() == 127
        assert np.all(np.abs(xs[t] - d[t] * q[t].astype(np.float32)) <= d[t] * 0.5 * (1 + 1e-5))

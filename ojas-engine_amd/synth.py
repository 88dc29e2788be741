"""Seeded synthetic inputs: GGUF block tensors, activations, router logits.

Two kinds of generator live here:
  * the benchmark configurations' own distributions (uniform codes, |N(0, sigma)| f16 scales,
    N(0,1) activations), one numpy PCG64 stream per tensor, seeded from (config, tensor) names;
  * procedures the reference's tests specify in their text, restated so the same bytes can be
    produced anywhere: `synth::blocks` (crates/ojas-formats/src/synth.rs:29-64), the `tvec` LCG
    (crates/ojas-cuda/tests/conformance.rs:223-231) and the closed-form Q8_0 rows of
    crates/ojas-metal/tests/dispatch.rs:357-429 and crates/ojas-formats/tests/rows.rs:13-18.
"""
from __future__ import annotations

import numpy as np

Q8_0, Q4_K, Q5_K, Q6_K, IQ4_NL, IQ4_XS = 8, 12, 13, 14, 20, 23
Q4_0, Q4_1, Q5_0, Q5_1 = 2, 3, 6, 7
Q2_K, Q3_K = 10, 11
IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M = 16, 17, 18, 19, 21, 22, 29
GRID_TYPES = (IQ2_XXS, IQ2_XS, IQ3_XXS, IQ1_S, IQ3_S, IQ2_S, IQ1_M)
MXFP4 = 139     # the reference's synthetic id for its 17-byte MXFP4 blocks (a safetensors format, not a GGUF type)
BLOCK_SHAPE = {Q8_0: (34, 32), Q4_K: (144, 256), Q5_K: (176, 256), Q6_K: (210, 256), IQ4_NL: (18, 32), IQ4_XS: (136, 256),
               Q4_0: (18, 32), Q4_1: (20, 32), Q5_0: (22, 32), Q5_1: (24, 32), Q2_K: (84, 256), Q3_K: (110, 256),
               IQ2_XXS: (66, 256), IQ2_XS: (74, 256), IQ3_XXS: (98, 256), IQ1_S: (50, 256), IQ3_S: (110, 256), IQ2_S: (82, 256),
               IQ1_M: (56, 256), MXFP4: (17, 32)}


def seed_of(*names) -> int:
    """FNV-1a-64 of the joined names: one independent stream per (config, tensor)."""
    h = 0xCBF29CE484222325
    for b in "/".join(str(n) for n in names).encode():
        h ^= b
        h = (h * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def rng(*names) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed_of(*names)))


def normal_f32(n, *names) -> np.ndarray:
    return rng(*names).standard_normal(n, dtype=np.float32)


def to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """f32 -> bf16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = u + 0x7FFF + ((u >> 16) & 1)
    return (u >> 16).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def _f16_abs_normal(g: np.random.Generator, n: int, sigma: float) -> np.ndarray:
    return np.abs(g.standard_normal(n) * sigma).astype(np.float16).view(np.uint16)


# ------------------------------------------------------------------ benchmark distributions
def q80_weights(n: int, k: int, *names) -> np.ndarray:
    """Q8_0 rows: per block d = f16(|N(0,0.02)| / 127), 32 int8 codes uniform in [-127, 127]."""
    g = rng(*names)
    nb = n * (k // 32)
    out = np.empty((nb, 34), np.uint8)
    d = (np.abs(g.standard_normal(nb) * 0.02) / 127.0).astype(np.float16).view(np.uint16)
    out[:, 0] = d & 0xFF
    out[:, 1] = d >> 8
    out[:, 2:] = g.integers(-127, 128, size=(nb, 32), dtype=np.int8).view(np.uint8)
    return out.reshape(-1)


def pack_scales_k4(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """Inverse of get_scale_min_k4 (crates/ojas-formats/src/gguf.rs:1132-1140): 8 six-bit scales
    and 8 six-bit mins per super-block -> the 12 packed bytes."""
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    q = np.empty((sc.shape[0], 12), np.uint8)
    q[:, 0:4] = sc[:, 0:4] | ((sc[:, 4:8] >> 4) << 6)
    q[:, 4:8] = mn[:, 0:4] | ((mn[:, 4:8] >> 4) << 6)
    q[:, 8:12] = (sc[:, 4:8] & 0xF) | ((mn[:, 4:8] & 0xF) << 4)
    return q


def q4k_weights(n: int, k: int, *names) -> np.ndarray:
    """Q4_K rows: d, dmin = f16(|N(0,0.01)|), scales and mins uniform in [0,63], uniform nibbles."""
    g = rng(*names)
    nb = n * (k // 256)
    out = np.empty((nb, 144), np.uint8)
    hdr = np.empty((nb, 2), np.uint16)
    hdr[:, 0] = _f16_abs_normal(g, nb, 0.01)
    hdr[:, 1] = _f16_abs_normal(g, nb, 0.01)
    out[:, 0:4] = hdr.view(np.uint8).reshape(nb, 4)
    out[:, 4:16] = pack_scales_k4(g.integers(0, 64, size=(nb, 8), dtype=np.uint8),
                                  g.integers(0, 64, size=(nb, 8), dtype=np.uint8))
    out[:, 16:] = g.integers(0, 256, size=(nb, 128), dtype=np.uint8)
    return out.reshape(-1)


def q5k_weights(n: int, k: int, *names) -> np.ndarray:
    """Q5_K rows: the Q4_K header, 32 bytes of fifth bits, 128 bytes of nibbles, all uniform."""
    g = rng(*names)
    nb = n * (k // 256)
    out = np.empty((nb, 176), np.uint8)
    hdr = np.empty((nb, 2), np.uint16)
    hdr[:, 0] = _f16_abs_normal(g, nb, 0.01)
    hdr[:, 1] = _f16_abs_normal(g, nb, 0.01)
    out[:, 0:4] = hdr.view(np.uint8).reshape(nb, 4)
    out[:, 4:16] = pack_scales_k4(g.integers(0, 64, size=(nb, 8), dtype=np.uint8),
                                  g.integers(0, 64, size=(nb, 8), dtype=np.uint8))
    out[:, 16:] = g.integers(0, 256, size=(nb, 160), dtype=np.uint8)
    return out.reshape(-1)


def q6k_weights(n: int, k: int, *names) -> np.ndarray:
    """Q6_K rows: uniform 6-bit codes, int8 sub-scales uniform in [-32,31], d = f16(|N(0,0.01)|)."""
    g = rng(*names)
    nb = n * (k // 256)
    out = np.empty((nb, 210), np.uint8)
    out[:, 0:192] = g.integers(0, 256, size=(nb, 192), dtype=np.uint8)
    out[:, 192:208] = g.integers(-32, 32, size=(nb, 16), dtype=np.int8).view(np.uint8)
    d = _f16_abs_normal(g, nb, 0.01)
    out[:, 208] = d & 0xFF
    out[:, 209] = d >> 8
    return out.reshape(-1)


def iq4nl_weights(n: int, k: int, *names) -> np.ndarray:
    """IQ4_NL rows: per 32-weight block d = f16(|N(0,0.02)| / 127), 16 bytes of uniform codebook indices."""
    g = rng(*names)
    nb = n * (k // 32)
    out = np.empty((nb, 18), np.uint8)
    d = (np.abs(g.standard_normal(nb) * 0.02) / 127.0).astype(np.float16).view(np.uint16)
    out[:, 0] = d & 0xFF
    out[:, 1] = d >> 8
    out[:, 2:] = g.integers(0, 256, size=(nb, 16), dtype=np.uint8)
    return out.reshape(-1)


def iq4xs_weights(n: int, k: int, *names) -> np.ndarray:
    """IQ4_XS rows: d = f16(|N(0,0.01)| / 127), the eight 6-bit sub-scales and the 128 index bytes uniform."""
    g = rng(*names)
    nb = n * (k // 256)
    out = np.empty((nb, 136), np.uint8)
    d = (np.abs(g.standard_normal(nb) * 0.01) / 127.0).astype(np.float16).view(np.uint16)
    out[:, 0] = d & 0xFF
    out[:, 1] = d >> 8
    out[:, 2:] = g.integers(0, 256, size=(nb, 134), dtype=np.uint8)
    return out.reshape(-1)


def legacy_weights(ty: int, n: int, k: int, *names) -> np.ndarray:
    """Q4_0 / Q4_1 / Q5_0 / Q5_1 rows: d = f16(|N(0,0.02)| / 8), m = f16(N(0,0.01)) where the format has one,
    every other byte (fifth-bit field, nibbles) uniform."""
    g = rng(*names)
    bb = BLOCK_SHAPE[ty][0]
    nb = n * (k // 32)
    out = g.integers(0, 256, size=(nb, bb), dtype=np.uint8)
    d = (np.abs(g.standard_normal(nb) * 0.02) / 8.0).astype(np.float16).view(np.uint16)
    out[:, 0] = d & 0xFF
    out[:, 1] = d >> 8
    if ty in (Q4_1, Q5_1):
        m = (g.standard_normal(nb) * 0.01).astype(np.float16).view(np.uint16)
        out[:, 2] = m & 0xFF
        out[:, 3] = m >> 8
    return out.reshape(-1)


def q2k_weights(n: int, k: int, *names) -> np.ndarray:
    """Q2_K rows: scales/mins nibbles and 2-bit codes uniform, d = f16(|N(0,0.02)| / 24), dmin = f16(|N(0,0.02)| / 60)
    in the block's last four bytes."""
    g = rng(*names)
    nb = n * (k // 256)
    out = g.integers(0, 256, size=(nb, 84), dtype=np.uint8)
    d = (np.abs(g.standard_normal(nb) * 0.02) / 24.0).astype(np.float16).view(np.uint16)
    m = (np.abs(g.standard_normal(nb) * 0.02) / 60.0).astype(np.float16).view(np.uint16)
    out[:, 80], out[:, 81], out[:, 82], out[:, 83] = d & 0xFF, d >> 8, m & 0xFF, m >> 8
    return out.reshape(-1)


def q3k_weights(n: int, k: int, *names) -> np.ndarray:
    """Q3_K rows: mask bits, 2-bit codes and packed 6-bit scales uniform, d = f16(|N(0,0.02)| / 64) in the last two bytes."""
    g = rng(*names)
    nb = n * (k // 256)
    out = g.integers(0, 256, size=(nb, 110), dtype=np.uint8)
    d = (np.abs(g.standard_normal(nb) * 0.02) / 64.0).astype(np.float16).view(np.uint16)
    out[:, 108], out[:, 109] = d & 0xFF, d >> 8
    return out.reshape(-1)


def weights(ty: int, n: int, k: int, *names) -> np.ndarray:
    if ty in (Q4_0, Q4_1, Q5_0, Q5_1):
        return legacy_weights(ty, n, k, *names)
    if ty in (Q2_K, Q3_K):
        return {Q2_K: q2k_weights, Q3_K: q3k_weights}[ty](n, k, *names)
    if ty in GRID_TYPES:
        return grid_weights(ty, n, k, *names)
    if ty == MXFP4:
        return mxfp4_weights(n, k, *names)
    return {Q8_0: q80_weights, Q4_K: q4k_weights, Q5_K: q5k_weights, Q6_K: q6k_weights,
            IQ4_NL: iq4nl_weights, IQ4_XS: iq4xs_weights}[ty](n, k, *names)


def mxfp4_weights(n: int, k: int, *names) -> np.ndarray:
    """MXFP4 rows: 17-byte blocks, an e8m0 scale exponent uniform in 112..124 (2^-15 .. 2^-3), 16 bytes of E2M1 codes uniform."""
    g = rng("mxfp4", n, k, *names)
    nb = n * (k // 32)
    out = g.integers(0, 256, size=(nb, 17), dtype=np.uint8)
    out[:, 0] = g.integers(112, 125, nb, dtype=np.uint8)
    return out.reshape(-1)


def grid_weights(ty: int, n: int, k: int, *names) -> np.ndarray:
    """Rows of a grid-codebook format: every byte uniform (each bit pattern is a legal block: indices are masked into
    their tables), the block scale d = f16(|N(0, 0.01)| / 16 + 1e-4); IQ1_M spreads its d over the top nibbles of its
    four scale words."""
    bb, _ = BLOCK_SHAPE[ty]
    nb = n * k // 256
    g = rng("grid", ty, n, k, *names)
    blocks = g.integers(0, 256, (nb, bb), dtype=np.uint8)
    d = (np.abs(g.normal(0.0, 0.01, nb)) / 16.0 + 1e-4).astype(np.float32).astype(np.float16).view(np.uint16)
    if ty == IQ1_M:
        for w in range(4):
            blocks[:, 49 + 2 * w] = (blocks[:, 49 + 2 * w] & 0x0F) | ((((d >> (4 * w)) & 0xF) << 4).astype(np.uint8))
    else:
        blocks[:, 0] = (d & 0xFF).astype(np.uint8)
        blocks[:, 1] = (d >> 8).astype(np.uint8)
    return blocks.reshape(-1)


# ------------------------------------------------------------------ the reference tests' procedures
def synth_blocks(ty: int, nb: int) -> np.ndarray:
    """`synth::blocks(t, nb)`: xorshift64 bytes with the f16 scale fields pinned."""
    bb, _ = BLOCK_SHAPE[ty]
    st = 0x2545F4914F6CDD1D
    mask = 0xFFFFFFFFFFFFFFFF
    out = np.empty(nb * bb, np.uint8)
    for i in range(nb * bb):
        st ^= (st << 13) & mask
        st ^= st >> 7
        st ^= (st << 17) & mask
        out[i] = (st >> 24) & 0xFF
    blocks = out.reshape(nb, bb)
    dmin = np.array([0.01], np.float32).astype(np.float16).view(np.uint16)[0]
    for i in range(nb):
        d = (np.float32(0.05) + np.float32(i % 7) * np.float32(0.01)).astype(np.float16).view(np.uint16)
        d = int(d)
        if ty in (Q4_K, Q5_K):
            blocks[i, 0], blocks[i, 1] = d & 0xFF, d >> 8
            blocks[i, 2], blocks[i, 3] = int(dmin) & 0xFF, int(dmin) >> 8
        elif ty == Q6_K:
            blocks[i, 208], blocks[i, 209] = d & 0xFF, d >> 8
        elif ty == Q2_K:
            blocks[i, 80], blocks[i, 81] = d & 0xFF, d >> 8
            blocks[i, 82], blocks[i, 83] = int(dmin) & 0xFF, int(dmin) >> 8
        elif ty == Q3_K:
            blocks[i, 108], blocks[i, 109] = d & 0xFF, d >> 8
        elif ty == MXFP4:      # (not a synth.rs type) an e8m0 exponent near 1.0 in byte 0
            blocks[i, 0] = 120 + i % 7
        elif ty == IQ1_M:      # no d field: f16(0.05) in the top nibbles of the four scale words, low nibble first
            db = int(np.array([0.05], np.float32).astype(np.float16).view(np.uint16)[0])
            for w in range(4):
                blocks[i, 49 + 2 * w] = (int(blocks[i, 49 + 2 * w]) & 0x0F) | (((db >> (4 * w)) & 0xF) << 4)
        else:
            blocks[i, 0], blocks[i, 1] = d & 0xFF, d >> 8
    return out


def tvec(n: int, seed: int) -> np.ndarray:
    """Deterministic vector in [-1, 1) from the reference's test LCG."""
    a, c = np.uint32(1664525), np.uint32(1013904223)
    s0 = np.uint32((seed * 2654435761 + 1) & 0xFFFFFFFF)
    with np.errstate(over="ignore"):
        A = np.multiply.accumulate(np.full(n, a, np.uint32), dtype=np.uint32)  # a^(i+1)
        S = np.concatenate(([np.uint32(1)], A[:-1])).astype(np.uint32)  # a^i
        Csum = np.add.accumulate(S, dtype=np.uint32)                     # sum_{j<=i} a^j
        s = A * s0 + c * Csum
    return ((s >> np.uint32(9)).astype(np.float32) / np.float32(1 << 23)) - np.float32(1.0)


def tvec_first(seeds: np.ndarray) -> np.ndarray:
    """tvec(1, seed)[0] for an array of seeds."""
    s = np.asarray(seeds, np.uint64) & np.uint64(0xFFFFFFFF)
    s = (s * np.uint64(2654435761) + np.uint64(1)) & np.uint64(0xFFFFFFFF)
    s = (s * np.uint64(1664525) + np.uint64(1013904223)) & np.uint64(0xFFFFFFFF)
    return ((s >> np.uint64(9)).astype(np.float32) / np.float32(1 << 23)) - np.float32(1.0)


def q8_rows(rows: int, k: int, seed: int) -> tuple[np.ndarray, np.ndarray]:
    """Row-int8 weights and their per-row scales as the reference's conformance tests make them
    (crates/ojas-cuda/tests/conformance.rs:248-258): w[i] = round(127 tvec(1, seed + i)) (halves away from zero),
    scale[r] = 0.01 + 0.001 |tvec(1, seed ^ (r + 7))|."""
    v = tvec_first((np.arange(rows * k, dtype=np.uint64) + np.uint64(seed)) & np.uint64(0xFFFFFFFF)) * np.float32(127.0)
    w = np.clip(np.sign(v) * np.floor(np.abs(v) + np.float32(0.5)), -127, 127).astype(np.int8).reshape(rows, k)
    t = tvec_first(np.uint64(seed) ^ (np.arange(rows, dtype=np.uint64) + np.uint64(7)))
    scale = (np.float32(0.01) + np.float32(0.001) * np.abs(t)).astype(np.float32)
    return w, scale


def q80_rows_mod5(rows: int, k: int, seed: int) -> tuple[np.ndarray, np.ndarray]:
    """Q8_0 rows of the reference's integer-dot conformance tests and the values a reader decodes them to
    (crates/ojas-cuda/tests/conformance.rs:607-628): block (r, b) has d = f16(0.004 + 0.001 ((r + b) % 5)),
    code i = round(127 tvec(1, seed + r k + 32 b + i)), halves away from zero."""
    nb = k // 32
    r, b = np.divmod(np.arange(rows * nb), nb)
    d = (np.float32(0.004) + np.float32(0.001) * ((r + b) % 5).astype(np.float32)).astype(np.float16)
    t = tvec_first(np.uint64(seed) + np.arange(rows * k, dtype=np.uint64)) * np.float32(127.0)
    q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8).reshape(rows * nb, 32)
    out = np.empty((rows * nb, 34), np.uint8)
    dv = d.view(np.uint16)
    out[:, 0] = dv & 0xFF
    out[:, 1] = dv >> 8
    out[:, 2:] = q.view(np.uint8)
    plain = (q.astype(np.float32) * d.astype(np.float32)[:, None]).reshape(rows, k)
    return out.reshape(-1), plain


def q80_rows_lcg(rows: int, k: int, seed: int) -> tuple[np.ndarray, np.ndarray]:
    """Q8_0 rows of the reference's GPU conformance tests and the values they decode to
    (crates/ojas-cuda/tests/conformance.rs:358-376): block (r, b) has d = f16(0.002 + 0.001 |tvec(1, seed ^ (r nb + b))|),
    code i = round(127 tvec(1, seed + r k + 32 b + i)), halves away from zero."""
    nb = k // 32
    blk = np.arange(rows * nb, dtype=np.uint64)
    d = (np.float32(0.002) + np.float32(0.001) * np.abs(tvec_first(np.uint64(seed) ^ blk))).astype(np.float16)
    t = tvec_first(np.uint64(seed) + np.arange(rows * k, dtype=np.uint64)) * np.float32(127.0)
    q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8).reshape(rows * nb, 32)
    out = np.empty((rows * nb, 34), np.uint8)
    dv = d.view(np.uint16)
    out[:, 0] = dv & 0xFF
    out[:, 1] = dv >> 8
    out[:, 2:] = q.view(np.uint8)
    plain = (q.astype(np.float32) * d.astype(np.float32)[:, None]).reshape(rows, k)
    return out.reshape(-1), plain


def q80_weights_lcg(n: int, k: int, seed: int) -> np.ndarray:
    """Q8_0 rows of crates/ojas-cuda/tests/conformance.rs:611-630: d = f16(0.004 + 0.001 ((r + b) mod 5)), codes as in
    `q80_rows_lcg`."""
    nb = k // 32
    raw, _ = q80_rows_lcg(n, k, seed)
    raw = raw.reshape(n, nb, 34).copy()
    r, b = np.arange(n)[:, None], np.arange(nb)[None, :]
    d = (np.float32(0.004) + np.float32(0.001) * ((r + b) % 5).astype(np.float32)).astype(np.float16).view(np.uint16)
    raw[:, :, 0] = d & 0xFF
    raw[:, :, 1] = d >> 8
    return raw.reshape(-1)


def iq4_rows_lcg(ty: int, rows: int, k: int, seed: int) -> np.ndarray:
    """IQ4_XS / IQ4_NL rows of the reference's GPU conformance test (crates/ojas-cuda/tests/conformance.rs:461-503):
    byte i = trunc(255 |tvec(1, seed + i)|), then d of block (r, b) = f16(0.01 + 0.002 ((r + b) mod 7 | 5))."""
    bb, wpb = BLOCK_SHAPE[ty]
    nb = k // wpb
    out = (np.abs(tvec_first(np.uint64(seed) + np.arange(rows * nb * bb, dtype=np.uint64))) * np.float32(255.0)).astype(np.uint8)
    out = out.reshape(rows, nb, bb)
    r, b = np.arange(rows)[:, None], np.arange(nb)[None, :]
    d = (np.float32(0.01) + np.float32(0.002) * ((r + b) % (7 if ty == IQ4_XS else 5)).astype(np.float32)).astype(np.float16)
    dv = d.view(np.uint16)
    out[:, :, 0] = dv & 0xFF
    out[:, :, 1] = dv >> 8
    return out.reshape(-1)


def q80_rows_closed_form(n: int, k: int):
    """Q8_0 rows and activations of the reference's `native_q8_matvec_ksplit_matches_cpu`:
    d = f16(0.003 + ((r+b) mod 7) * 0.001), q = ((17r + 11b + 5j) mod 31) - 15,
    x_i = ((37 i mod 257) - 128) / 127."""
    nb = k // 32
    r = np.arange(n)[:, None, None]
    b = np.arange(nb)[None, :, None]
    j = np.arange(32)[None, None, :]
    q = (((17 * r + 11 * b + 5 * j) % 31) - 15).astype(np.int8)
    d = (np.float32(0.003) + ((r + b) % 7).astype(np.float32) * np.float32(0.001)).astype(np.float16)
    out = np.empty((n, nb, 34), np.uint8)
    dv = d.view(np.uint16).reshape(n, nb)
    out[:, :, 0] = dv & 0xFF
    out[:, :, 1] = dv >> 8
    out[:, :, 2:] = q.view(np.uint8)
    i = np.arange(k)
    x = (((37 * i) % 257) - 128).astype(np.float32) / np.float32(127.0)
    return out.reshape(-1), x


def q80_rows_table() -> tuple[np.ndarray, np.ndarray]:
    """The 3 x 32 Q8_0 table of crates/ojas-formats/tests/rows.rs:13-18 and its exact values:
    d = 0.25 (r+1), q_j = j - 16 + r."""
    out = np.empty((3, 34), np.uint8)
    want = np.empty((3, 32), np.float32)
    for r in range(3):
        d = np.array([0.25 * (r + 1)], np.float16)
        out[r, 0:2] = d.view(np.uint8)
        q = (np.arange(32) - 16 + r).astype(np.int8)
        out[r, 2:] = q.view(np.uint8)
        want[r] = np.float32(d[0]) * q.astype(np.float32)
    return out.reshape(-1), want

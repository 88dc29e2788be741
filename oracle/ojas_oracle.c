/*
 * TEST INFRASTRUCTURE — CPU restatement of the reference's quantized-matmul arithmetic.
 * See ojas_oracle.h for what this is, who may use it and how each function is pinned.
 * Paths in comments are relative to the reference tree.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (the reference is Rust: one IEEE rounding per
 * operator, no fused multiply-add).
 */
#include "ojas_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdatomic.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- f16 / bf16 */

/* IEEE binary16 -> binary32 (crate half 2.7.1, f16::to_f32; used at gguf.rs:606-608). */
float ojo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (half::f16::from_f32; gguf.rs:602-604). */
uint16_t ojo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 0xFF) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7C00u | 0x200u | (man >> 13));
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return sign; /* below half the smallest subnormal */
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t hm = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm); /* a carry into bit 10 is the smallest normal: correct */
    }
    uint32_t hm = man >> 13;
    uint32_t rem = man & 0x1FFFu;
    uint16_t out = (uint16_t)(sign | ((uint32_t)e << 10) | hm);
    if (rem > 0x1000u || (rem == 0x1000u && (hm & 1u))) out++; /* carry may roll into exp / inf */
    return out;
}

uint16_t ojo_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7F800000u) == 0x7F800000u && (x & 0x7FFFFFu)) return (uint16_t)((x >> 16) | 0x40u);
    uint32_t lsb = (x >> 16) & 1u;
    x += 0x7FFFu + lsb;
    return (uint16_t)(x >> 16);
}

float ojo_bf16_to_f32(uint16_t h) {
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

static inline float rdh(const uint8_t *b, size_t i) { /* gguf.rs:606-608 */
    return ojo_f16_to_f32((uint16_t)(b[i] | (b[i + 1] << 8)));
}

/* ---------------------------------------------------------------- block shapes, synth */

int ojo_block_shape(uint32_t ty, uint32_t *bytes, uint32_t *weights) { /* synth.rs:12-21 */
    uint32_t b, w;
    switch (ty) {
    case OJO_Q8_0: b = 34; w = 32; break;
    case OJO_Q2_K: b = 84; w = 256; break;
    case OJO_Q3_K: b = 110; w = 256; break;
    case OJO_Q4_K: b = 144; w = 256; break;
    case OJO_Q5_K: b = 176; w = 256; break;
    case OJO_Q6_K: b = 210; w = 256; break;
    case OJO_IQ4_NL: b = 18; w = 32; break;
    case OJO_Q4_0: b = 18; w = 32; break;
    case OJO_Q4_1: b = 20; w = 32; break;
    case OJO_Q5_0: b = 22; w = 32; break;
    case OJO_Q5_1: b = 24; w = 32; break;
    case OJO_IQ4_XS: b = 136; w = 256; break;
    case OJO_MXFP4: b = 17; w = 32; break;
    case OJO_IQ2_XXS: b = 66; w = 256; break;
    case OJO_IQ2_XS: b = 74; w = 256; break;
    case OJO_IQ3_XXS: b = 98; w = 256; break;
    case OJO_IQ1_S: b = 50; w = 256; break;
    case OJO_IQ3_S: b = 110; w = 256; break;
    case OJO_IQ2_S: b = 82; w = 256; break;
    case OJO_IQ1_M: b = 56; w = 256; break;
    default: return 0;
    }
    if (bytes) *bytes = b;
    if (weights) *weights = w;
    return 1;
}

int ojo_synth_blocks(uint32_t ty, size_t nb, uint8_t *out) { /* synth.rs:29-64 */
    uint32_t bb;
    if (!ojo_block_shape(ty, &bb, NULL)) return -1;
    uint64_t st = 0x2545F4914F6CDD1DULL;
    for (size_t i = 0; i < nb * bb; i++) {
        st ^= st << 13; st ^= st >> 7; st ^= st << 17;
        out[i] = (uint8_t)(st >> 24);
    }
    for (size_t i = 0; i < nb; i++) {
        uint8_t *blk = out + i * bb;
        uint16_t d = ojo_f32_to_f16(0.05f + (float)(i % 7) * 0.01f);
        uint16_t dmin = ojo_f32_to_f16(0.01f);
        switch (ty) {
        case OJO_Q4_K: case OJO_Q5_K:
            blk[0] = (uint8_t)d; blk[1] = (uint8_t)(d >> 8);
            blk[2] = (uint8_t)dmin; blk[3] = (uint8_t)(dmin >> 8);
            break;
        case OJO_Q6_K:
            blk[208] = (uint8_t)d; blk[209] = (uint8_t)(d >> 8);
            break;
        case OJO_Q2_K: /* d and dmin close the block */
            blk[80] = (uint8_t)d; blk[81] = (uint8_t)(d >> 8);
            blk[82] = (uint8_t)dmin; blk[83] = (uint8_t)(dmin >> 8);
            break;
        case OJO_Q3_K:
            blk[108] = (uint8_t)d; blk[109] = (uint8_t)(d >> 8);
            break;
        case OJO_MXFP4: /* not a synth.rs type: an e8m0 exponent near 1.0 in byte 0 keeps the values finite */
            blk[0] = (uint8_t)(120 + i % 7);
            break;
        case OJO_IQ1_M: { /* no d field: f16(0.05) spread over the top nibbles of the four scale words, low nibble first */
            uint16_t db = ojo_f32_to_f16(0.05f);
            for (int w = 0; w < 4; w++) {
                uint16_t cur = (uint16_t)(blk[48 + 2 * w] | (blk[49 + 2 * w] << 8));
                uint16_t v = (uint16_t)((cur & 0x0FFF) | (((db >> (4 * w)) & 0xF) << 12));
                blk[48 + 2 * w] = (uint8_t)v; blk[49 + 2 * w] = (uint8_t)(v >> 8);
            }
        } break;
        default:
            blk[0] = (uint8_t)d; blk[1] = (uint8_t)(d >> 8);
        }
    }
    return 0;
}

/* ---------------------------------------------------------------- dequant */

/* The 16 levels of the IQ4 codebook (crates/ojas-core/src/iq_tables.rs:881-884). */
static const int8_t kvalues_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

/* get_scale_min_k4 (gguf.rs:1132-1140; twin cpu_math.rs:566-574). */
static inline void scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* Sixteen 6-bit scales of a Q3_K block from its 12 packed bytes (gguf.rs:764-774): scale i has its low
 * nibble in byte i (i < 8) or in the high nibble of byte i - 8, and its two high bits in byte 8 + i % 4
 * at bit 2 (i / 4).  Stored biased by 32. */
static inline int q3k_scale(const uint8_t *raw, int i) {
    int lo = i < 8 ? raw[i] & 0xF : raw[i - 8] >> 4;
    int hi = (raw[8 + (i & 3)] >> (2 * (i >> 2))) & 3;
    return (int)(int8_t)(lo | (hi << 4)) - 32;
}

int ojo_dequant_to_f16(const uint8_t *b, uint32_t ty, size_t n, uint16_t *out) {
    uint32_t bb, wpb;
    if (!ojo_block_shape(ty, &bb, &wpb) || n % wpb) return -1;
    size_t nblk = n / wpb;
    if (ojo_iq_is_grid_type(ty)) { /* gguf.rs:840-1041 */
        float w32[256];
        for (size_t ib = 0; ib < nblk; ib++) {
            ojo_iq_block(ty, b + ib * bb, w32, NULL);
            for (int j = 0; j < 256; j++) out[ib * 256 + j] = ojo_f32_to_f16(w32[j]);
        }
        return 0;
    }
    for (size_t ib = 0; ib < nblk; ib++) {
        const uint8_t *blk = b + ib * bb;
        uint16_t *o = out + ib * wpb;
        switch (ty) {
        case OJO_MXFP4: { /* crates/ojas-formats/src/mxfp4.rs:40-58: weight 2j = low nibble of qs[j], 2j+1 = high; d = 2^(e-127) */
            static const float lut[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f, -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};
            union { uint32_t u; float f; } d = { (uint32_t)blk[0] << 23 };
            for (int j = 0; j < 16; j++) {
                o[2 * j] = ojo_f32_to_f16(d.f * lut[blk[1 + j] & 0xF]);
                o[2 * j + 1] = ojo_f32_to_f16(d.f * lut[blk[1 + j] >> 4]);
            }
        } break;
        case OJO_Q8_0: { /* gguf.rs:704-709 */
            float d = rdh(blk, 0);
            for (int j = 0; j < 32; j++) o[j] = ojo_f32_to_f16(d * (float)(int8_t)blk[2 + j]);
        } break;
        case OJO_Q2_K: { /* gguf.rs:730-754: scales[16], qs[64], d, dmin; w = (d * sc) * q - dmin * m */
            const uint8_t *sc = blk, *qs = blk + 16;
            float d = rdh(blk, 80), dmin = rdh(blk, 82);
            int is = 0;
            for (int half = 0; half < 2; half++)
                for (int j = 0; j < 4; j++)
                    for (int part = 0; part < 2; part++, is++) {
                        float dl = d * (float)(sc[is] & 0xF), ml = dmin * (float)(sc[is] >> 4);
                        for (int l = 0; l < 16; l++) {
                            int q = (qs[half * 32 + part * 16 + l] >> (2 * j)) & 3;
                            o[half * 128 + j * 32 + part * 16 + l] = ojo_f32_to_f16(dl * (float)q - ml);
                        }
                    }
        } break;
        case OJO_Q3_K: { /* gguf.rs:755-795: hmask[32], qs[64], scales[12], d; a clear mask bit subtracts 4 */
            const uint8_t *hm = blk, *qs = blk + 32, *raw = blk + 96;
            float d = rdh(blk, 108);
            int is = 0;
            for (int half = 0; half < 2; half++)
                for (int j = 0; j < 4; j++)
                    for (int part = 0; part < 2; part++, is++) {
                        float dl = d * (float)q3k_scale(raw, is);
                        for (int l = 0; l < 16; l++) {
                            int q = (qs[half * 32 + part * 16 + l] >> (2 * j)) & 3;
                            int hi = (hm[part * 16 + l] >> (half * 4 + j)) & 1 ? 0 : 4;
                            o[half * 128 + j * 32 + part * 16 + l] = ojo_f32_to_f16(dl * (float)(q - hi));
                        }
                    }
        } break;
        case OJO_Q4_0: { /* gguf.rs:653-661: w = d * (nib - 8); low nibbles first, then high nibbles */
            float d = rdh(blk, 0);
            for (int j = 0; j < 16; j++) {
                o[j] = ojo_f32_to_f16(d * ((float)(blk[2 + j] & 0xF) - 8.0f));
                o[j + 16] = ojo_f32_to_f16(d * ((float)(blk[2 + j] >> 4) - 8.0f));
            }
        } break;
        case OJO_Q5_0: { /* gguf.rs:662-678: fifth bit of weight j is bit j of qh; w = d * (q - 16) */
            float d = rdh(blk, 0);
            uint32_t qh = (uint32_t)blk[2] | ((uint32_t)blk[3] << 8) | ((uint32_t)blk[4] << 16) | ((uint32_t)blk[5] << 24);
            for (int j = 0; j < 16; j++) {
                uint32_t lo = (uint32_t)(blk[6 + j] & 0xF) | (((qh >> j) & 1u) << 4);
                uint32_t hi = (uint32_t)(blk[6 + j] >> 4) | (((qh >> (j + 16)) & 1u) << 4);
                o[j] = ojo_f32_to_f16(d * ((float)lo - 16.0f));
                o[j + 16] = ojo_f32_to_f16(d * ((float)hi - 16.0f));
            }
        } break;
        case OJO_Q4_1: { /* gguf.rs:679-686: w = d * nib + m, a product and a sum, each rounded */
            float d = rdh(blk, 0), m = rdh(blk, 2);
            for (int j = 0; j < 16; j++) {
                o[j] = ojo_f32_to_f16(d * (float)(blk[4 + j] & 0xF) + m);
                o[j + 16] = ojo_f32_to_f16(d * (float)(blk[4 + j] >> 4) + m);
            }
        } break;
        case OJO_Q5_1: { /* gguf.rs:687-703 (and the threaded copy :616-649): w = d * q + m */
            float d = rdh(blk, 0), m = rdh(blk, 2);
            uint32_t qh = (uint32_t)blk[4] | ((uint32_t)blk[5] << 8) | ((uint32_t)blk[6] << 16) | ((uint32_t)blk[7] << 24);
            for (int j = 0; j < 16; j++) {
                uint32_t lo = (uint32_t)(blk[8 + j] & 0xF) | (((qh >> j) & 1u) << 4);
                uint32_t hi = (uint32_t)(blk[8 + j] >> 4) | (((qh >> (j + 16)) & 1u) << 4);
                o[j] = ojo_f32_to_f16(d * (float)lo + m);
                o[j + 16] = ojo_f32_to_f16(d * (float)hi + m);
            }
        } break;
        case OJO_IQ4_NL: { /* gguf.rs:796-813: low nibbles fill the first half, high nibbles the second */
            float d = rdh(blk, 0);
            const uint8_t *qs = blk + 2;
            for (int j = 0; j < 16; j++) {
                o[j] = ojo_f32_to_f16(d * (float)kvalues_iq4nl[qs[j] & 0xF]);
                o[j + 16] = ojo_f32_to_f16(d * (float)kvalues_iq4nl[qs[j] >> 4]);
            }
        } break;
        case OJO_IQ4_XS: { /* gguf.rs:814-840 */
            float d = rdh(blk, 0);
            uint16_t sh = (uint16_t)(blk[2] | (blk[3] << 8));
            const uint8_t *sl = blk + 4, *qs = blk + 8;
            for (int ib = 0; ib < 8; ib++) {
                uint32_t ls = (uint32_t)((sl[ib / 2] >> (4 * (ib % 2))) & 0xF) | ((uint32_t)((sh >> (2 * ib)) & 3) << 4);
                float dl = d * (float)((int32_t)ls - 32);
                const uint8_t *q = qs + ib * 16;
                for (int j = 0; j < 16; j++) {
                    o[ib * 32 + j] = ojo_f32_to_f16(dl * (float)kvalues_iq4nl[q[j] & 0xF]);
                    o[ib * 32 + j + 16] = ojo_f32_to_f16(dl * (float)kvalues_iq4nl[q[j] >> 4]);
                }
            }
        } break;
        case OJO_Q4_K: { /* gguf.rs:1042-1059 */
            float d = rdh(blk, 0), dmin = rdh(blk, 2);
            const uint8_t *sc = blk + 4, *qs = blk + 16;
            for (int chunk = 0; chunk < 4; chunk++) {
                uint8_t s1, m1, s2, m2;
                scale_min_k4(chunk * 2, sc, &s1, &m1);
                scale_min_k4(chunk * 2 + 1, sc, &s2, &m2);
                float dl1 = d * (float)s1, ml1 = dmin * (float)m1;
                float dl2 = d * (float)s2, ml2 = dmin * (float)m2;
                const uint8_t *q = qs + chunk * 32;
                for (int l = 0; l < 32; l++) *o++ = ojo_f32_to_f16(dl1 * (float)(q[l] & 0xF) - ml1);
                for (int l = 0; l < 32; l++) *o++ = ojo_f32_to_f16(dl2 * (float)(q[l] >> 4) - ml2);
            }
        } break;
        case OJO_Q5_K: { /* gguf.rs:1060-1085 */
            float d = rdh(blk, 0), dmin = rdh(blk, 2);
            const uint8_t *sc = blk + 4, *qh = blk + 16, *qs = blk + 48;
            uint8_t u1 = 1, u2 = 2;
            for (int chunk = 0; chunk < 4; chunk++) {
                uint8_t s1, m1, s2, m2;
                scale_min_k4(chunk * 2, sc, &s1, &m1);
                scale_min_k4(chunk * 2 + 1, sc, &s2, &m2);
                float dl1 = d * (float)s1, ml1 = dmin * (float)m1;
                float dl2 = d * (float)s2, ml2 = dmin * (float)m2;
                const uint8_t *ql = qs + chunk * 32;
                for (int l = 0; l < 32; l++) {
                    float hi = (qh[l] & u1) ? 16.0f : 0.0f;
                    *o++ = ojo_f32_to_f16(dl1 * ((float)(ql[l] & 0xF) + hi) - ml1);
                }
                for (int l = 0; l < 32; l++) {
                    float hi = (qh[l] & u2) ? 16.0f : 0.0f;
                    *o++ = ojo_f32_to_f16(dl2 * ((float)(ql[l] >> 4) + hi) - ml2);
                }
                u1 = (uint8_t)(u1 << 2); u2 = (uint8_t)(u2 << 2);
            }
        } break;
        case OJO_Q6_K: { /* gguf.rs:1086-1108 */
            float d = rdh(blk, 208);
            float y[128];
            for (int hf = 0; hf < 2; hf++) {
                const uint8_t *ql = blk + hf * 64, *qh = blk + 128 + hf * 32;
                const int8_t *sc = (const int8_t *)(blk + 192 + hf * 8);
                for (int l = 0; l < 32; l++) {
                    int is = l / 16;
                    int q1 = ((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    int q2 = ((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    int q3 = ((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    int q4 = ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    /* `d * sc as f32 * q as f32` is left-associative: (d*sc)*q */
                    y[l]      = d * (float)sc[is]     * (float)q1;
                    y[l + 32] = d * (float)sc[is + 2] * (float)q2;
                    y[l + 64] = d * (float)sc[is + 4] * (float)q3;
                    y[l + 96] = d * (float)sc[is + 6] * (float)q4;
                }
                for (int l = 0; l < 128; l++) *o++ = ojo_f32_to_f16(y[l]);
            }
        } break;
        }
    }
    return 0;
}

int ojo_dequant_to_f64(const uint8_t *b, uint32_t ty, size_t n, double *out) {
    /* Same decoders, exact in double: f16 scale x 6-bit x 6-bit products fit a double
     * (crates/ojas-models/examples/q6k_gate.rs:60-110 derives its oracle the same way). */
    uint32_t bb, wpb;
    if (!ojo_block_shape(ty, &bb, &wpb) || n % wpb) return -1;
    size_t nblk = n / wpb;
    if (ojo_iq_is_grid_type(ty)) {
        for (size_t ib = 0; ib < nblk; ib++) ojo_iq_block(ty, b + ib * bb, NULL, out + ib * 256);
        return 0;
    }
    for (size_t ib = 0; ib < nblk; ib++) {
        const uint8_t *blk = b + ib * bb;
        double *o = out + ib * wpb;
        switch (ty) {
        case OJO_MXFP4: {
            static const double lut[16] = {0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0};
            union { uint32_t u; float f; } d = { (uint32_t)blk[0] << 23 };
            for (int j = 0; j < 16; j++) {
                o[2 * j] = (double)d.f * lut[blk[1 + j] & 0xF];
                o[2 * j + 1] = (double)d.f * lut[blk[1 + j] >> 4];
            }
        } break;
        case OJO_Q8_0: {
            double d = rdh(blk, 0);
            for (int j = 0; j < 32; j++) o[j] = d * (double)(int8_t)blk[2 + j];
        } break;
        case OJO_Q2_K: {
            double d = rdh(blk, 80), dmin = rdh(blk, 82);
            for (int i = 0; i < 256; i++) {
                int half = i >> 7, j = (i >> 5) & 3, l = i & 31, is = half * 8 + j * 2 + (l >> 4);
                int q = (blk[16 + half * 32 + l] >> (2 * j)) & 3;
                o[i] = d * (double)(blk[is] & 0xF) * (double)q - dmin * (double)(blk[is] >> 4);
            }
        } break;
        case OJO_Q3_K: {
            double d = rdh(blk, 108);
            for (int i = 0; i < 256; i++) {
                int half = i >> 7, j = (i >> 5) & 3, l = i & 31, is = half * 8 + j * 2 + (l >> 4);
                int q = (blk[32 + half * 32 + l] >> (2 * j)) & 3;
                int hi = (blk[l] >> (half * 4 + j)) & 1 ? 0 : 4;
                o[i] = d * (double)q3k_scale(blk + 96, is) * (double)(q - hi);
            }
        } break;
        case OJO_Q4_0: case OJO_Q4_1: case OJO_Q5_0: case OJO_Q5_1: {
            const int five = ty == OJO_Q5_0 || ty == OJO_Q5_1, affine = ty == OJO_Q4_1 || ty == OJO_Q5_1;
            double d = rdh(blk, 0), m = affine ? (double)rdh(blk, 2) : 0.0;
            const uint8_t *hb = blk + (affine ? 4 : 2), *qs = hb + (five ? 4 : 0);
            uint32_t qh = five ? (uint32_t)hb[0] | ((uint32_t)hb[1] << 8) | ((uint32_t)hb[2] << 16) | ((uint32_t)hb[3] << 24) : 0;
            double off = affine ? 0.0 : (five ? 16.0 : 8.0);
            for (int j = 0; j < 16; j++) {
                uint32_t lo = (uint32_t)(qs[j] & 0xF) | (((qh >> j) & 1u) << 4);
                uint32_t hi = (uint32_t)(qs[j] >> 4) | (((qh >> (j + 16)) & 1u) << 4);
                o[j] = d * ((double)lo - off) + m;
                o[j + 16] = d * ((double)hi - off) + m;
            }
        } break;
        case OJO_IQ4_NL: {
            double d = rdh(blk, 0);
            for (int j = 0; j < 16; j++) {
                o[j] = d * (double)kvalues_iq4nl[blk[2 + j] & 0xF];
                o[j + 16] = d * (double)kvalues_iq4nl[blk[2 + j] >> 4];
            }
        } break;
        case OJO_IQ4_XS: {
            double d = rdh(blk, 0);
            uint16_t sh = (uint16_t)(blk[2] | (blk[3] << 8));
            for (int ib = 0; ib < 8; ib++) {
                int ls = ((blk[4 + ib / 2] >> (4 * (ib % 2))) & 0xF) | (((sh >> (2 * ib)) & 3) << 4);
                double dl = d * (double)(ls - 32);
                for (int j = 0; j < 16; j++) {
                    o[ib * 32 + j] = dl * (double)kvalues_iq4nl[blk[8 + ib * 16 + j] & 0xF];
                    o[ib * 32 + j + 16] = dl * (double)kvalues_iq4nl[blk[8 + ib * 16 + j] >> 4];
                }
            }
        } break;
        case OJO_Q4_K: case OJO_Q5_K: {
            double d = rdh(blk, 0), dmin = rdh(blk, 2);
            const uint8_t *sc = blk + 4;
            const uint8_t *qh = ty == OJO_Q5_K ? blk + 16 : NULL;
            const uint8_t *qs = ty == OJO_Q5_K ? blk + 48 : blk + 16;
            for (int chunk = 0; chunk < 4; chunk++) {
                uint8_t s1, m1, s2, m2;
                scale_min_k4(chunk * 2, sc, &s1, &m1);
                scale_min_k4(chunk * 2 + 1, sc, &s2, &m2);
                const uint8_t *q = qs + chunk * 32;
                for (int l = 0; l < 32; l++) {
                    int v = (q[l] & 0xF) + ((qh && (qh[l] & (1 << (2 * chunk)))) ? 16 : 0);
                    *o++ = d * s1 * v - dmin * m1;
                }
                for (int l = 0; l < 32; l++) {
                    int v = (q[l] >> 4) + ((qh && (qh[l] & (2 << (2 * chunk)))) ? 16 : 0);
                    *o++ = d * s2 * v - dmin * m2;
                }
            }
        } break;
        case OJO_Q6_K: {
            double d = rdh(blk, 208);
            for (int hf = 0; hf < 2; hf++) {
                const uint8_t *ql = blk + hf * 64, *qh = blk + 128 + hf * 32;
                const int8_t *sc = (const int8_t *)(blk + 192 + hf * 8);
                for (int l = 0; l < 32; l++) {
                    int is = l / 16;
                    int q1 = ((ql[l] & 0xF) | (((qh[l] >> 0) & 3) << 4)) - 32;
                    int q2 = ((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32;
                    int q3 = ((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                    int q4 = ((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                    o[l]      = d * sc[is]     * q1;
                    o[l + 32] = d * sc[is + 2] * q2;
                    o[l + 64] = d * sc[is + 4] * q3;
                    o[l + 96] = d * sc[is + 6] * q4;
                }
                o += 128;
            }
        } break;
        }
    }
    return 0;
}

uint64_t ojo_digest_f16(const uint16_t *v, size_t n) { /* quant_formats.rs:20-31 */
    uint64_t h = 0xcbf29ce484222325ULL;
    char buf[64];
    for (size_t i = 0; i < n; i++) {
        int len = snprintf(buf, sizeof buf, "%.6f", (double)ojo_f16_to_f32(v[i]));
        for (int c = 0; c < len; c++) {
            h ^= (uint8_t)buf[c];
            h *= 0x00000100000001B3ULL;
        }
    }
    return h;
}

/* ---------------------------------------------------------------- activations */

static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }
/* `x.round().clamp(-127.0, 127.0) as i8`: clamp passes a NaN through and Rust's float-to-int cast maps NaN to 0
 * (in C that cast is undefined, so the case is spelled out). */
static inline int8_t sat_i8(float r) { return r != r ? (int8_t)0 : (int8_t)clampf(r, -127.0f, 127.0f); }

void ojo_quant_q8k(const float *x, size_t k, float *scales, int8_t *q, int32_t *bsums) {
    /* cpu_math.rs:545-563. f32::round is round-half-away-from-zero == roundf. */
    size_t nsb = (k + 255) / 256;
    memset(q, 0, nsb * 256);
    memset(bsums, 0, nsb * 8 * sizeof(int32_t));
    for (size_t sb = 0; sb < nsb; sb++) {
        size_t lo = sb * 256, hi = lo + 256 < k ? lo + 256 : k;
        float m = 0.0f;
        for (size_t i = lo; i < hi; i++) { float a = fabsf(x[i]); if (a > m) m = a; }
        float scale = m > 0.0f ? m / 127.0f : 1.0f;
        float inv = 1.0f / scale;
        scales[sb] = scale;
        for (size_t i = lo; i < hi; i++) {
            int8_t qi = sat_i8(roundf(x[i] * inv));
            q[i] = qi;
            bsums[sb * 8 + (i - lo) / 32] += qi;
        }
    }
}

float ojo_quant_row_i8(const float *row, size_t k, int8_t *q) { /* cpu_math.rs:174-179 */
    float m = 0.0f;
    for (size_t i = 0; i < k; i++) { float a = fabsf(row[i]); if (a > m) m = a; }
    float scale = m > 0.0f ? m / 127.0f : 1.0f;
    float inv = 1.0f / scale;
    for (size_t i = 0; i < k; i++) q[i] = sat_i8(roundf(row[i] * inv));
    return scale;
}

/* The reference GPU decode path's activation quantizer (crates/ojas-cuda/src/kernels/gemv.rs:33-52): per block of 32,
 * d8 = amax / 127, id = d8 > 0 ? 1 / d8 : 0, q = clamp(round-to-nearest-even(x * id), -127, 127), d8sum = d8 * sum q. */
void ojo_quantize_q8_1(const float *x, size_t k, int8_t *q8, float *d8, float *d8sum) {
    for (size_t b = 0; b < k / 32; b++) {
        const float *xb = x + b * 32;
        float a = 0.0f;
        for (int i = 0; i < 32; i++) a = fmaxf(a, fabsf(xb[i]));
        float d = a / 127.0f, id = d > 0.0f ? 1.0f / d : 0.0f, s = 0.0f;
        for (int i = 0; i < 32; i++) {
            float r = rintf(xb[i] * id);
            int qi = r != r ? 0 : r > 127.0f ? 127 : r < -127.0f ? -127 : (int)r;
            q8[b * 32 + i] = (int8_t)qi;
            s += (float)qi;
        }
        d8[b] = d;
        d8sum[b] = d * s;
    }
}
/* The reference GPU decoder's row-int8 matvec (crates/ojas-cuda/src/kernels/gemv_q8.rs:31-55): K plain int8 per row and
 * one f32 scale per row against f32 activations, y[n] = scale[n] * sum_k (float) w[n][k] * x[k].  The GPU adds a lane's
 * terms and then the lanes in an order of its own; here the terms (exact in a double) meet in a double and the row scale
 * is applied in f32, as the reference's test oracle does after its own f32 sum (crates/ojas-cuda/tests/conformance.rs:259-268). */
void ojo_gemv_q8_rows(const int8_t *w, const float *scale, const float *x, size_t k, size_t n, float *y) {
    for (size_t r = 0; r < n; r++) {
        double acc = 0.0;
        for (size_t i = 0; i < k; i++) acc += (double)w[r * k + i] * (double)x[i];
        y[r] = (float)acc * scale[r];
    }
}
/* Per-token activation quantizer of the reference's batched int8 GEMM (crates/ojas-cuda/src/kernels/gemv.rs:57-74):
 * d = amax / 127, id = d > 0 ? 1 / d : 0, q = clamp(round-to-nearest-even(x * id), -127, 127); d8[token] = d. */
void ojo_quantize_q8_pertoken(const float *x, size_t m, size_t k, int8_t *q8, float *d8) {
    for (size_t t = 0; t < m; t++) {
        const float *xr = x + t * k;
        float a = 0.0f;
        for (size_t i = 0; i < k; i++) a = fmaxf(a, fabsf(xr[i]));
        float d = a / 127.0f, id = d > 0.0f ? 1.0f / d : 0.0f;
        for (size_t i = 0; i < k; i++) {
            float r = rintf(xr[i] * id);
            int qi = r != r ? 0 : r > 127.0f ? 127 : r < -127.0f ? -127 : (int)r;
            q8[t * k + i] = (int8_t)qi;
        }
        d8[t] = d;
    }
}
/* One block_q8_0 row against q8_1 activations (crates/ojas-cuda/src/kernels/gemv_q8.rs:178-193): a lane's term is
 * dw * d8[b] * (float) idot over its 8 weights; the GPU adds the terms in a lane and then across lanes in an order of its
 * own, here they meet in a double (the kernels are compared to a tolerance of a few f32 roundings). */
double ojo_row_q80_dp4a(const uint8_t *row, const int8_t *q8, const float *d8, size_t k) {
    double sum = 0.0;
    for (size_t b = 0; b < k / 32; b++) {
        const uint8_t *blk = row + b * 34;
        float dw = rdh(blk, 0);
        for (int sub = 0; sub < 4; sub++) {
            int32_t si = 0;
            for (int i = 0; i < 8; i++) si += (int32_t)(int8_t)blk[2 + sub * 8 + i] * (int32_t)q8[b * 32 + sub * 8 + i];
            sum += (double)(dw * d8[b] * (float)si);
        }
    }
    return sum;
}
void ojo_gemv_q80_dp4a(const uint8_t *w, const int8_t *q8, const float *d8, size_t k, size_t n, float *y) {
    for (size_t r = 0; r < n; r++) y[r] = (float)ojo_row_q80_dp4a(w + r * (k / 32) * 34, q8, d8, k);
}

/* ---------------------------------------------------------------- row dots */

float ojo_dot_q80(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:971-981 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 32; b++) {
        const uint8_t *blk = row + b * 34;
        const float *xb = x + b * 32;
        float d = rdh(blk, 0);
        float acc = 0.0f;
        for (int j = 0; j < 32; j++) acc += (float)(int8_t)blk[2 + j] * xb[j];
        sum += d * acc;
    }
    return sum;
}

float ojo_dot_iq4nl(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:993-1010 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 32; b++) {
        const uint8_t *blk = row + b * 18;
        const float *xb = x + b * 32;
        float d = rdh(blk, 0);
        float bsum = 0.0f;
        for (int j = 0; j < 16; j++) {
            uint8_t q = blk[2 + j];
            bsum += (float)kvalues_iq4nl[q & 0xF] * xb[j];
            bsum += (float)kvalues_iq4nl[q >> 4] * xb[j + 16];
        }
        sum += d * bsum;
    }
    return sum;
}

float ojo_dot_iq4xs(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:943-967 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 256; b++) {
        const uint8_t *blk = row + b * 136;
        const float *xb = x + b * 256;
        float d = rdh(blk, 0);
        uint16_t sh = (uint16_t)(blk[2] | (blk[3] << 8));
        const uint8_t *sl = blk + 4, *qs = blk + 8;
        float bsum = 0.0f;
        for (int g = 0; g < 8; g++) {
            int32_t ls = (int32_t)((sl[g / 2] >> (4 * (g % 2))) & 0xF) | ((int32_t)((sh >> (2 * g)) & 3) << 4);
            const float *xg = xb + g * 32;
            float gsum = 0.0f;
            for (int j = 0; j < 16; j++) {
                uint8_t q = qs[16 * g + j];
                gsum += (float)kvalues_iq4nl[q & 0xF] * xg[j];
                gsum += (float)kvalues_iq4nl[q >> 4] * xg[j + 16];
            }
            bsum += (float)(ls - 32) * gsum;
        }
        sum += d * bsum;
    }
    return sum;
}

static inline int32_t idot32(const uint8_t *w, const int8_t *x) { /* cpu_math.rs:583-593 */
    int32_t s = 0;
    for (int i = 0; i < 32; i++) s += (int32_t)w[i] * (int32_t)x[i];
    return s;
}

float ojo_dot_q4k(const uint8_t *row, size_t k, const float *scales, const int8_t *q,
                  const int32_t *bsums) { /* cpu_math.rs:609-635 */
    float total = 0.0f;
    for (size_t sb = 0; sb < k / 256; sb++) {
        const uint8_t *blk = row + sb * 144;
        float d = rdh(blk, 0), dmin = rdh(blk, 2);
        const uint8_t *sc = blk + 4, *qs = blk + 16;
        float sx = scales[sb];
        const int8_t *xq = q + sb * 256;
        const int32_t *bs = bsums + sb * 8;
        float sumd = 0.0f, summ = 0.0f;
        uint8_t lo[32], hi[32];
        for (int c = 0; c < 4; c++) {
            const uint8_t *qq = qs + c * 32;
            for (int l = 0; l < 32; l++) { lo[l] = qq[l] & 0xF; hi[l] = qq[l] >> 4; }
            uint8_t s1, m1, s2, m2;
            scale_min_k4(c * 2, sc, &s1, &m1);
            scale_min_k4(c * 2 + 1, sc, &s2, &m2);
            sumd += (float)s1 * (float)idot32(lo, xq + c * 64);
            sumd += (float)s2 * (float)idot32(hi, xq + c * 64 + 32);
            summ += (float)m1 * (float)bs[c * 2] + (float)m2 * (float)bs[c * 2 + 1];
        }
        total += sx * (d * sumd - dmin * summ);
    }
    return total;
}

float ojo_dot_q5k(const uint8_t *row, size_t k, const float *scales, const int8_t *q,
                  const int32_t *bsums) { /* cpu_math.rs:638-670 */
    float total = 0.0f;
    for (size_t sb = 0; sb < k / 256; sb++) {
        const uint8_t *blk = row + sb * 176;
        float d = rdh(blk, 0), dmin = rdh(blk, 2);
        const uint8_t *sc = blk + 4, *qh = blk + 16, *qs = blk + 48;
        float sx = scales[sb];
        const int8_t *xq = q + sb * 256;
        const int32_t *bs = bsums + sb * 8;
        float sumd = 0.0f, summ = 0.0f;
        uint8_t lo[32], hi[32];
        uint8_t u1 = 1, u2 = 2;
        for (int c = 0; c < 4; c++) {
            const uint8_t *qq = qs + c * 32;
            for (int l = 0; l < 32; l++) {
                lo[l] = (uint8_t)((qq[l] & 0xF) | ((qh[l] & u1) ? 16 : 0));
                hi[l] = (uint8_t)((qq[l] >> 4) | ((qh[l] & u2) ? 16 : 0));
            }
            uint8_t s1, m1, s2, m2;
            scale_min_k4(c * 2, sc, &s1, &m1);
            scale_min_k4(c * 2 + 1, sc, &s2, &m2);
            sumd += (float)s1 * (float)idot32(lo, xq + c * 64);
            sumd += (float)s2 * (float)idot32(hi, xq + c * 64 + 32);
            summ += (float)m1 * (float)bs[c * 2] + (float)m2 * (float)bs[c * 2 + 1];
            u1 = (uint8_t)(u1 << 2); u2 = (uint8_t)(u2 << 2);
        }
        total += sx * (d * sumd - dmin * summ);
    }
    return total;
}

float ojo_dot_q6k(const uint8_t *row, size_t k, const float *scales, const int8_t *q,
                  const int32_t *bsums) { /* cpu_math.rs:674-722 */
    (void)bsums;
    float total = 0.0f;
    uint8_t w[32];
    for (size_t sb = 0; sb < k / 256; sb++) {
        const uint8_t *blk = row + sb * 210;
        float d = rdh(blk, 208);
        float sx = scales[sb];
        const int8_t *xq = q + sb * 256;
        float sum = 0.0f, sub = 0.0f;
        for (int hf = 0; hf < 2; hf++) {
            const uint8_t *ql = blk + hf * 64, *qh = blk + 128 + hf * 32;
            const int8_t *sc = (const int8_t *)(blk + 192 + hf * 8);
            const int8_t *xh = xq + hf * 128;
            for (int quarter = 0; quarter < 4; quarter++) {
                for (int l = 0; l < 32; l++) {
                    switch (quarter) {
                    case 0: w[l] = (uint8_t)((ql[l] & 0xF) | ((qh[l] & 3) << 4)); break;
                    case 1: w[l] = (uint8_t)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)); break;
                    case 2: w[l] = (uint8_t)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)); break;
                    default: w[l] = (uint8_t)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4));
                    }
                }
                const int8_t *x32 = xh + quarter * 32;
                float s0 = (float)sc[quarter * 2], s1 = (float)sc[quarter * 2 + 1];
                int32_t i0 = 0, i1 = 0, x0 = 0, x1 = 0;
                for (int l = 0; l < 16; l++) {
                    i0 += (int32_t)w[l] * x32[l];
                    x0 += x32[l];
                    i1 += (int32_t)w[l + 16] * x32[l + 16];
                    x1 += x32[l + 16];
                }
                sum += s0 * (float)i0 + s1 * (float)i1;
                sub += s0 * (float)x0 + s1 * (float)x1;
            }
        }
        total += sx * d * (sum - 32.0f * sub);
    }
    return total;
}

/* ---------------------------------------------------------------- workers */

typedef void (*row_fn)(void *ctx, size_t row);

struct steal {
    atomic_size_t next;
    size_t n, block;
    row_fn fn;
    void *ctx;
};

static void *steal_worker(void *p) {
    struct steal *s = (struct steal *)p;
    for (;;) {
        size_t r0 = atomic_fetch_add_explicit(&s->next, s->block, memory_order_relaxed);
        if (r0 >= s->n) break;
        size_t r1 = r0 + s->block < s->n ? r0 + s->block : s->n;
        for (size_t r = r0; r < r1; r++) s->fn(s->ctx, r);
    }
    return NULL;
}

/* Rows handed out in blocks from one atomic counter, as matvec_kq (cpu_math.rs:1165-1172,
 * block 8) and matmul (cpu_math.rs:204-216, block 16) do. */
static void steal_rows(size_t n, size_t block, int threads, row_fn fn, void *ctx) {
    struct steal s;
    atomic_init(&s.next, 0);
    s.n = n; s.block = block; s.fn = fn; s.ctx = ctx;
    if (threads > (int)n) threads = (int)(n ? n : 1);
    if (threads <= 1) { steal_worker(&s); return; }
    pthread_t *th = (pthread_t *)malloc(sizeof(pthread_t) * (size_t)threads);
    int started = 0;
    for (int i = 0; i < threads - 1; i++)
        if (pthread_create(&th[started], NULL, steal_worker, &s) == 0) started++;
    steal_worker(&s);
    for (int i = 0; i < started; i++) pthread_join(th[i], NULL);
    free(th);
}

/* ---------------------------------------------------------------- matvec_kq */

struct kq_ctx {
    const uint8_t *raw; uint32_t ty; size_t k, row_bytes;
    const float *x; const float *scales; const int8_t *q; const int32_t *bsums; float *y;
};

static void kq_row(void *p, size_t row) {
    struct kq_ctx *c = (struct kq_ctx *)p;
    const uint8_t *rb = c->raw + row * c->row_bytes;
    float v;
    switch (c->ty) { /* cpu_math.rs:1174-1181 */
    case OJO_Q4_K: v = ojo_dot_q4k(rb, c->k, c->scales, c->q, c->bsums); break;
    case OJO_Q5_K: v = ojo_dot_q5k(rb, c->k, c->scales, c->q, c->bsums); break;
    case OJO_Q8_0: v = ojo_dot_q80(rb, c->x, c->k); break;
    case OJO_IQ4_NL: v = ojo_dot_iq4nl(rb, c->x, c->k); break;   /* dot_iq, cpu_math.rs:1131-1141: f32 activations */
    case OJO_IQ4_XS: v = ojo_dot_iq4xs(rb, c->x, c->k); break;
    case OJO_IQ2_XXS: v = ojo_dot_iq2xxs_q8k(rb, c->k, c->scales, c->q); break;
    case OJO_IQ3_XXS: v = ojo_dot_iq3xxs_q8k(rb, c->k, c->scales, c->q); break;
    case OJO_IQ3_S: case OJO_IQ2_S: v = ojo_dot_iq_grid(c->ty, rb, c->x, c->k); break;
    default:       v = ojo_dot_q6k(rb, c->k, c->scales, c->q, c->bsums);
    }
    c->y[row] = v;
}

int ojo_matvec_kq(const uint8_t *raw, uint32_t ty, size_t n, size_t k, const float *x,
                  int threads, float *y) { /* cpu_math.rs:1145-1189 */
    size_t per256;
    switch (ty) {
    case OJO_Q4_K: per256 = 144; break;
    case OJO_Q5_K: per256 = 176; break;
    case OJO_Q6_K: per256 = 210; break;
    case OJO_Q8_0: per256 = 272; break;
    case OJO_IQ4_NL: per256 = 144; break;
    case OJO_IQ4_XS: per256 = 136; break;
    case OJO_IQ2_XXS: per256 = 66; break;
    case OJO_IQ3_XXS: per256 = 98; break;
    case OJO_IQ3_S: per256 = 110; break;
    case OJO_IQ2_S: per256 = 82; break;
    default: return -1;
    }
    size_t nsb = (k + 255) / 256;
    float *scales = (float *)malloc(nsb * sizeof(float));
    int8_t *q = (int8_t *)malloc(nsb * 256);
    int32_t *bsums = (int32_t *)malloc(nsb * 8 * sizeof(int32_t));
    ojo_quant_q8k(x, k, scales, q, bsums); /* done for every type, used by the K-quants */
    struct kq_ctx c = { raw, ty, k, k / 256 * per256, x, scales, q, bsums, y };
    /* (the reference's k / 256 form covers whole multiples of 256 only; rows of 32-weight blocks are sized per block here) */
    if (ty == OJO_Q8_0) c.row_bytes = k / 32 * 34;
    if (ty == OJO_IQ4_NL) c.row_bytes = k / 32 * 18;
    steal_rows(n, 8, threads, kq_row, &c);
    free(scales); free(q); free(bsums);
    return 0;
}

/* ---------------------------------------------------------------- row-int8 path */

void ojo_q8_rows_from_f16(const uint16_t *w16, size_t n, size_t k, int8_t *q, float *scale) {
    /* crates/ojas-formats/src/quant.rs:16-39 — note the division by sv, not a reciprocal. */
    for (size_t r = 0; r < n; r++) {
        float amax = 0.0f;
        for (size_t c = 0; c < k; c++) {
            float a = fabsf(ojo_f16_to_f32(w16[r * k + c]));
            if (a > amax) amax = a;
        }
        float sv = amax > 0.0f ? amax / 127.0f : 1.0f;
        scale[r] = sv;
        for (size_t c = 0; c < k; c++)
            q[r * k + c] = sat_i8(roundf(ojo_f16_to_f32(w16[r * k + c]) / sv));
    }
}

struct q8_ctx {
    const int8_t *wq; const float *wscale; size_t k, n, m;
    const int8_t *xq; const float *xs; const float *bias; float *ys;
};

static void q8_row(void *p, size_t row) { /* cpu_math.rs:217-231, dot_i8 :404-415 */
    struct q8_ctx *c = (struct q8_ctx *)p;
    const int8_t *qrow = c->wq + row * c->k;
    float b = c->bias ? c->bias[row] : 0.0f;
    float sw = c->wscale[row];
    for (size_t t = 0; t < c->m; t++) {
        const int8_t *qx = c->xq + t * c->k;
        int32_t acc = 0;
        for (size_t i = 0; i < c->k; i++) acc += (int32_t)qrow[i] * (int32_t)qx[i];
        c->ys[t * c->n + row] = b + (float)acc * sw * c->xs[t];
    }
}

void ojo_matmul_q8(const int8_t *wq, const float *wscale, size_t n, size_t k, const float *xs,
                   size_t m, const float *bias, int threads, float *ys) { /* cpu_math.rs:187-274 */
    int8_t *xq = (int8_t *)malloc(m * k);
    float *sx = (float *)malloc(m * sizeof(float));
    for (size_t t = 0; t < m; t++) sx[t] = ojo_quant_row_i8(xs + t * k, k, xq + t * k);
    struct q8_ctx c = { wq, wscale, k, n, m, xq, sx, bias, ys };
    int nt = (n * k * m < ((size_t)1 << 22)) ? 1 : threads; /* cpu_math.rs:202 */
    steal_rows(n, 16, nt, q8_row, &c);
    free(xq); free(sx);
}

/* ---------------------------------------------------------------- relayout */

void ojo_relayout_q4k_q4l(const uint8_t *w, size_t k, size_t n, uint8_t *nib, uint16_t *qa,
                          uint16_t *qb) { /* crates/ojas-formats/src/quant.rs:192-222 */
    size_t nblk = k / 32, nsb = k / 256;
    for (size_t r = 0; r < n; r++) {
        for (size_t b = 0; b < nblk; b++) {
            size_t sb = b >> 3; int j = (int)(b & 7);
            int g = j >> 1, hi = j & 1;
            const uint8_t *blk = w + (r * nsb + sb) * 144;
            float d = rdh(blk, 0), dm = rdh(blk, 2);
            uint8_t s_, m_;
            scale_min_k4(j, blk + 4, &s_, &m_);
            qa[r * nblk + b] = ojo_f32_to_f16(d * (float)s_);
            qb[r * nblk + b] = ojo_f32_to_f16(-dm * (float)m_);
            const uint8_t *qq = blk + 16 + g * 32;
            for (int i = 0; i < 16; i++) {
                uint8_t a = hi ? qq[2 * i] >> 4 : qq[2 * i] & 15;
                uint8_t c = hi ? qq[2 * i + 1] >> 4 : qq[2 * i + 1] & 15;
                nib[r * (k / 2) + b * 16 + i] = (uint8_t)(a | (c << 4));
            }
        }
    }
}

/* double -> binary16, round to nearest even, directly (no intermediate f32 rounding) */
static uint16_t f64_to_f16(double v) {
    uint16_t h = ojo_f32_to_f16((float)v);
    uint16_t sign = h & 0x8000u, mag = h & 0x7FFFu;
    if (mag >= 0x7C00u || v != v) return h;
    double a = v < 0 ? -v : v, best = -1.0;
    uint16_t pick = mag;
    for (int dlt = -1; dlt <= 1; dlt++) {
        int c = (int)mag + dlt;
        if (c < 0 || c >= 0x7C00) continue;
        double cv = (double)ojo_f16_to_f32((uint16_t)c), e = cv > a ? cv - a : a - cv;
        if (best < 0 || e < best || (e == best && !(c & 1))) { best = e; pick = (uint16_t)c; }
    }
    return (uint16_t)(sign | pick);
}

void ojo_q4l_weights_f16(const uint8_t *w, size_t k, size_t n, uint16_t *out) {
    /* What the reference's GPU prefill kernel puts in its tile for a Q4L weight
     * (crates/ojas-cuda/src/kernels/gemm_q.rs:104-140): q as a half, then one fused multiply-add
     * qa*q + qb in binary16 — the exact value rounded once.  qa*q + qb is exact in double
     * (11-bit x 4-bit product plus an 11-bit addend within the binary16 exponent range). */
    size_t nblk = k / 32;
    uint8_t *nib = (uint8_t *)malloc(n * k / 2);
    uint16_t *qa = (uint16_t *)malloc(n * nblk * 2), *qb = (uint16_t *)malloc(n * nblk * 2);
    ojo_relayout_q4k_q4l(w, k, n, nib, qa, qb);
    for (size_t r = 0; r < n; r++)
        for (size_t b = 0; b < nblk; b++) {
            double a = (double)ojo_f16_to_f32(qa[r * nblk + b]), c = (double)ojo_f16_to_f32(qb[r * nblk + b]);
            for (int i = 0; i < 16; i++) {
                uint8_t v = nib[r * (k / 2) + b * 16 + i];
                out[r * k + b * 32 + 2 * i] = f64_to_f16(a * (double)(v & 15) + c);
                out[r * k + b * 32 + 2 * i + 1] = f64_to_f16(a * (double)(v >> 4) + c);
            }
        }
    free(nib); free(qa); free(qb);
}

/* ---------------------------------------------------------------- double-precision reference */

struct ref_ctx {
    const uint8_t *raw; uint32_t ty; size_t n, k, m, row_bytes; int wmode;
    const double *xd; double *y;
};

static void ref_row(void *p, size_t row) {
    struct ref_ctx *c = (struct ref_ctx *)p;
    double *w = (double *)malloc(c->k * sizeof(double));
    const uint8_t *rb = c->raw + row * c->row_bytes;
    if (c->wmode == 1 || c->wmode == 2) {
        uint16_t *h = (uint16_t *)malloc(c->k * sizeof(uint16_t));
        if (c->wmode == 2) ojo_q4l_weights_f16(rb, c->k, 1, h);
        else ojo_dequant_to_f16(rb, c->ty, c->k, h);
        for (size_t i = 0; i < c->k; i++) w[i] = ojo_f16_to_f32(h[i]);
        free(h);
    } else {
        ojo_dequant_to_f64(rb, c->ty, c->k, w);
    }
    for (size_t t = 0; t < c->m; t++) {
        const double *x = c->xd + t * c->k;
        double acc = 0.0;
        for (size_t i = 0; i < c->k; i++) acc += w[i] * x[i];
        c->y[t * c->n + row] = acc;
    }
    free(w);
}

int ojo_matmul_ref(const uint8_t *raw, uint32_t ty, size_t n, size_t k, const float *x, size_t m,
                   int wmode, int xmode, int threads, double *y) {
    uint32_t bb, wpb;
    if (!ojo_block_shape(ty, &bb, &wpb) || k % wpb) return -1;
    if (wmode == 2 && ty != 12) return -1; /* the Q4L arithmetic exists for Q4_K only */
    double *xd = (double *)malloc(m * k * sizeof(double));
    for (size_t i = 0; i < m * k; i++) {
        float v = x[i];
        if (xmode == 1) v = ojo_f16_to_f32(ojo_f32_to_f16(v));
        else if (xmode == 2) v = ojo_bf16_to_f32(ojo_f32_to_bf16(v));
        xd[i] = v;
    }
    struct ref_ctx c = { raw, ty, n, k, m, k / wpb * bb, wmode, xd, y };
    steal_rows(n, 8, threads, ref_row, &c);
    free(xd);
    return 0;
}

/* ---------------------------------------------------------------- decode-layer glue */

void ojo_rmsnorm(const float *x, const float *w, size_t k, float eps, float *y) {
    /* crates/ojas-cpu/src/cpu_math.rs:456-460: f32 sum of squares in index order, / len,
     * inv = 1 / sqrt(ss + eps), y = (x * inv) * w */
    float ss = 0.0f;
    for (size_t i = 0; i < k; i++) ss += x[i] * x[i];
    ss = ss / (float)k;
    float inv = 1.0f / sqrtf(ss + eps);
    for (size_t i = 0; i < k; i++) y[i] = x[i] * inv * w[i];
}

float ojo_ffn_act(float g, int act) {
    /* act 0: silu, cpu_math.rs:486; act 1: gelu (tanh form), cpu_math.rs:497-501 */
    if (act == 1) {
        const float c = 0.7978845608028654f, a = 0.044715f;
        return 0.5f * g * (1.0f + tanhf(c * g * (1.0f + a * g * g)));
    }
    return g / (1.0f + expf(-g));
}

/* ---------------------------------------------------------------- MoE */

void ojo_moe_topk(const float *lg, int E, int ksel, uint32_t *idx, float *wgt) {
    /* crates/ojas-cuda/src/kernels/moe.rs:45-70; crates/ojas-cuda/tests/conformance.rs:385-392 */
    float *pr = (float *)malloc((size_t)E * sizeof(float));
    float mx = -3.4028235e38f;
    for (int e = 0; e < E; e++) if (lg[e] > mx) mx = lg[e];
    float sum = 0.0f;
    for (int e = 0; e < E; e++) { pr[e] = expf(lg[e] - mx); sum += pr[e]; }
    for (int e = 0; e < E; e++) pr[e] = pr[e] / sum;
    float wsum = 0.0f;
    for (int j = 0; j < ksel; j++) {
        float bv = -1.0f; int bi = 0;
        for (int e = 0; e < E; e++) if (pr[e] > bv) { bv = pr[e]; bi = e; }
        idx[j] = (uint32_t)bi;
        wgt[j] = bv;
        wsum += bv;
        pr[bi] = -1.0f;
    }
    for (int j = 0; j < ksel; j++) wgt[j] = wgt[j] / wsum;
    free(pr);
}

/* The reference's other routers.  nonorm (DeepSeek-V2): softmax, top-k by strict '>' (lowest index wins ties), the raw
 * probability exp(l - max) / sum of the chosen — crates/ojas-metal/src/kernels/moe.rs:130-150,
 * crates/ojas-cpu/src/cpu_deepseek.rs:286-305.  v3 (DeepSeek-V3 / GLM): s = sigmoid(l); chosen by s + bias; weight = s of
 * the chosen times 1/sum(chosen s) when `norm` and the sum is positive, times the routed scaling factor —
 * crates/ojas-metal/src/kernels/moe.rs:531-551, crates/ojas-cpu/src/cpu_glm.rs:526-548. */
void ojo_moe_topk_nonorm(const float *lg, int E, int ksel, uint32_t *idx, float *wgt) {
    float *pr = (float *)malloc((size_t)E * sizeof(float));
    float mx = -1e30f;
    for (int e = 0; e < E; e++) if (lg[e] > mx) mx = lg[e];
    float sum = 0.0f;
    for (int e = 0; e < E; e++) { pr[e] = expf(lg[e] - mx); sum += pr[e]; }
    for (int j = 0; j < ksel; j++) {
        float bv = -1.0f; int bi = 0;
        for (int e = 0; e < E; e++) if (pr[e] > bv) { bv = pr[e]; bi = e; }
        idx[j] = (uint32_t)bi;
        wgt[j] = bv / sum;
        pr[bi] = -1.0f;
    }
    free(pr);
}
void ojo_moe_topk_v3(const float *lg, const float *bias, int E, int ksel, float rscale, int norm, uint32_t *idx, float *wgt) {
    float *sg = (float *)malloc((size_t)E * sizeof(float)), *ch = (float *)malloc((size_t)E * sizeof(float));
    for (int e = 0; e < E; e++) { sg[e] = 1.0f / (1.0f + expf(-lg[e])); ch[e] = sg[e] + bias[e]; }
    float sum = 0.0f;
    for (int j = 0; j < ksel; j++) {
        float bv = -1e30f; int bi = 0;
        for (int e = 0; e < E; e++) if (ch[e] > bv) { bv = ch[e]; bi = e; }
        idx[j] = (uint32_t)bi;
        wgt[j] = sg[bi];
        sum += sg[bi];
        ch[bi] = -1e30f;
    }
    float inv = (norm && sum > 0.0f) ? 1.0f / sum : 1.0f;
    for (int j = 0; j < ksel; j++) wgt[j] = wgt[j] * inv * rscale;
    free(sg); free(ch);
}

static inline float silu(float x) { return x / (1.0f + expf(-x)); } /* cpu_math.rs:486 */

static int matvec_mode(const uint8_t *raw, uint32_t ty, size_t n, size_t k, const float *x,
                       int mode, int threads, float *y) {
    if (mode == 0) return ojo_matvec_kq(raw, ty, n, k, x, threads, y);
    double *yd = (double *)malloc(n * sizeof(double));
    int rc = ojo_matmul_ref(raw, ty, n, k, x, 1, 0, 0, threads, yd);
    for (size_t i = 0; i < n; i++) y[i] = (float)yd[i];
    free(yd);
    return rc;
}

int ojo_moe_ffn(const float *x, size_t T, size_t d, size_t n_ff, int n_expert, int ksel,
                const uint32_t *idx, const float *wgt, const uint8_t *gate, const uint8_t *up,
                uint32_t ty_gu, const uint8_t *down, uint32_t ty_d, int mode, int threads,
                float *y) { /* crates/ojas-cpu/src/cpu_glm.rs:551-582 */
    uint32_t bb_gu, w_gu, bb_d, w_d;
    if (!ojo_block_shape(ty_gu, &bb_gu, &w_gu) || !ojo_block_shape(ty_d, &bb_d, &w_d)) return -1;
    if (d % w_gu || n_ff % w_d) return -1;
    size_t gu_bytes = n_ff * (d / w_gu) * bb_gu;  /* one expert's gate (or up) */
    size_t dn_bytes = d * (n_ff / w_d) * bb_d;    /* one expert's down */
    float *gv = (float *)malloc(n_ff * sizeof(float));
    float *uv = (float *)malloc(n_ff * sizeof(float));
    float *dv = (float *)malloc(d * sizeof(float));
    int rc = 0;
    for (size_t t = 0; t < T && !rc; t++) {
        const float *xt = x + t * d;
        for (int j = 0; j < ksel && !rc; j++) {
            uint32_t e = idx[t * (size_t)ksel + j];
            if ((int)e >= n_expert) { rc = -2; break; }
            rc |= matvec_mode(gate + e * gu_bytes, ty_gu, n_ff, d, xt, mode, threads, gv);
            rc |= matvec_mode(up + e * gu_bytes, ty_gu, n_ff, d, xt, mode, threads, uv);
            for (size_t i = 0; i < n_ff; i++) gv[i] = silu(gv[i]) * uv[i];
            rc |= matvec_mode(down + e * dn_bytes, ty_d, d, n_ff, gv, mode, threads, dv);
            float w = wgt[t * (size_t)ksel + j];
            for (size_t i = 0; i < d; i++) y[t * d + i] += w * dv[i];
        }
    }
    free(gv); free(uv); free(dv);
    return rc;
}

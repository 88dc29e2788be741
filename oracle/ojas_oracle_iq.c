/*
 * TEST INFRASTRUCTURE — CPU restatement of the reference's arithmetic for the grid-codebook GGUF formats
 * (IQ2_XXS 16, IQ2_XS 17, IQ3_XXS 18, IQ1_S 19, IQ3_S 21, IQ2_S 22, IQ1_M 29).  Part of the oracle library:
 * only the test-suite, the smoke check and the CPU-baseline leg of the benchmark may load it.
 *
 * Decoders follow crates/ojas-formats/src/gguf.rs:840-1041, the row dots crates/ojas-cpu/src/cpu_math.rs:728-757
 * (dot_iq2xxs), :884-913 (dot_iq3xxs), :915-941 (dot_iq2s), :1023-1052 (dot_iq3s), :1057-1090 (dot_iq2xxs_q8k),
 * :1093-1128 (dot_iq3xxs_q8k).  The codebooks come packed (ojk_iq_grids.h: 16 bits per entry) and are expanded
 * here; tests/golden/iq_grid_digests.json holds a digest of every published table for the round trip.
 *
 * Pins: the decoders by the digests of crates/ojas-formats/tests/quant_formats.rs:41-44,46-47,49 (random blocks sweep
 * the codebooks) and by closed forms on hand-built blocks (tests/test_oracle_golden.py); the f32 dots by an f64 dot
 * over the exactly decoded row and by one-hot activations; the int8-activation dots by the identity
 * dot(row, quant_q8k(x)) == sum_b xs_b * sum_j w_j * q_j evaluated in double.
 */
#include <math.h>
#include <string.h>
#include "ojas_oracle.h"
#include "../ojas-engine_amd/csrc/kernels/ojk_iq_grids.h"

static inline float rdh(const uint8_t *b, size_t i) { return ojo_f16_to_f32((uint16_t)(b[i] | (b[i + 1] << 8))); }
static inline uint32_t rd32(const uint8_t *b) { return (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) | ((uint32_t)b[3] << 24); }
static inline uint16_t rd16(const uint8_t *b) { return (uint16_t)(b[0] | (b[1] << 8)); }

/* ksigns_iq2xs[i]: the seven stored sign bits plus an eighth that makes the number of set bits even. */
static inline uint8_t ksigns(uint32_t i) {
    uint32_t p = i & 127u;
    p ^= p >> 4; p ^= p >> 2; p ^= p >> 1;
    return (uint8_t)((i & 127u) | ((p & 1u) << 7));
}

static const uint8_t mag_iq2[3] = {8, 25, 43};
static const uint8_t mag_iq3xxs[8] = {4, 12, 20, 28, 36, 44, 52, 62};

static inline void grid8_iq2(const unsigned short *pk, uint32_t i, uint8_t g[8]) {
    for (int j = 0; j < 8; j++) g[j] = mag_iq2[(pk[i] >> (2 * j)) & 3];
}
static inline void grid8_iq1(uint32_t i, int8_t g[8]) {
    for (int j = 0; j < 8; j++) g[j] = (int8_t)((int)((ojk_iq1s_grid_pk[i] >> (2 * j)) & 3) - 1);
}
static inline void grid4_iq3xxs(uint32_t i, uint8_t g[4]) {
    for (int j = 0; j < 4; j++) g[j] = mag_iq3xxs[(ojk_iq3xxs_grid_pk[i] >> (3 * j)) & 7];
}
static inline void grid4_iq3s(uint32_t i, uint8_t g[4]) {
    for (int j = 0; j < 4; j++) g[j] = (uint8_t)(2 * ((ojk_iq3s_grid_pk[i] >> (3 * j)) & 7) + 1);
}

/* The published table `which` (0 iq2xxs, 1 iq2xs, 2 iq2s, 3 iq3xxs, 4 iq3s, 5 iq1s) as little-endian bytes of its
 * u64 / u32 entries; returns the byte count (out may be NULL). */
size_t ojo_iq_grid_bytes(int which, uint8_t *out) {
    static const size_t entries[6] = {256, 512, 1024, 256, 512, 2048};
    static const size_t width[6] = {8, 8, 8, 4, 4, 8};
    if (which < 0 || which > 5) return 0;
    if (out)
        for (size_t i = 0; i < entries[which]; i++) {
            uint8_t *o = out + i * width[which];
            switch (which) {
            case 0: grid8_iq2(ojk_iq2xxs_grid_pk, (uint32_t)i, o); break;
            case 1: grid8_iq2(ojk_iq2xs_grid_pk, (uint32_t)i, o); break;
            case 2: grid8_iq2(ojk_iq2s_grid_pk, (uint32_t)i, o); break;
            case 3: grid4_iq3xxs((uint32_t)i, o); break;
            case 4: grid4_iq3s((uint32_t)i, o); break;
            default: grid8_iq1((uint32_t)i, (int8_t *)o);
            }
        }
    return entries[which] * width[which];
}

int ojo_iq_is_grid_type(uint32_t ty) {
    return ty == OJO_IQ2_XXS || ty == OJO_IQ2_XS || ty == OJO_IQ3_XXS || ty == OJO_IQ1_S || ty == OJO_IQ3_S ||
           ty == OJO_IQ2_S || ty == OJO_IQ1_M;
}

/* One 256-weight block: `of` = the f32 value the reference rounds to f16 (its operators, its order), `od` = the same
 * product of exact factors in double.  Either may be NULL. */
#define PUT(i, scale32, scale64, v)                                        \
    do {                                                                   \
        if (of) of[i] = (scale32) * (float)(v);                            \
        if (od) od[i] = (scale64) * (double)(v);                           \
    } while (0)

void ojo_iq_block(uint32_t ty, const uint8_t *blk, float *of, double *od) {
    const float DELTA = 0.125f;
    switch (ty) {
    case OJO_IQ2_XXS: { /* gguf.rs:840-864 */
        float d = rdh(blk, 0);
        const uint8_t *qs = blk + 2;
        for (int ib = 0; ib < 8; ib++) {
            uint32_t a0 = rd32(qs + 8 * ib), a1 = rd32(qs + 8 * ib + 4);
            float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
            double db64 = (double)d * (0.5 + (double)(a1 >> 28)) * 0.25;
            for (int l = 0; l < 4; l++) {
                uint8_t g[8];
                grid8_iq2(ojk_iq2xxs_grid_pk, (a0 >> (8 * l)) & 255, g);
                uint8_t s = ksigns((a1 >> (7 * l)) & 127);
                for (int j = 0; j < 8; j++) {
                    float sg = (s >> j) & 1 ? -1.0f : 1.0f;
                    if (of) of[ib * 32 + l * 8 + j] = db * (float)g[j] * sg;
                    if (od) od[ib * 32 + l * 8 + j] = db64 * (double)g[j] * (double)sg;
                }
            }
        }
    } break;
    case OJO_IQ2_XS: { /* gguf.rs:865-888 */
        float d = rdh(blk, 0);
        const uint8_t *qs = blk + 2, *sc = blk + 66;
        for (int ib = 0; ib < 8; ib++) {
            float db[2] = {d * (0.5f + (float)(sc[ib] & 0xF)) * 0.25f, d * (0.5f + (float)(sc[ib] >> 4)) * 0.25f};
            double db64[2] = {(double)d * (0.5 + (double)(sc[ib] & 0xF)) * 0.25, (double)d * (0.5 + (double)(sc[ib] >> 4)) * 0.25};
            for (int l = 0; l < 4; l++) {
                uint16_t q = rd16(qs + 2 * (4 * ib + l));
                uint8_t g[8];
                grid8_iq2(ojk_iq2xs_grid_pk, q & 511, g);
                uint8_t s = ksigns(q >> 9);
                for (int j = 0; j < 8; j++) {
                    float sg = (s >> j) & 1 ? -1.0f : 1.0f;
                    if (of) of[ib * 32 + l * 8 + j] = db[l / 2] * (float)g[j] * sg;
                    if (od) od[ib * 32 + l * 8 + j] = db64[l / 2] * (double)g[j] * (double)sg;
                }
            }
        }
    } break;
    case OJO_IQ2_S: { /* gguf.rs:889-914 */
        float d = rdh(blk, 0);
        const uint8_t *qs = blk + 2, *qh = blk + 66, *sc = blk + 74;
        for (int ib = 0; ib < 8; ib++) {
            float db[2] = {d * (0.5f + (float)(sc[ib] & 0xF)) * 0.25f, d * (0.5f + (float)(sc[ib] >> 4)) * 0.25f};
            double db64[2] = {(double)d * (0.5 + (double)(sc[ib] & 0xF)) * 0.25, (double)d * (0.5 + (double)(sc[ib] >> 4)) * 0.25};
            for (int l = 0; l < 4; l++) {
                uint32_t gi = (uint32_t)qs[4 * ib + l] | ((((uint32_t)qh[ib]) << (8 - 2 * l)) & 0x300);
                uint8_t g[8];
                grid8_iq2(ojk_iq2s_grid_pk, gi, g);
                uint8_t s = qs[32 + 4 * ib + l];
                for (int j = 0; j < 8; j++) {
                    float sg = (s >> j) & 1 ? -1.0f : 1.0f;
                    if (of) of[ib * 32 + l * 8 + j] = db[l / 2] * (float)g[j] * sg;
                    if (od) od[ib * 32 + l * 8 + j] = db64[l / 2] * (double)g[j] * (double)sg;
                }
            }
        }
    } break;
    case OJO_IQ3_XXS: { /* gguf.rs:915-940 */
        float d = rdh(blk, 0);
        const uint8_t *qs = blk + 2, *ss = qs + 64;
        for (int ib = 0; ib < 8; ib++) {
            uint32_t a = rd32(ss + 4 * ib);
            float db = d * (0.5f + (float)(a >> 28)) * 0.5f;
            double db64 = (double)d * (0.5 + (double)(a >> 28)) * 0.5;
            const uint8_t *q = qs + 8 * ib;
            for (int l = 0; l < 4; l++) {
                uint8_t s = ksigns((a >> (7 * l)) & 127), g[8];
                grid4_iq3xxs(q[2 * l], g);
                grid4_iq3xxs(q[2 * l + 1], g + 4);
                for (int j = 0; j < 8; j++) {
                    float sg = (s >> j) & 1 ? -1.0f : 1.0f;
                    if (of) of[ib * 32 + l * 8 + j] = db * (float)g[j] * sg;
                    if (od) od[ib * 32 + l * 8 + j] = db64 * (double)g[j] * (double)sg;
                }
            }
        }
    } break;
    case OJO_IQ3_S: { /* gguf.rs:941-976 */
        float d = rdh(blk, 0);
        const uint8_t *qs = blk + 2, *qh = blk + 66, *sgn = blk + 74, *sc = blk + 106;
        for (int p = 0; p < 4; p++) {
            float dbs[2] = {d * (1.0f + 2.0f * (float)(sc[p] & 0xF)), d * (1.0f + 2.0f * (float)(sc[p] >> 4))};
            double dbs64[2] = {(double)d * (1.0 + 2.0 * (double)(sc[p] & 0xF)), (double)d * (1.0 + 2.0 * (double)(sc[p] >> 4))};
            for (int half = 0; half < 2; half++) {
                uint32_t h = qh[2 * p + half];
                int qo = 16 * p + 8 * half, so = 8 * p + 4 * half;
                for (int l = 0; l < 4; l++) {
                    uint8_t g[8], s = sgn[so + l];
                    grid4_iq3s((uint32_t)qs[qo + 2 * l] | ((h << (8 - 2 * l)) & 256), g);
                    grid4_iq3s((uint32_t)qs[qo + 2 * l + 1] | ((h << (7 - 2 * l)) & 256), g + 4);
                    for (int j = 0; j < 8; j++) {
                        float sg = (s >> j) & 1 ? -1.0f : 1.0f;
                        int at = (2 * p + half) * 32 + l * 8 + j;
                        if (of) of[at] = dbs[half] * (float)g[j] * sg;
                        if (od) od[at] = dbs64[half] * (double)g[j] * (double)sg;
                    }
                }
            }
        }
    } break;
    case OJO_IQ1_S: { /* gguf.rs:977-999 */
        float d = rdh(blk, 0);
        const uint8_t *qs = blk + 2;
        for (int ib = 0; ib < 8; ib++) {
            uint16_t qh = rd16(blk + 34 + 2 * ib);
            float dl = d * (float)(2 * ((qh >> 12) & 7) + 1);
            double dl64 = (double)d * (double)(2 * ((qh >> 12) & 7) + 1);
            float delta = qh & 0x8000 ? -DELTA : DELTA;
            for (int l = 0; l < 4; l++) {
                int8_t g[8];
                grid8_iq1((uint32_t)qs[4 * ib + l] | ((uint32_t)((qh >> (3 * l)) & 7) << 8), g);
                for (int j = 0; j < 8; j++) PUT(ib * 32 + l * 8 + j, dl, dl64, (float)g[j] + delta);
            }
        }
    } break;
    case OJO_IQ1_M: { /* gguf.rs:1000-1041 */
        const uint8_t *qs = blk, *qh = blk + 32;
        uint16_t sc[4];
        for (int i = 0; i < 4; i++) sc[i] = rd16(blk + 48 + 2 * i);
        uint16_t dbits = (uint16_t)((sc[0] >> 12) | ((sc[1] >> 8) & 0x00f0) | ((sc[2] >> 4) & 0x0f00) | (sc[3] & 0xf000));
        float d = ojo_f16_to_f32(dbits);
        for (int ib = 0; ib < 8; ib++) {
            uint16_t w = sc[ib / 2];
            int sh = 6 * (ib % 2);
            float dl[2] = {d * (float)(2 * ((w >> sh) & 7) + 1), d * (float)(2 * ((w >> (sh + 3)) & 7) + 1)};
            double dl64[2] = {(double)d * (double)(2 * ((w >> sh) & 7) + 1), (double)d * (double)(2 * ((w >> (sh + 3)) & 7) + 1)};
            uint32_t h0 = qh[2 * ib], h1 = qh[2 * ib + 1];
            uint32_t idx[4] = {qs[4 * ib] | ((h0 << 8) & 0x700), qs[4 * ib + 1] | ((h0 << 4) & 0x700),
                               qs[4 * ib + 2] | ((h1 << 8) & 0x700), qs[4 * ib + 3] | ((h1 << 4) & 0x700)};
            float dq[4] = {h0 & 0x08 ? -DELTA : DELTA, h0 & 0x80 ? -DELTA : DELTA, h1 & 0x08 ? -DELTA : DELTA,
                           h1 & 0x80 ? -DELTA : DELTA};
            for (int l = 0; l < 4; l++) {
                int8_t g[8];
                grid8_iq1(idx[l], g);
                for (int j = 0; j < 8; j++) PUT(ib * 32 + l * 8 + j, dl[l / 2], dl64[l / 2], (float)g[j] + dq[l]);
            }
        }
    } break;
    default: break;
    }
}

/* ---------------------------------------------------------------- f32-activation row dots */

float ojo_dot_iq2xxs(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:728-757 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 256; b++) {
        const uint8_t *blk = row + b * 66, *qs = blk + 2;
        const float *xb = x + b * 256;
        float d = rdh(blk, 0), bsum = 0.0f;
        for (int g = 0; g < 8; g++) {
            uint32_t a0 = rd32(qs + 8 * g), a1 = rd32(qs + 8 * g + 4);
            float db = (0.5f + (float)(a1 >> 28)) * 0.25f, gsum = 0.0f;
            for (int l = 0; l < 4; l++) {
                uint8_t grid[8], signs = ksigns((a1 >> (7 * l)) & 127);
                grid8_iq2(ojk_iq2xxs_grid_pk, (a0 >> (8 * l)) & 255, grid);
                const float *xg = xb + g * 32 + l * 8;
                for (int j = 0; j < 8; j++) {
                    float mag = (float)grid[j], v = (signs >> j) & 1 ? -mag : mag;
                    gsum += v * xg[j];
                }
            }
            bsum += db * gsum;
        }
        sum += d * bsum;
    }
    return sum;
}

float ojo_dot_iq3xxs(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:884-913 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 256; b++) {
        const uint8_t *blk = row + b * 98, *qs = blk + 2, *ss = blk + 66;
        const float *xb = x + b * 256;
        float d = rdh(blk, 0), bsum = 0.0f;
        for (int g = 0; g < 8; g++) {
            uint32_t aux = rd32(ss + 4 * g);
            float db = 0.5f + (float)(aux >> 28), gsum = 0.0f;
            for (int l = 0; l < 4; l++) {
                uint8_t signs = ksigns((aux >> (7 * l)) & 127), g1[4], g2[4];
                grid4_iq3xxs(qs[8 * g + 2 * l], g1);
                grid4_iq3xxs(qs[8 * g + 2 * l + 1], g2);
                const float *xg = xb + g * 32 + l * 8;
                for (int j = 0; j < 4; j++) {
                    float m1 = (float)g1[j], m2 = (float)g2[j];
                    gsum += ((signs >> j) & 1 ? -m1 : m1) * xg[j];
                    gsum += ((signs >> (j + 4)) & 1 ? -m2 : m2) * xg[j + 4];
                }
            }
            bsum += db * gsum;
        }
        sum += d * 0.5f * bsum;
    }
    return sum;
}

float ojo_dot_iq2s(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:915-941 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 256; b++) {
        const uint8_t *blk = row + b * 82, *qs = blk + 2, *signs = blk + 34, *qh = blk + 66, *scales = blk + 74;
        const float *xb = x + b * 256;
        float d = rdh(blk, 0), bsum = 0.0f;
        for (int g = 0; g < 8; g++) {
            float db[2] = {0.5f + (float)(scales[g] & 0xf), 0.5f + (float)(scales[g] >> 4)};
            for (int l = 0; l < 4; l++) {
                uint32_t gi = (uint32_t)qs[4 * g + l] | ((((uint32_t)qh[g]) << (8 - 2 * l)) & 0x300);
                uint8_t grid[8], sb = signs[4 * g + l];
                grid8_iq2(ojk_iq2s_grid_pk, gi, grid);
                const float *xg = xb + g * 32 + l * 8;
                float gsum = 0.0f;
                for (int j = 0; j < 8; j++) {
                    float m = (float)grid[j];
                    gsum += ((sb >> j) & 1 ? -m : m) * xg[j];
                }
                bsum += db[l / 2] * gsum;
            }
        }
        sum += d * 0.25f * bsum;
    }
    return sum;
}

float ojo_dot_iq3s(const uint8_t *row, const float *x, size_t k) { /* cpu_math.rs:1023-1052 */
    float sum = 0.0f;
    for (size_t b = 0; b < k / 256; b++) {
        const uint8_t *blk = row + b * 110, *qs = blk + 2, *qh = blk + 66, *sg = blk + 74, *sc = blk + 106;
        const float *xb = x + b * 256;
        float d = rdh(blk, 0), bsum = 0.0f;
        for (int g = 0; g < 8; g++) {
            uint32_t h = qh[g];
            const float *xg = xb + g * 32;
            float gsum = 0.0f;
            for (int l = 0; l < 4; l++) {
                uint8_t g1[4], g2[4], s = sg[4 * g + l];
                grid4_iq3s((uint32_t)qs[8 * g + 2 * l] | ((h << (8 - 2 * l)) & 256), g1);
                grid4_iq3s((uint32_t)qs[8 * g + 2 * l + 1] | ((h << (7 - 2 * l)) & 256), g2);
                for (int j = 0; j < 4; j++) {
                    float s1 = (s >> j) & 1 ? -1.0f : 1.0f, s2 = (s >> (j + 4)) & 1 ? -1.0f : 1.0f;
                    gsum += (float)g1[j] * s1 * xg[8 * l + j];
                    gsum += (float)g2[j] * s2 * xg[8 * l + j + 4];
                }
            }
            bsum += (1.0f + 2.0f * (float)((sc[g >> 1] >> (4 * (g & 1))) & 0xF)) * gsum;
        }
        sum += d * bsum;
    }
    return sum;
}

/* ---------------------------------------------------------------- int8-activation row dots */

static int32_t dot_i8_32(const int8_t *a, const int8_t *b) { /* cpu_math.rs:404-415 */
    int32_t s = 0;
    for (int i = 0; i < 32; i++) s += (int32_t)a[i] * (int32_t)b[i];
    return s;
}

float ojo_dot_iq2xxs_q8k(const uint8_t *row, size_t k, const float *scales, const int8_t *q) { /* cpu_math.rs:1057-1090 */
    float sum = 0.0f;
    int8_t w[256];
    for (size_t b = 0; b < (k + 255) / 256; b++) {
        const uint8_t *blk = row + b * 66, *qs = blk + 2;
        float d = rdh(blk, 0), sc[8];
        for (int g = 0; g < 8; g++) {
            uint32_t a0 = rd32(qs + 8 * g), a1 = rd32(qs + 8 * g + 4);
            sc[g] = (0.5f + (float)(a1 >> 28)) * 0.25f;
            for (int l = 0; l < 4; l++) {
                uint8_t grid[8], signs = ksigns((a1 >> (7 * l)) & 127);
                grid8_iq2(ojk_iq2xxs_grid_pk, (a0 >> (8 * l)) & 255, grid);
                for (int j = 0; j < 8; j++) {
                    int8_t m = (int8_t)grid[j];
                    w[g * 32 + l * 8 + j] = (signs >> j) & 1 ? (int8_t)-m : m;
                }
            }
        }
        const int8_t *xq = q + b * 256;
        float bsum = 0.0f;
        for (int g = 0; g < 8; g++) bsum += sc[g] * (float)dot_i8_32(w + g * 32, xq + g * 32);
        sum += d * scales[b] * bsum;
    }
    return sum;
}

float ojo_dot_iq3xxs_q8k(const uint8_t *row, size_t k, const float *scales, const int8_t *q) { /* cpu_math.rs:1093-1128 */
    float sum = 0.0f;
    int8_t w[256];
    for (size_t b = 0; b < (k + 255) / 256; b++) {
        const uint8_t *blk = row + b * 98, *qs = blk + 2, *ss = blk + 66;
        float d = rdh(blk, 0), sc[8];
        for (int g = 0; g < 8; g++) {
            uint32_t aux = rd32(ss + 4 * g);
            sc[g] = (0.5f + (float)(aux >> 28)) * 0.5f;
            for (int l = 0; l < 4; l++) {
                uint8_t signs = ksigns((aux >> (7 * l)) & 127), g1[4], g2[4];
                grid4_iq3xxs(qs[8 * g + 2 * l], g1);
                grid4_iq3xxs(qs[8 * g + 2 * l + 1], g2);
                for (int j = 0; j < 4; j++) {
                    int8_t m1 = (int8_t)g1[j], m2 = (int8_t)g2[j];
                    w[g * 32 + l * 8 + j] = (signs >> j) & 1 ? (int8_t)-m1 : m1;
                    w[g * 32 + l * 8 + j + 4] = (signs >> (j + 4)) & 1 ? (int8_t)-m2 : m2;
                }
            }
        }
        const int8_t *xq = q + b * 256;
        float bsum = 0.0f;
        for (int g = 0; g < 8; g++) bsum += sc[g] * (float)dot_i8_32(w + g * 32, xq + g * 32);
        sum += d * scales[b] * bsum;
    }
    return sum;
}

/* dot_iq (cpu_math.rs:1131-1141) for the grid types it serves. */
float ojo_dot_iq_grid(uint32_t ty, const uint8_t *row, const float *x, size_t k) {
    switch (ty) {
    case OJO_IQ2_XXS: return ojo_dot_iq2xxs(row, x, k);
    case OJO_IQ3_XXS: return ojo_dot_iq3xxs(row, x, k);
    case OJO_IQ3_S: return ojo_dot_iq3s(row, x, k);
    case OJO_IQ2_S: return ojo_dot_iq2s(row, x, k);
    default: return NAN;
    }
}

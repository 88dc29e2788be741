// Kernel manifest: one row per canonical entry name, with the family (code object) that defines
// it, its positional signature (buffers first, then u32 constants — the convention the
// reference enforces in crates/ojas-cuda/tests/conformance.rs:85-109), the bytes each buffer
// must hold at given constants, and the wave64 launch shape.  The reference keeps the
// equivalent tables in crates/ojas-core/src/quant_src.rs:83-111 (FORMATS) and :168-193
// (MOE_FORMATS), and the name -> family registry in crates/ojas-cuda/src/kernels/mod.rs:111-145.
#include <cstring>
#include <deque>

#include "ojh_internal.h"

static const ojh_block_format kFormats[] = {
    {OJH_Q8_0, 34, 32, "q80"},
    {OJH_Q4_K, 144, 256, "q4k"},
    {OJH_Q5_K, 176, 256, "q5k"},
    {OJH_Q6_K, 210, 256, "q6k"},
    {OJH_IQ4_NL, 18, 32, "iq4nl"},
    {OJH_IQ4_XS, 136, 256, "iq4xs"},
    {OJH_Q4_0, 18, 32, "q40"},
    {OJH_Q4_1, 20, 32, "q41"},
    {OJH_Q5_0, 22, 32, "q50"},
    {OJH_Q5_1, 24, 32, "q51"},
    {OJH_Q2_K, 84, 256, "q2k"},
    {OJH_Q3_K, 110, 256, "q3k"},
    {OJH_IQ2_XXS, 66, 256, "iq2xxs"},
    {OJH_IQ2_XS, 74, 256, "iq2xs"},
    {OJH_IQ2_S, 82, 256, "iq2s"},
    {OJH_IQ3_XXS, 98, 256, "iq3xxs"},
    {OJH_IQ3_S, 110, 256, "iq3s"},
    {OJH_IQ1_S, 50, 256, "iq1s"},
    {OJH_IQ1_M, 56, 256, "iq1m"},
    {OJH_MXFP4, 17, 32, "mxfp4"},
};

// Formats whose CPU path multiplies the raw row with f32 activations (dot_q80, dot_iq4nl, dot_iq4xs:
// crates/ojas-cpu/src/cpu_math.rs:1131-1141, :1179) instead of quantizing them per 256.
bool ojh_float_rows(uint32_t t) { return t == OJH_Q8_0 || ojh_float_only(t); }
// ... and for which this library has the f32-activation matvecs only: no int8-activation form, no MFMA tile
// (the IQ4 types, and the legacy 32-weight blocks and Q2_K / Q3_K, which the reference runs on its GPU path alone)
// (of the grid-codebook formats the CPU path multiplies IQ3_S and IQ2_S with f32 activations, dot_iq3s / dot_iq2s, and
// IQ2_XXS and IQ3_XXS with int8 activations, dot_iq2xxs_q8k / dot_iq3xxs_q8k: cpu_math.rs:1177-1179; IQ2_XS, IQ1_S and
// IQ1_M run on the reference's GPU path alone)
bool ojh_float_only(uint32_t t) {
    return t == OJH_IQ4_NL || t == OJH_IQ4_XS || t == OJH_Q4_0 || t == OJH_Q4_1 || t == OJH_Q5_0 || t == OJH_Q5_1 ||
           t == OJH_Q2_K || t == OJH_Q3_K || t == OJH_IQ3_S || t == OJH_IQ2_S || t == OJH_IQ2_XS || t == OJH_IQ1_S ||
           t == OJH_IQ1_M || t == OJH_MXFP4;
}
bool ojh_grid_type(uint32_t t) {
    return t == OJH_IQ2_XXS || t == OJH_IQ2_XS || t == OJH_IQ2_S || t == OJH_IQ3_XXS || t == OJH_IQ3_S || t == OJH_IQ1_S ||
           t == OJH_IQ1_M;
}

// What the kernels' loads need of a block tensor's address: the widest power of two (up to 16) dividing the
// block size, except that only Q2_K's kernels use the 4 of a block size that is 4 mod 8.
size_t ojh_block_align(const ojh_block_format *f) {
    return f->bytes % 16 == 0 ? 16 : f->bytes % 8 == 0 ? 8 : f->type == OJH_Q2_K ? 4 : f->bytes % 2 == 0 ? 2 : 1;
}

const ojh_block_format *ojh_format(uint32_t t) {
    for (const auto &f : kFormats)
        if (f.type == t) return &f;
    return nullptr;
}

size_t ojh_row_bytes(uint32_t ggml_type, uint32_t k) {
    const ojh_block_format *f = ojh_format(ggml_type);
    if (!f || k == 0 || k % f->weights) return 0;
    return (size_t)(k / f->weights) * f->bytes;
}

// A check fills need[i] = bytes buffer i must hold from its offset, and may lower align[i], the
// alignment (pointer + offset) must have (16 unless the kernel reads the buffer with narrower
// loads).

static int check_block(const uint32_t block[3], uint32_t exact) {
    if (block[1] != 1 || block[2] != 1) return ojh_fail(OJH_ERR_ARG, "block must be [x,1,1]");
    if (exact) {
        if (block[0] != exact) return ojh_fail(OJH_ERR_ARG, "block.x must be %u, got %u", exact, block[0]);
    } else if (block[0] == 0 || block[0] % 64 || block[0] > 256) {
        return ojh_fail(OJH_ERR_ARG, "block.x must be a multiple of 64 up to 256, got %u", block[0]);
    }
    return OJH_OK;
}

static int check_kn(const ojh_kernel_spec *s, uint32_t K, uint32_t N, const ojh_block_format **fmt) {
    const ojh_block_format *f = ojh_format(s->type);
    if (!f) return ojh_fail(OJH_ERR_ARG, "%s: no block format", s->name);
    if (K == 0 || N == 0 || K % f->weights)
        return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a positive multiple of %u and N=%u positive",
                        s->name, K, f->weights, N);
    *fmt = f;
    return OJH_OK;
}

// gemv_nat_<fmt>{,_accum,_bias,_rN}(x, w, y[, bs], K, N)
static int check_gemv_nat(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if ((rc = check_block(block, 0))) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    uint64_t cover = (uint64_t)grid[0] * (block[0] / 64) * s->rows_per_wave;
    if (cover < N) return ojh_fail(OJH_ERR_ARG, "%s: grid covers %llu rows of N=%u", s->name,
                                   (unsigned long long)cover, N);
    need[0] = (size_t)K * 4;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)N * 4;
    if (s->n_bufs == 4) need[3] = (size_t)N * 4;
    align[1] = ojh_block_align(f);
    align[2] = align[3] = 4;
    return OJH_OK;
}

// The LDS-staged Q8_0 matvec cuts K into KC chunks of K / 32 / KC blocks: the smallest KC of 1, 2, 4
// whose chunk is at most 128 blocks and a multiple of 8 blocks (16-byte copy units); 0 if none.
uint32_t ojh_q80_lds_kc(uint32_t K) {
    if (!K || K % 256) return 0;
    const uint32_t nb = K / 32;
    for (uint32_t kc = 1; kc <= 4; kc *= 2)
        if (nb % kc == 0 && nb / kc <= 128 && (nb / kc) % 8 == 0) return kc;
    return 0;
}

// gemv_nat_q80_lds{,_accum,_bias}(x, w, y[, bs], K, N, KC): rows grid-stride, 4 / KC per workgroup step
static int check_gemv_q80_lds(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                              const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t K = c[0], N = c[1], KC = c[2];
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (!N) return ojh_fail(OJH_ERR_ARG, "%s: N must be positive", s->name);
    const uint32_t want = ojh_q80_lds_kc(K);
    if (!want) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: K=%u has no chunking of 1, 2 or 4 pieces of <= 128 blocks in 16-byte units", s->name, K);
    if (KC != want) return ojh_fail(OJH_ERR_ARG, "%s: KC=%u, K=%u takes KC=%u", s->name, KC, K, want);
    if (!grid[0] || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1], x > 0", s->name);
    need[0] = (size_t)K * 4;
    need[1] = (size_t)N * (K / 32) * 34;
    need[2] = (size_t)N * 4;
    if (s->n_bufs == 4) need[3] = (size_t)N * 4;
    align[0] = align[1] = 16;
    align[2] = align[3] = 4;
    return OJH_OK;
}
// A whole multiple of the CU count: two workgroups per CU when a wave owns whole rows, three when four
// waves share a row (measured; uneven grids lose 5-10 %)
static int shape_q80_lds(const ojh_kernel_spec *, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t,
                         uint32_t grid[3], uint32_t block[3]) {
    uint32_t kc = ojh_q80_lds_kc(K);
    if (!kc) return ojh_fail(OJH_ERR_UNSUPPORTED, "gemv_nat_q80_lds: K=%u cannot be chunked", K);
    uint32_t steps = (N + 4 / kc - 1) / (4 / kc);
    uint32_t bpc = dev->q80_lds_bpc ? dev->q80_lds_bpc : (kc == 1 ? 2u : 3u);
    uint32_t resident = (uint32_t)dev->prop.multiProcessorCount * bpc;
    grid[0] = steps < resident ? steps : resident;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// gemm_q8k_q4k_mf(xq, xs, w, y, K, N, M, ACC, RW, RT): 16 RW RT rows x up to 64 tokens per workgroup.
// The tokens of a workgroup wait in 76 KB of LDS chunk by chunk of K; a chunk must hold at least
// 4 / RW super-blocks (the waves that split K).  RT (row tiles per wave) must be 1.
uint32_t ojh_gemm_q8k_fit(uint32_t M, uint32_t RW, uint32_t RT) {   // super-blocks of K that fit for the largest token tile
    uint32_t left = M > 64 ? 64 : M, bm = left <= 16 ? 16 : left <= 32 ? 32 : 64;
    uint32_t red = RW < 4 ? 256 * bm * RT : 0;     // the K-slices' reduction buffer comes first
    return ((77824 - red) / bm - 32) / 276;
}
static int check_gemm_q8k(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1], M = c[2], RW = c[4], RT = c[5];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if ((rc = check_block(block, 256))) return rc;
    if (!M || M > 65535) return ojh_fail(OJH_ERR_ARG, "%s: M=%u out of range", s->name, M);
    if (RW != 1 && RW != 2 && RW != 4) return ojh_fail(OJH_ERR_ARG, "%s: RW=%u must be 1, 2 or 4", s->name, RW);
    if (RT != 1) return ojh_fail(OJH_ERR_ARG, "%s: RT=%u: only one row tile per wave is built", s->name, RT);
    const uint32_t fit = ojh_gemm_q8k_fit(M, RW, RT);
    if (K / 256 > fit && fit < 4 / RW)
        return ojh_fail(OJH_ERR_ARG, "%s: RW=%u leaves %u waves on K but only %u super-blocks of %u tokens fit in LDS", s->name,
                        RW, 4 / RW, fit, M > 64 ? 64 : M);
    const uint32_t groups = (N + 16 * RW * RT - 1) / (16 * RW * RT);
    if (!grid[0] || grid[0] > groups || grid[1] != (M + 63) / 64 || grid[2] != 1)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [1 .. ceil(N / (16 RW RT)), ceil(M / 64), 1]", s->name);
    need[0] = (size_t)M * K;
    need[1] = (size_t)M * (K / 256) * 4;
    need[2] = (size_t)N * (K / 256) * 144;
    need[3] = (size_t)M * N * 4;
    align[1] = 4;
    align[3] = 4;
    return OJH_OK;
}
// Row tiles per workgroup (RW side by side, RT = 1 per wave): as many side by side as still give every CU a
// workgroup and a half (measured on 14336 x 4096 and 4096 x 4096), at least what the LDS chunk asks for.
void ojh_gemm_q8k_tiles(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M, uint32_t *rw_out, uint32_t *rt_out) {
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
    const uint64_t tiles_m = (M + 63) / 64;
    uint32_t rw = 4;
    for (;;) {
        const uint32_t fit = ojh_gemm_q8k_fit(M, rw, 1);
        const bool ok = K / 256 <= fit || fit >= 4 / rw;
        const bool enough = (uint64_t)((N + 16 * rw - 1) / (16 * rw)) * tiles_m * 2 >= 3ull * cus;
        if (rw == 1 || (ok && enough)) break;
        // fewer rows per workgroup only if the chunk still feeds the extra waves on K
        const uint32_t fit2 = ojh_gemm_q8k_fit(M, rw / 2, 1);
        if (!(K / 256 <= fit2 || fit2 >= 4 / (rw / 2))) break;
        rw /= 2;
    }
    *rw_out = rw;
    *rt_out = 1;
}
// q8k_token_sides(xq, xs, xst, sums, K, M, MP): grid [K / 256, ceil(MP / 256), 1] x 256
// gemm_q8k_q4k_xt(xq, xst, sums, w, y, K, N, M, ACC, MP): grid [ceil(N / 128), MP / 128, 1] x 512; MP = M rounded up to 128
static int check_gemm_q8k_xt(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    const bool sides = s->rows_per_wave == 0;
    const uint32_t K = c[0], N = sides ? 1 : c[1], M = sides ? c[1] : c[2], MP = sides ? c[2] : c[4];
    if (!K || K % 256 || !N || !M) return ojh_fail(OJH_ERR_ARG, "%s: K=%u (a multiple of 256) N=%u M=%u", s->name, K, N, M);
    if (MP != (M + 127) / 128 * 128) return ojh_fail(OJH_ERR_ARG, "%s: MP=%u must be M=%u rounded up to 128", s->name, MP, M);
    if ((uint64_t)M * K > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: M*K exceeds 2^32 activations", s->name);
    const size_t nsb = K / 256;
    int rc;
    if (sides) {
        if ((rc = check_block(block, 256))) return rc;
        if (grid[0] != nsb || grid[1] != (MP + 255) / 256 || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%zu,%u,1]", s->name, nsb, (MP + 255) / 256);
        need[0] = (size_t)M * K;
        need[1] = (size_t)M * nsb * 4;
        need[2] = nsb * MP * 4;
        need[3] = nsb * MP * 32;
        align[1] = align[2] = 4;
        return OJH_OK;
    }
    if (c[3] > 1) return ojh_fail(OJH_ERR_ARG, "%s: ACC=%u", s->name, c[3]);
    if ((rc = check_block(block, 512))) return rc;
    const uint32_t br = s->rows_per_wave == 2 ? 64 : 128;
    if (grid[0] != (N + br - 1) / br || grid[1] != MP / 128 || grid[2] != 1)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,1]", s->name, (N + br - 1) / br, MP / 128);
    if ((uint64_t)N * nsb * 144 > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: the weight tensor exceeds 4 GiB", s->name);
    need[0] = (size_t)M * K;
    need[1] = nsb * MP * 4;
    need[2] = nsb * MP * 32;
    need[3] = (size_t)N * nsb * 144;
    need[4] = (size_t)M * N * 4;
    align[1] = align[4] = 4;
    return OJH_OK;
}
// gemm_q8k_q4k_xt64_sr(xq, xst, sums, w, y, part, cnt, K, N, M, ACC, MP, NSPLIT): grid [ceil(N / 64), MP / 128, slices],
// slices = those of NSPLIT that hold a super-block; part: 32 KB per tile and slice; cnt: a zeroed word per tile
static int check_gemm_q8k_xt_sr(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                                const uint32_t block[3], size_t need[16], size_t align[16]) {
    const uint32_t K = c[0], N = c[1], M = c[2], MP = c[4], nsplit = c[5];
    if (!K || K % 256 || !N || !M) return ojh_fail(OJH_ERR_ARG, "%s: K=%u (a multiple of 256) N=%u M=%u", s->name, K, N, M);
    if (MP != (M + 127) / 128 * 128) return ojh_fail(OJH_ERR_ARG, "%s: MP=%u must be M=%u rounded up to 128", s->name, MP, M);
    if ((uint64_t)M * K > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: M*K exceeds 2^32 activations", s->name);
    if (c[3] > 1) return ojh_fail(OJH_ERR_ARG, "%s: ACC=%u", s->name, c[3]);
    const size_t nsb = K / 256;
    if (!nsplit || nsplit > nsb) return ojh_fail(OJH_ERR_ARG, "%s: NSPLIT=%u (1 .. K/256)", s->name, nsplit);
    int rc;
    if ((rc = check_block(block, 512))) return rc;
    const uint32_t slices = ojh_gemm_sr_slices(K, nsplit);
    if (grid[0] != (N + 63) / 64 || grid[1] != MP / 128 || grid[2] != slices)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,%u]", s->name, (N + 63) / 64, MP / 128, slices);
    if ((uint64_t)N * nsb * 144 > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: the weight tensor exceeds 4 GiB", s->name);
    const size_t tiles = (size_t)grid[0] * grid[1];
    need[0] = (size_t)M * K;
    need[1] = nsb * MP * 4;
    need[2] = nsb * MP * 32;
    need[3] = (size_t)N * nsb * 144;
    need[4] = (size_t)M * N * 4;
    need[5] = tiles * slices * 32768;
    need[6] = tiles * 4;
    align[1] = align[4] = align[6] = 4;
    align[5] = 8;
    return OJH_OK;
}
static int shape_gemm_q8k_xt_sr(const ojh_kernel_spec *, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                                uint32_t grid[3], uint32_t block[3]) {
    if (!M) M = 1;
    grid[0] = (N + 63) / 64;
    grid[1] = (M + 127) / 128;
    if (!grid[0]) grid[0] = 1;
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, nsb = K / 256;
    uint32_t z = (cus + grid[0] * grid[1] - 1) / (grid[0] * grid[1]);
    if (z > nsb / 2) z = nsb / 2;
    if (z > 8) z = 8;
    if (z < 1) z = 1;
    grid[2] = ojh_gemm_sr_slices(K, z);
    block[0] = 512;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// Family "gemv_q8": row-int8 weights (K int8 per row, one f32 scale per row) against f32 activations, the reference's
// own names and argument order (crates/ojas-cuda/src/kernels/gemv_q8.rs:48-152).  `rows_per_wave` tells the entries apart:
//   0 gemv_q8 / gemv_q8_accum(x, w, y, scale, K, N)       2 gemv_q8_bias(x, w, y, scale, bias, K, N)
//   3 gemv_q8_ksplit(x, w, y, scale, K, N): grid [N]      4 ffn_gu_q8(x, wg, wu, out, sg, su, K, N, act)
//   5 qkv_q8(x, wq, wk, wv, yq, yk, yv, sq, sk, sv, bq, bk, bv, K, Nq, Nkv): the three biases may be NULL
//   6 embed_q8(table, scale, out, token, D)               7 quantize_q8_pertoken(x, q8, d8, K): grid [M]
static int check_gemv_q8(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                         const uint32_t block[3], size_t need[16], size_t align[16]) {
    const int kind = s->rows_per_wave;
    if (grid[1] != 1 || grid[2] != 1 || !grid[0]) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    const uint32_t bmax = kind >= 6 ? 256u : 1024u;
    if (block[1] != 1 || block[2] != 1 || !block[0] || block[0] % 64 || block[0] > bmax)
        return ojh_fail(OJH_ERR_ARG, "%s: block must be [64 .. %u in whole waves,1,1]", s->name, bmax);
    if (kind == 6) {
        const size_t token = c[0], D = c[1];
        if (!D) return ojh_fail(OJH_ERR_ARG, "%s: D=0", s->name);
        need[0] = (token + 1) * D;
        need[1] = (token + 1) * 4;
        need[2] = D * 4;
        align[0] = 1;
        align[1] = align[2] = 4;
        return OJH_OK;
    }
    const size_t K = c[0];
    if (kind == 7) {
        if (!K) return ojh_fail(OJH_ERR_ARG, "%s: K=0", s->name);
        const size_t M = grid[0];
        need[0] = M * K * 4;
        need[1] = M * K;
        need[2] = M * 4;
        align[0] = align[2] = 4;
        align[1] = 1;
        return OJH_OK;
    }
    if (!K || K % 4) return ojh_fail(OJH_ERR_ARG, "%s: K=%zu must be a positive multiple of 4", s->name, K);
    const size_t wa = K % 16 ? 4 : 16;
    need[0] = K * 4;
    if (kind == 5) {
        const size_t Nq = c[1], Nkv = c[2];
        if (!Nq || !Nkv) return ojh_fail(OJH_ERR_ARG, "%s: Nq=%zu Nkv=%zu", s->name, Nq, Nkv);
        for (int i = 0; i < 3; i++) {
            const size_t n = i ? Nkv : Nq;
            need[1 + i] = n * K;
            align[1 + i] = wa;
            need[4 + i] = need[7 + i] = need[10 + i] = n * 4;
            align[4 + i] = align[7 + i] = 4;
            align[10 + i] = 0;                  // 0: the buffer may be NULL (4-byte aligned when given)
        }
        return OJH_OK;
    }
    const size_t N = c[1];
    if (!N) return ojh_fail(OJH_ERR_ARG, "%s: N=0", s->name);
    if (kind == 3 && grid[0] != N) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [N,1,1]", s->name);
    if (kind == 4) {
        if (c[2] > 1) return ojh_fail(OJH_ERR_ARG, "%s: act=%u (0 SiLU, 1 GELU)", s->name, c[2]);
        need[1] = need[2] = N * K;
        align[1] = align[2] = wa;
        need[3] = need[4] = need[5] = N * 4;
        align[3] = align[4] = align[5] = 4;
        return OJH_OK;
    }
    need[1] = N * K;
    align[1] = wa;
    need[2] = need[3] = N * 4;
    align[2] = align[3] = 4;
    if (kind == 2) { need[4] = N * 4; align[4] = 4; }
    return OJH_OK;
}
// rows grid-stride: four workgroups per CU at most (the activations are staged once per workgroup)
static int shape_gemv_q8(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                         uint32_t grid[3], uint32_t block[3]) {
    const int kind = s->rows_per_wave;
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
    block[0] = 256;
    block[1] = block[2] = grid[1] = grid[2] = 1;
    if (kind == 3) { grid[0] = N ? N : 1; block[0] = K >= 8192 ? 512 : 256; return OJH_OK; }
    if (kind == 7) { grid[0] = M ? M : 1; return OJH_OK; }
    if (kind == 6) { grid[0] = (N + 255) / 256 ? (N + 255) / 256 : 1; return OJH_OK; }   // N: the row length D
    // Up to two workgroups per CU (each stages the activations in 64 KB of LDS), as many waves in each as the rows give
    // work for: a wave takes two rows (one output of ffn_gu_q8) per pass.
    const uint32_t per_wave = kind == 4 ? 1 : 2;
    // (measured, K = 4096: 4096 rows 256 threads x 512 workgroups 6.2 us against 7.3 for 512 x 256; 14336 rows 1024 x 448
    // 14.9 against 17.1 for 256 x 512; 128256 rows 1024 x 256 96.6 us = 5.4 TB/s against 125 for 256 x 512)
    uint32_t waves = 4;
    while (waves < 16 && (uint64_t)2 * cus * waves * per_wave < N) waves *= 2;
    block[0] = 64 * waves;
    uint32_t g = (N + waves * per_wave - 1) / (waves * per_wave);
    if (g > 2 * cus) g = cus;                 // several passes: one large workgroup per CU
    grid[0] = g ? g : 1;
    return OJH_OK;
}
// gemm_q8k_{q6k,q5k}_gs(xq, xs, w, y, K, N, M, ACC): grid [ceil(N / 128), ceil(M / 64), 1] x 256
// gemm_q8k_{q6k,q5k}_gs_sr(xq, xs, w, y, part, cnt, K, N, M, ACC, NSPLIT): grid [.., .., slices]; part: 32 KB per tile
// and slice; cnt: a zeroed word per tile (`rows_per_wave` = 1 marks the sliced entries)
static int check_gemm_q8k_gs(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    const bool sr = s->rows_per_wave & 1;
    const uint32_t br = 128, bt = 64;
    const ojh_block_format *f;
    const uint32_t K = c[0], N = c[1], M = c[2], nsplit = sr ? c[4] : 1;
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if (K % 256) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a multiple of 256", s->name, K);
    if (!M || M > 65535) return ojh_fail(OJH_ERR_ARG, "%s: M=%u out of range", s->name, M);
    if (c[3] > 1) return ojh_fail(OJH_ERR_ARG, "%s: ACC=%u", s->name, c[3]);
    if ((rc = check_block(block, 256))) return rc;
    const size_t nsb = K / 256;
    if (!nsplit || nsplit > nsb) return ojh_fail(OJH_ERR_ARG, "%s: NSPLIT=%u (1 .. K/256)", s->name, nsplit);
    const uint32_t slices = sr ? ojh_gemm_sr_slices(K, nsplit) : 1;
    if (grid[0] != (N + br - 1) / br || grid[1] != (M + bt - 1) / bt || grid[2] != slices)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,%u]", s->name, (N + br - 1) / br, (M + bt - 1) / bt, slices);
    need[0] = (size_t)M * K;
    need[1] = (size_t)M * nsb * 4;
    need[2] = (size_t)N * nsb * f->bytes;
    need[3] = (size_t)M * N * 4;
    align[0] = 16;
    align[1] = align[3] = 4;
    align[2] = s->type == OJH_Q5_K ? 16 : 2;
    if (sr) {
        const size_t tiles = (size_t)grid[0] * grid[1];
        need[4] = tiles * slices * 32768;
        need[5] = tiles * 4;
        align[4] = 8;
        align[5] = 4;
    }
    return OJH_OK;
}
// K slices of that tile: two workgroups per CU is the aim (a wave alone on its SIMD waits for every matrix result and
// LDS read itself), at most eight slices of at least two super-blocks — eight, where the tiles already cover more than
// half the CUs.  OJAS_HIP_KQ_GS_SPLIT: 0 never, n > 1 that many.
uint32_t ojh_gemm_q8k_gs_slices(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M) {
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, nsb = K / 256;
    const uint32_t mode = dev ? dev->kq_gs_split : 1u;
    const uint32_t br = 128, bt = 64;
    const uint64_t tiles = (uint64_t)((N + br - 1) / br) * ((M + bt - 1) / bt);
    if (!tiles || mode == 0) return 1;
    uint32_t z = (uint32_t)(2 * (uint64_t)cus / tiles);
    if (z > 8) z = 8;
    const uint32_t cap = tiles * 2 > cus ? nsb / 8 : nsb / 2;
    if (z > cap) z = cap;
    if (mode > 1) z = mode <= nsb ? mode : nsb;
    return z < 2 ? 1 : ojh_gemm_sr_slices(K, z);
}
static int shape_gemm_q8k_gs(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                             uint32_t grid[3], uint32_t block[3]) {
    if (!M) M = 1;
    grid[0] = (N + 127) / 128;
    if (!grid[0]) grid[0] = 1;
    grid[1] = (M + 63) / 64;
    grid[2] = s->rows_per_wave & 1 ? ojh_gemm_q8k_gs_slices(dev, K, N, M) : 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// quantize_q8k{,_bf16}_sides(x, q, scales, xst, sums, K, M, MP): grid [K / 256 * MP / 4, 1, 1]
static int check_quantize_sides(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                                const uint32_t block[3], size_t need[16], size_t align[16]) {
    const uint32_t K = c[0], M = c[1], MP = c[2];
    if (!K || K % 256 || !M) return ojh_fail(OJH_ERR_ARG, "%s: K=%u (a multiple of 256) M=%u", s->name, K, M);
    if (MP != (M + 127) / 128 * 128) return ojh_fail(OJH_ERR_ARG, "%s: MP=%u must be M=%u rounded up to 128", s->name, MP, M);
    if ((uint64_t)M * K > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: M*K exceeds 2^32 activations", s->name);
    int rc = check_block(block, 256);
    if (rc) return rc;
    const size_t nsb = K / 256, esz = strstr(s->name, "bf16") ? 2 : 4;
    if ((uint64_t)nsb * MP / 4 > 0x7FFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: too many segments for one launch", s->name);
    if (grid[0] != nsb * MP / 4 || grid[1] != 1 || grid[2] != 1)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%zu,1,1]", s->name, nsb * MP / 4);
    need[0] = (size_t)M * K * esz;
    need[1] = (size_t)M * K;
    need[2] = (size_t)M * nsb * 4;
    need[3] = nsb * MP * 4;
    need[4] = nsb * MP * 32;
    align[0] = 4 * esz;
    align[1] = align[2] = align[3] = 4;
    return OJH_OK;
}
static int shape_quantize_sides(const ojh_kernel_spec *, const ojh_device *, uint32_t K, uint32_t, uint32_t M,
                                uint32_t grid[3], uint32_t block[3]) {
    if (!M) M = 1;
    grid[0] = (K / 256 ? K / 256 : 1) * ((M + 127) / 128 * 32);
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
static int shape_gemm_q8k_xt(const ojh_kernel_spec *s, const ojh_device *, uint32_t K, uint32_t N, uint32_t M,
                             uint32_t grid[3], uint32_t block[3]) {
    if (!M) M = 1;
    const uint32_t MP = (M + 127) / 128 * 128;
    if (s->rows_per_wave == 0) { grid[0] = K / 256; grid[1] = (MP + 255) / 256; block[0] = 256; }
    else { const uint32_t br = s->rows_per_wave == 2 ? 64 : 128; grid[0] = (N + br - 1) / br; grid[1] = MP / 128; block[0] = 512; }
    if (!grid[0]) grid[0] = 1;
    grid[2] = 1;
    block[1] = block[2] = 1;
    return OJH_OK;
}
static int shape_gemm_q8k(const ojh_kernel_spec *, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                          uint32_t grid[3], uint32_t block[3]) {
    if (!M) M = 1;
    uint32_t rw, rt;
    ojh_gemm_q8k_tiles(dev, K, N, M, &rw, &rt);
    grid[0] = (N + 16 * rw * rt - 1) / (16 * rw * rt);
    grid[1] = (M + 63) / 64;
    grid[2] = 1;
    // the whole K staged once: row groups grid-stride over two workgroups per CU
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
    if (K / 256 <= ojh_gemm_q8k_fit(M, rw, rt) && grid[0] * grid[1] > 2 * cus) {
        uint32_t gx = 2 * cus / grid[1];
        grid[0] = gx ? gx : 1;
    }
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// one 512-thread workgroup per CU (all of its LDS), a 16-row tile per workgroup step
static int shape_mk(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                    uint32_t grid[3], uint32_t block[3]) {
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, tiles = (N + 15) / 16;
    grid[0] = tiles < cus ? tiles : cus;
    grid[1] = grid[2] = 1;
    block[0] = 512;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// one 512-thread workgroup per CU (all of its LDS), 16-row tiles grid-stride over the waves
static int shape_ml(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                    uint32_t grid[3], uint32_t block[3]) {
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, wgs = (N + 127) / 128;
    grid[0] = wgs < cus ? wgs : cus;
    grid[1] = grid[2] = 1;
    block[0] = 512;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// gemm_q8k_q4k_ml(xq, xs, w, y, K, N, M, ACC): up to 16 tokens, each wave's rows copied through its own LDS ring.
// LDS: 16 token rows, their scales and split sums, eight rings of four 2304-byte units.
uint64_t ojh_gemm_q8k_ml_lds(uint32_t K) { return 16 * ((uint64_t)K + 32) + K / 4 + K + 256 + 8 * 4 * 2304; }
// gemm_q8k_q4k_mk: M token rows, scales, split sums, a zero block, eight waves' partial sums
uint64_t ojh_gemm_q8k_mk_lds(uint32_t K, uint32_t M) { return (uint64_t)M * ((uint64_t)K + 32) + K / 4 + K + 256 + 8192; }
static int check_gemm_q8k_ml(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1], M = c[2];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    const bool mk = s->rows_per_wave == 2;      // gemm_q8k_q4k_mk: a tile per workgroup, K split over its eight waves
    if (mk ? (rc = check_block(block, 512)) != 0 : block[1] != 1 || block[2] != 1 || !block[0] || block[0] % 64 || block[0] > 512)
        return mk ? rc : ojh_fail(OJH_ERR_ARG, "%s: block must be [64 .. 512 in whole waves,1,1], got [%u,%u,%u]", s->name, block[0], block[1], block[2]);
    if (grid[1] != 1 || grid[2] != 1 || !grid[0]) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1], x > 0", s->name);
    const uint64_t lds = mk ? ojh_gemm_q8k_mk_lds(K, M) : ojh_gemm_q8k_ml_lds(K);
    if (!M || M > 16 || lds > 163840)
        return ojh_fail(OJH_ERR_ARG, "%s: M=%u tokens of K=%u do not fit its 160 KB of LDS (1 <= M <= 16, %llu bytes needed)", s->name,
                        M, K, (unsigned long long)lds);
    if (!mk && (uint64_t)N * (K / 256) * 144 > 0xFFFFFFFFull)
        return ojh_fail(OJH_ERR_ARG, "%s: %u rows of K=%u pass 4 GiB, the reach of its 32-bit row offsets", s->name, N, K);
    need[0] = (size_t)M * K;
    need[1] = (size_t)M * (K / 256) * 4;
    need[2] = (size_t)N * (K / 256) * 144;
    need[3] = (size_t)M * N * 4;
    align[0] = 16;
    align[1] = 4;
    align[2] = 16;
    align[3] = 4;
    return OJH_OK;
}

// gemv_q8k_q6k_px(xq, xs, w, y, K, N): rows grid-stride, activations in registers (K <= 8192)
static int check_gemv_q8k_px(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if ((rc = check_block(block, 256))) return rc;
    if (K > 8192) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: K=%u exceeds the 8192 activations a wave keeps in registers", s->name, K);
    if (!grid[0] || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1], x > 0", s->name);
    need[0] = (size_t)K;
    need[1] = (size_t)(K / 256) * 4;
    need[2] = (size_t)N * (K / f->weights) * f->bytes;
    need[3] = (size_t)N * 4;
    align[1] = 4;
    align[2] = ojh_block_align(f);
    align[3] = 4;
    return OJH_OK;
}
// gemv_nat_{q4k,q6k,iq4nl,iq4xs}_px(x, w, y, K, N): rows grid-stride, two per wave and step, f32 activations in registers
static int check_gemv_nat_px(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if ((rc = check_block(block, 256))) return rc;
    if (K > 4096) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: K=%u exceeds the 4096 activations a wave keeps in registers", s->name, K);
    if (!grid[0] || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1], x > 0", s->name);
    need[0] = (size_t)K * 4;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)N * 4;
    align[1] = ojh_block_align(f);
    align[2] = 4;
    return OJH_OK;
}
static int shape_px(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                    uint32_t grid[3], uint32_t block[3]) {
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, cover = (N + 7) / 8;
    uint32_t bpc = dev && dev->px_bpc ? dev->px_bpc : 8u;
    grid[0] = cover < bpc * cus ? cover : bpc * cus;   // a whole multiple of the CU count
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// gemv_q8k_<fmt>{,_accum,_bias,_rN}(xq, xs, w, y[, bs], K, N)
static int check_gemv_q8k(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if ((rc = check_block(block, 0))) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    uint64_t cover = (uint64_t)grid[0] * (block[0] / 64) * s->rows_per_wave;
    if (cover < N) return ojh_fail(OJH_ERR_ARG, "%s: grid covers %llu rows of N=%u", s->name,
                                   (unsigned long long)cover, N);
    need[0] = (size_t)K;
    need[1] = (size_t)(K / 256) * 4;
    need[2] = (size_t)N * (K / f->weights) * f->bytes;
    need[3] = (size_t)N * 4;
    if (s->n_bufs == 5) need[4] = (size_t)N * 4;
    align[1] = 4;
    align[2] = ojh_block_align(f);
    align[3] = align[4] = 4;
    return OJH_OK;
}

// gemv_q8k_<fmt>_x4_{r1,r2}(xq, xs, w0..w3, y0..y3, K, E0..E3): up to four tensors, one activation;
// E are running row totals (non-decreasing; a tensor with no rows still needs a valid pointer)
static int check_gemv_q8k_x4(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], E[4] = {c[1], c[2], c[3], c[4]};
    int rc = check_kn(s, K, E[3], &f);
    if (rc) return rc;
    if ((rc = check_block(block, 0))) return rc;
    if (E[0] > E[1] || E[1] > E[2] || E[2] > E[3])
        return ojh_fail(OJH_ERR_ARG, "%s: row totals %u,%u,%u,%u must not decrease", s->name, E[0], E[1], E[2], E[3]);
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    uint64_t cover = (uint64_t)grid[0] * (block[0] / 64) * s->rows_per_wave;
    if (cover < E[3]) return ojh_fail(OJH_ERR_ARG, "%s: grid covers %llu rows of N=%u", s->name,
                                      (unsigned long long)cover, E[3]);
    need[0] = (size_t)K;
    need[1] = (size_t)(K / 256) * 4;
    align[1] = 4;
    for (int i = 0; i < 4; i++) {
        size_t rows = E[i] - (i ? E[i - 1] : 0);
        need[2 + i] = rows * (K / f->weights) * f->bytes;
        need[6 + i] = rows * 4;
        align[2 + i] = ojh_block_align(f);
        align[6 + i] = 4;
    }
    return OJH_OK;
}

// The same launches with a GGUF type per tensor (a byte each of the last constant): Q4_K, Q5_K or Q6_K.
static const ojh_block_format *kq_type(const ojh_kernel_spec *s, uint32_t t, int which) {
    if (t != OJH_Q4_K && t != OJH_Q5_K && t != OJH_Q6_K) {
        ojh_fail(OJH_ERR_UNSUPPORTED, "%s: tensor %d has GGUF type %u; takes Q4_K (12), Q5_K (13) or Q6_K (14)", s->name, which, t);
        return nullptr;
    }
    return ojh_format(t);
}
static int check_gemv_q8k_kq_x4(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                                const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t K = c[0], E[4] = {c[1], c[2], c[3], c[4]}, T = c[5];
    if (K == 0 || K % 256) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a positive multiple of 256", s->name, K);
    int rc;
    if ((rc = check_block(block, 0))) return rc;
    if (E[0] > E[1] || E[1] > E[2] || E[2] > E[3] || E[3] == 0)
        return ojh_fail(OJH_ERR_ARG, "%s: row totals %u,%u,%u,%u must not decrease", s->name, E[0], E[1], E[2], E[3]);
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * (block[0] / 64) < E[3])
        return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover N=%u rows", s->name, E[3]);
    need[0] = (size_t)K;
    need[1] = (size_t)(K / 256) * 4;
    align[1] = 4;
    for (int i = 0; i < 4; i++) {
        const ojh_block_format *f = kq_type(s, (T >> (8 * i)) & 0xFFu, i);
        if (!f) return OJH_ERR_UNSUPPORTED;
        size_t rows = E[i] - (i ? E[i - 1] : 0);
        need[2 + i] = rows * (K / 256) * f->bytes;
        need[6 + i] = rows * 4;
        align[2 + i] = ojh_block_align(f);
        align[6 + i] = 4;
    }
    return OJH_OK;
}
static int check_ffn_gu_kq(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                           const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t K = c[0], N = c[1], ACT = c[2], T = c[3];
    if (K == 0 || K % 256 || N == 0) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a positive multiple of 256, N=%u positive", s->name, K, N);
    if (ACT > 1) return ojh_fail(OJH_ERR_ARG, "%s: ACT=%u (0 = SiLU, 1 = GELU)", s->name, ACT);
    if (T >> 16) return ojh_fail(OJH_ERR_ARG, "%s: TYPES=%#x carries two type bytes", s->name, T);
    int rc;
    if ((rc = check_block(block, 0))) return rc;
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * (block[0] / 64) < N)
        return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover N=%u rows", s->name, N);
    const ojh_block_format *fg = kq_type(s, T & 0xFFu, 0), *fu = kq_type(s, (T >> 8) & 0xFFu, 1);
    if (!fg || !fu) return OJH_ERR_UNSUPPORTED;
    need[0] = (size_t)K;
    need[1] = (size_t)(K / 256) * 4;
    need[2] = (size_t)N * (K / 256) * fg->bytes;
    need[3] = (size_t)N * (K / 256) * fu->bytes;
    need[4] = (size_t)N * 4;
    align[1] = align[4] = 4;
    align[2] = ojh_block_align(fg);
    align[3] = ojh_block_align(fu);
    return OJH_OK;
}

// ffn_gu_q8k_<fmt>(xq, xs, wg, wu, out, K, N, ACT): one wave per row
static int check_ffn_gu(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                        const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1], ACT = c[2];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if (ACT > 1) return ojh_fail(OJH_ERR_ARG, "%s: ACT=%u (0 = SiLU, 1 = GELU)", s->name, ACT);
    if ((rc = check_block(block, 0))) return rc;
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * (block[0] / 64) * s->rows_per_wave < N)
        return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover N=%u rows", s->name, N);
    need[0] = (size_t)K;
    need[1] = (size_t)(K / 256) * 4;
    need[2] = need[3] = (size_t)N * (K / f->weights) * f->bytes;
    need[4] = (size_t)N * 4;
    align[1] = align[4] = 4;
    return OJH_OK;
}

// rmsnorm_q8k(x, gamma, q, scales, xn, K, M, EPS_BITS, WRITE_XN): grid [M,1,1] x 256
static int check_rmsnorm_q8k(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t K = c[0], M = c[1], WR = c[3];
    if (!K || !M || K > 16384) return ojh_fail(OJH_ERR_ARG, "%s: K=%u (1..16384) M=%u", s->name, K, M);
    int rc = check_block(block, block[0] == 1024 ? 1024 : 256);     // four or sixteen waves: the same bits
    if (rc) return rc;
    if (grid[0] != M || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,1,1]", s->name, M);
    uint32_t nsb = (K + 255) / 256;
    need[0] = (size_t)M * K * 4;
    need[1] = (size_t)K * 4;
    need[2] = (size_t)M * nsb * 256;
    need[3] = (size_t)M * nsb * 4;
    need[4] = WR ? (size_t)M * K * 4 : 0;
    align[0] = align[1] = align[3] = align[4] = 4;
    return OJH_OK;
}
static int shape_rmsnorm(const ojh_kernel_spec *, const ojh_device *, uint32_t, uint32_t, uint32_t M,
                         uint32_t grid[3], uint32_t block[3]) {
    grid[0] = M ? M : 1;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// gemv_fq8k_<fmt>_{r1,r2,wide}(x, w, y, K, N, NRB): quantizer folded in; 4 waves per block,
// K <= 16384, NRB rows per block (a multiple of 4 * rows per wave)
static int check_gemv_fq8k(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                           const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1], NRB = c[2];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if ((rc = check_block(block, 256))) return rc;
    if (K > 16384) return ojh_fail(OJH_ERR_ARG, "%s: K=%u exceeds 16384", s->name, K);
    uint32_t unit = 4u * (uint32_t)s->rows_per_wave;
    if (!NRB || NRB % unit) return ojh_fail(OJH_ERR_ARG, "%s: NRB=%u must be a positive multiple of %u", s->name, NRB, unit);
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * NRB < N)
        return ojh_fail(OJH_ERR_ARG, "%s: grid x NRB does not cover N=%u rows", s->name, N);
    need[0] = (size_t)K * 4;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)N * 4;
    align[2] = 4;
    return OJH_OK;
}

// gemv_fq8k_<fmt>_x4_{r1,r2}(x, w0..w3, y0..y3, K, E0..E3, NRB, ACC): the folded quantizer over up to four tensors
static int check_gemv_fq8k_x4(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                              const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], E[4] = {c[1], c[2], c[3], c[4]}, NRB = c[5], ACC = c[6];
    int rc = check_kn(s, K, E[3], &f);
    if (rc) return rc;
    if ((rc = check_block(block, 0))) return rc;
    if (block[0] > 1024) return ojh_fail(OJH_ERR_ARG, "%s: at most 1024 threads per workgroup", s->name);
    if (K > 16384) return ojh_fail(OJH_ERR_ARG, "%s: K=%u exceeds 16384", s->name, K);
    if (ACC > 1) return ojh_fail(OJH_ERR_ARG, "%s: ACC=%u", s->name, ACC);
    if (E[0] > E[1] || E[1] > E[2] || E[2] > E[3])
        return ojh_fail(OJH_ERR_ARG, "%s: row totals %u,%u,%u,%u must not decrease", s->name, E[0], E[1], E[2], E[3]);
    if (!NRB) return ojh_fail(OJH_ERR_ARG, "%s: NRB must be positive", s->name);
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * NRB < E[3])
        return ojh_fail(OJH_ERR_ARG, "%s: grid x NRB does not cover N=%u rows", s->name, E[3]);
    need[0] = (size_t)K * 4;
    for (int i = 0; i < 4; i++) {
        size_t rows = E[i] - (i ? E[i - 1] : 0);
        need[1 + i] = rows * (K / f->weights) * f->bytes;
        need[5 + i] = rows * 4;
        align[1 + i] = ojh_block_align(f);
        align[5 + i] = 4;
    }
    return OJH_OK;
}

// gemv_nat_<fmt>_m(x, w, y, K, N, M, ACC)
static int check_gemv_nat_m(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                            const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1], M = c[2];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if (M == 0) return ojh_fail(OJH_ERR_ARG, "%s: M must be positive", s->name);
    if ((rc = check_block(block, 0))) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    if ((uint64_t)grid[0] * (block[0] / 64) < N)
        return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover N=%u rows", s->name, N);
    need[0] = (size_t)M * K * 4;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)M * N * 4;
    align[1] = ojh_block_align(f);
    align[2] = 4;
    return OJH_OK;
}

// LDS of gemv_q8k_q6k_mk: token rows, their scales, a zero region, eight waves' partial sums
uint64_t ojh_q6k_mk_lds(uint32_t K, uint32_t M) {
    const uint64_t p = M <= 8 ? 1 : 2;
    return 8 * p * ((uint64_t)K + 32) + K / 4 + 256 + 4096 * p;
}
// least LDS of gemv_q8k_q6k_ml: token rows, their scales, eight waves' copy rings (3 units deep up to 8 tokens, 2
// beyond; the kernel takes one more where it fits)
uint64_t ojh_q6k_ml_lds(uint32_t K, uint32_t M) {
    const uint64_t p = M <= 8 ? 1 : 2;
    return 8 * p * ((uint64_t)K + 32) + K / 4 + 256 + 8 * (p == 1 ? 3 : 2) * 3616;
}

// gemv_q8k_<fmt>_m(xq, xs, w, y, K, N, M, ACC)
static int check_gemv_q8k_m(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                            const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    uint32_t K = c[0], N = c[1], M = c[2];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if (M == 0) return ojh_fail(OJH_ERR_ARG, "%s: M must be positive", s->name);
    const bool mx = s->rows_per_wave == 0;   // the LDS-staged, grid-stride entry
    const bool mf = s->rows_per_wave == -1;  // the same on the int8 matrix cores
    const bool ml = s->rows_per_wave == -2;  // ... with the rows copied through LDS
    const bool mk = s->rows_per_wave == -3;  // ... with a tile's super-blocks split over eight waves
    if (ml) {   // one to eight waves, each with its own copy ring
        if (block[1] != 1 || block[2] != 1 || !block[0] || block[0] % 64 || block[0] > 512)
            return ojh_fail(OJH_ERR_ARG, "%s: block must be [64 .. 512 in whole waves,1,1], got [%u,%u,%u]", s->name, block[0], block[1], block[2]);
    } else if ((rc = check_block(block, mk ? 512 : mx || mf ? 256 : 0))) return rc;
    if (grid[1] != 1 || grid[2] != 1 || !grid[0]) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1], x > 0", s->name);
    if (mk) {
        const uint64_t lds = ojh_q6k_mk_lds(K, M);
        if (M > 16 || lds > 163840)
            return ojh_fail(OJH_ERR_ARG, "%s: M=%u tokens of K=%u do not fit its 160 KB of LDS (M <= 16, %llu bytes needed)",
                            s->name, M, K, (unsigned long long)lds);
    } else if (mf) {
        const uint64_t lds = (uint64_t)(M <= 8 ? 8 : 16) * (K + 32) + K / 4 + 256;
        if (M > 16 || lds > 69632)
            return ojh_fail(OJH_ERR_ARG, "%s: M=%u tokens of K=%u do not fit its 68 KB of LDS (M <= 16, %llu bytes needed)",
                            s->name, M, K, (unsigned long long)lds);
    } else if (ml) {
        const uint64_t lds = ojh_q6k_ml_lds(K, M);
        if (M > 16 || lds > 163840)
            return ojh_fail(OJH_ERR_ARG, "%s: M=%u tokens of K=%u do not fit its 160 KB of LDS (M <= 16, %llu bytes needed)",
                            s->name, M, K, (unsigned long long)lds);
        if ((uint64_t)N * (K / 256) * 210 > 0xFFFFFFFFull)
            return ojh_fail(OJH_ERR_ARG, "%s: %u rows of K=%u pass 4 GiB, the reach of its 32-bit row offsets", s->name, N, K);
    } else if (mx) {
        if (M > 16 || (uint64_t)M * ((K + 4095) / 4096) > 19)
            return ojh_fail(OJH_ERR_ARG, "%s: M=%u tokens of K=%u do not fit its 80 KB of LDS (M <= 16, M*ceil(K/4096) <= 19)",
                            s->name, M, K);
    } else if ((uint64_t)grid[0] * (block[0] / 64) < N) {
        return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover N=%u rows", s->name, N);
    }
    need[0] = (size_t)M * K;
    need[1] = (size_t)M * (K / 256) * 4;
    need[2] = (size_t)N * (K / f->weights) * f->bytes;
    need[3] = (size_t)M * N * 4;
    align[1] = 4;
    align[2] = ojh_block_align(f);
    align[3] = 4;
    if (mf || mk) {           // whole aligned dwords around every piece: the last one may end 2 bytes on
        need[2] = (need[2] + 3) & ~(size_t)3;
        align[2] = 4;
    }
    if (ml) {                 // whole aligned 16-byte pieces around every super-block
        need[2] = (need[2] + 15) & ~(size_t)15;
        align[2] = 16;
    }
    return OJH_OK;
}

// quantize_q8k{,_bf16}(x, q, scales, K, M)
static int check_quantize(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t K = c[0], M = c[1];
    if (K == 0 || M == 0) return ojh_fail(OJH_ERR_ARG, "%s: K and M must be positive", s->name);
    int rc = check_block(block, 256);
    if (rc) return rc;
    uint32_t nsb = (K + 255) / 256;
    if (s->rows_per_wave == 1) {   // the `_w` entries: a segment per wave, grid [ceil(nsb M / 4),1,1]
        const uint64_t segs = (uint64_t)nsb * M;
        if (segs > 0xFFFFFFFFull || grid[0] != (segs + 3) / 4 || grid[1] != 1 || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%llu,1,1]", s->name, (unsigned long long)((segs + 3) / 4));
    } else if (grid[0] != nsb || grid[1] != M || grid[2] != 1)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,1]", s->name, nsb, M);
    size_t esz = strstr(s->name, "bf16") ? 2 : 4;
    need[0] = (size_t)M * K * esz;
    need[1] = (size_t)M * nsb * 256;
    need[2] = (size_t)M * nsb * 4;
    align[0] = esz;
    align[2] = 4;
    return OJH_OK;
}

// The row-int8 family; `rows_per_wave` selects the entry:
//   0 rows_q8_from_f16(w16, q, scale, K, N)   1 quant_rows_i8(x, q, scale, K, M)       grid [rows,1,1]
//   2 matmul_q8row(xq, sx, wq, sw, y, K, N, M)   3 matmul_q8row_bias(.., y, bs, K, N, M)  grid [ceil(N/4),1,1]
//   4 matmul_q8row_mt(xq, sx, wq, sw, y, bs, K, N, M)                                   grid [ceil(N/128),ceil(M/64),1]
//   5 matmul_q8row_mt_sr(xq, sx, wq, sw, y, bs, part, cnt, K, N, M, NSPLIT)             grid [.., .., slices]
//   6 matmul_q8row_mt128(xq, sx, wq, sw, y, bs, K, N, M)                                grid [ceil(N/128),ceil(M/128),1]
//   7 matmul_q8row_dec(xq, sx, wq, sw, y, bs, K, N, M)     M <= 8, M K <= 64 KB          grid [x,1,1] (rows grid-stride),
//   8 matmul_q8row_dec_l(..)                               M <= 8, M K <= 128 KB         block 64 .. 1024 in whole waves
//     (bs may be NULL; part: tiles x slices x 32 KB; cnt: a zeroed uint per tile)
static int check_rowq8(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                       const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t K = c[0], R = c[1];
    if (!K || !R) return ojh_fail(OJH_ERR_ARG, "%s: K and the row count must be positive", s->name);
    if (s->rows_per_wave >= 7) {
        const uint32_t N = R, M = c[2];
        const size_t lds = s->rows_per_wave == 7 ? 65536 : 131072;
        if (grid[1] != 1 || grid[2] != 1 || !grid[0]) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
        if (block[1] != 1 || block[2] != 1 || !block[0] || block[0] % 64 || block[0] > 1024)
            return ojh_fail(OJH_ERR_ARG, "%s: block must be [64 .. 1024 in whole waves,1,1]", s->name);
        if (!M || M > 8 || K % 16) return ojh_fail(OJH_ERR_ARG, "%s: M=%u (1 .. 8), K=%u a multiple of 16", s->name, M, K);
        if ((size_t)M * K > lds) return ojh_fail(OJH_ERR_ARG, "%s: M K = %zu exceeds the %zu bytes staged", s->name, (size_t)M * K, lds);
        need[0] = (size_t)M * K;
        need[1] = (size_t)M * 4;
        need[2] = (size_t)N * K;
        need[3] = (size_t)N * 4;
        need[4] = (size_t)M * N * 4;
        need[5] = (size_t)N * 4;
        align[0] = align[2] = 16;
        align[1] = align[3] = align[4] = 4;
        align[5] = 0;                               // 0: the buffer may be NULL (4-byte aligned when given)
        return OJH_OK;
    }
    int rc = OJH_OK;
    if (s->rows_per_wave == 1) {
        if (block[1] != 1 || block[2] != 1 || !block[0] || block[0] % 64 || block[0] > 1024)
            return ojh_fail(OJH_ERR_ARG, "%s: block must be [64 .. 1024 in whole waves,1,1]", s->name);
    } else if ((rc = check_block(block, 256))) {
        return rc;
    }
    if (s->rows_per_wave >= 4) {
        const uint32_t N = R, M = c[2];
        if (!M || K % 16) return ojh_fail(OJH_ERR_ARG, "%s: M must be positive and K=%u a multiple of 16", s->name, K);
        const bool sr = s->rows_per_wave == 5;
        const uint32_t nks = (K + 127) / 128, nsplit = sr ? c[3] : 1;
        if (!nsplit || nsplit > nks) return ojh_fail(OJH_ERR_ARG, "%s: NSPLIT=%u of %u steps of 128", s->name, nsplit, nks);
        const uint32_t per = (nks + nsplit - 1) / nsplit, slices = (nks + per - 1) / per;
        const uint32_t bt = s->rows_per_wave == 6 ? 128 : 64;
        const uint32_t gx = (N + 127) / 128, gy = (M + bt - 1) / bt;
        if (gy > 65535) return ojh_fail(OJH_ERR_ARG, "%s: M=%u gives more than 65535 token tiles", s->name, M);
        if (grid[0] != gx || grid[1] != gy || grid[2] != slices)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,%u]", s->name, gx, gy, slices);
        need[0] = (size_t)M * K;
        need[1] = (size_t)M * 4;
        need[2] = (size_t)N * K;
        need[3] = (size_t)N * 4;
        need[4] = (size_t)M * N * 4;
        need[5] = (size_t)N * 4;
        align[0] = align[2] = 16;
        align[1] = align[3] = align[4] = 4;
        align[5] = 0;                               // 0: the buffer may be NULL (4-byte aligned when given)
        if (sr) {
            need[6] = (size_t)gx * gy * slices * 32768;
            need[7] = (size_t)gx * gy * 4;
            align[6] = 8;
            align[7] = 4;
        }
        return OJH_OK;
    }
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    if (s->rows_per_wave < 2) {
        if (grid[0] != R) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,1,1]", s->name, R);
        size_t esz = s->rows_per_wave == 0 ? 2 : 4;
        need[0] = (size_t)R * K * esz;
        need[1] = (size_t)R * K;
        need[2] = (size_t)R * 4;
        align[0] = esz;
        align[1] = 1;
        align[2] = 4;
        return OJH_OK;
    }
    uint32_t N = R, M = c[2];
    if (!M || K % 16) return ojh_fail(OJH_ERR_ARG, "%s: M must be positive and K=%u a multiple of 16", s->name, K);
    if ((uint64_t)grid[0] * 4 < N) return ojh_fail(OJH_ERR_ARG, "%s: grid covers %u rows of N=%u", s->name, grid[0] * 4, N);
    need[0] = (size_t)M * K;
    need[1] = (size_t)M * 4;
    need[2] = (size_t)N * K;
    need[3] = (size_t)N * 4;
    need[4] = (size_t)M * N * 4;
    if (s->n_bufs == 6) need[5] = (size_t)N * 4;
    align[1] = align[3] = align[4] = align[5] = 4;
    return OJH_OK;
}
// K slices of the row-int8 tile: two workgroups per CU is the aim, at most sixteen slices of at least four steps of 128.
// OJAS_HIP_Q8ROW_SPLIT: 0 never, n > 1 that many.
uint32_t ojh_matmul_q8row_slices(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M) {
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, nks = (K + 127) / 128;
    const uint32_t mode = dev ? dev->q8row_split : 1u;
    const uint64_t tiles = (uint64_t)((N + 127) / 128) * ((M + 63) / 64);
    if (!tiles || mode == 0) return 1;
    uint32_t z = (uint32_t)(2 * (uint64_t)cus / tiles);
    if (z > 16) z = 16;
    if (z > nks / 4) z = nks / 4;
    if (mode > 1) z = mode <= nks ? mode : nks;
    if (z < 2) return 1;
    const uint32_t per = (nks + z - 1) / z;
    return (nks + per - 1) / per;
}
static int shape_rowq8(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                       uint32_t grid[3], uint32_t block[3]) {
    grid[0] = s->rows_per_wave == 0 ? N : s->rows_per_wave == 1 ? M : (N + 3) / 4;
    grid[1] = grid[2] = 1;
    if (s->rows_per_wave == 1) {
        // a float4 per thread where the row gives as many (every load in flight at once), sixteen waves at most
        const uint32_t want = (K / 4 + 63) / 64 * 64;
        block[0] = want < 256 ? 256 : want > 1024 ? 1024 : want;
        block[1] = block[2] = 1;
        return OJH_OK;
    }
    if (s->rows_per_wave >= 7) {
        // a wave takes two rows per pass; two workgroups per CU where the staged tokens are small, else one
        const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
        const uint32_t lim = s->rows_per_wave == 7 && (uint64_t)(M ? M : 1) * K <= 16384 ? 2 : 1;
        uint32_t waves = 4;
        while (waves < 16 && (uint64_t)lim * cus * waves * 2 < N) waves *= 2;
        block[0] = 64 * waves;
        block[1] = block[2] = 1;
        uint32_t g = (N + waves * 2 - 1) / (waves * 2);
        if (g > lim * cus) g = cus;
        grid[0] = g ? g : 1;
        return OJH_OK;
    }
    if (s->rows_per_wave >= 4) {
        grid[0] = (N + 127) / 128;
        grid[1] = s->rows_per_wave == 6 ? ((M ? M : 1) + 127) / 128 : ((M ? M : 1) + 63) / 64;
        if (s->rows_per_wave == 5) grid[2] = ojh_matmul_q8row_slices(dev, K, N, M ? M : 1);
    }
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// Family "q80_dp4a" (block_q8_0 rows against activations quantized per 32): `rows_per_wave` selects the entry
//   0 quantize_q8_1(x, q8, d8, d8sum, K)                           grid [ceil(K/256),1,1]
//   1 gemv_q80_dp4a(w, q8, d8, y, K, N)   2 .._bias(+ bias)   3 .._accum    grid [ceil(N/8),1,1]
//   4 qkv_q80_dp4a(wq, wk, wv, q8, d8, q, k, v, bias, K, Nq, Nkv)    grid [ceil((Nq + 2 Nkv)/8),1,1]
//   5 ffn_gu_q80_dp4a(wg, wu, q8, d8, out, K, N, act)               grid [ceil(N/4),1,1]
static int check_q80_dp4a(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    const uint32_t K = c[0];
    if (!K || K % 32) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a positive multiple of 32", s->name, K);
    const size_t nblk = K / 32, rb = nblk * 34;
    uint32_t rows = 0, per = 8;
    switch (s->rows_per_wave) {
    case 0:
        rows = K; per = 256;
        need[0] = (size_t)K * 4; need[1] = K; need[2] = need[3] = nblk * 4;
        align[0] = align[2] = align[3] = 4;
        break;
    case 1: case 2: case 3: {
        const uint32_t N = c[1];
        if (!N) return ojh_fail(OJH_ERR_ARG, "%s: N must be positive", s->name);
        rows = N;
        need[0] = (size_t)N * rb; need[1] = K; need[2] = nblk * 4; need[3] = (size_t)N * 4;
        if (s->rows_per_wave == 2) need[4] = (size_t)N * 4;
        align[0] = 2; align[1] = 8; align[2] = align[3] = align[4] = 4;
        break;
    }
    case 4: {
        const uint32_t Nq = c[1], Nkv = c[2];
        if (!Nq || !Nkv || (uint64_t)Nq + 2ull * Nkv > 0x7FFFFFFFull) return ojh_fail(OJH_ERR_ARG, "%s: Nq=%u Nkv=%u", s->name, Nq, Nkv);
        rows = Nq + 2 * Nkv;
        need[0] = (size_t)Nq * rb; need[1] = need[2] = (size_t)Nkv * rb; need[3] = K; need[4] = nblk * 4;
        need[5] = (size_t)Nq * 4; need[6] = need[7] = (size_t)Nkv * 4; need[8] = (size_t)rows * 4;
        align[0] = align[1] = align[2] = 2; align[3] = 8;
        for (int i = 4; i < 9; i++) align[i] = 4;
        break;
    }
    default: {
        const uint32_t N = c[1], act = c[2];
        if (!N || act > 1) return ojh_fail(OJH_ERR_ARG, "%s: N=%u act=%u", s->name, N, act);
        rows = N; per = 4;
        need[0] = need[1] = (size_t)N * rb; need[2] = K; need[3] = nblk * 4; need[4] = (size_t)N * 4;
        align[0] = align[1] = 2; align[2] = 8; align[3] = align[4] = 4;
        break;
    }
    }
    if ((uint64_t)grid[0] * per < rows || !grid[0])
        return ojh_fail(OJH_ERR_ARG, "%s: grid [%u] x %u does not cover %u", s->name, grid[0], per, rows);
    return OJH_OK;
}
// (K, N, M) = (K, rows — for qkv: Nq + 2 Nkv, -)
static int shape_q80_dp4a(const ojh_kernel_spec *s, const ojh_device *, uint32_t K, uint32_t N, uint32_t,
                          uint32_t grid[3], uint32_t block[3]) {
    grid[0] = s->rows_per_wave == 0 ? (K + 255) / 256 : s->rows_per_wave == 5 ? (N + 3) / 4 : (N + 7) / 8;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// relayout_q4k_q4l(w, nib, qa, qb, nblocks): 8 threads per super-block
static int check_relayout(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t nb = c[0];
    if (!nb || nb > 0x0FFFFFFFu) return ojh_fail(OJH_ERR_ARG, "%s: nblocks=%u out of range", s->name, nb);
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * 32 < nb)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must cover %u super-blocks, 32 per workgroup", s->name, nb);
    need[0] = (size_t)nb * 144;
    need[1] = (size_t)nb * 128;
    need[2] = need[3] = (size_t)nb * 16;
    align[2] = align[3] = 2;
    return OJH_OK;
}
static int shape_relayout(const ojh_kernel_spec *, const ojh_device *, uint32_t, uint32_t N, uint32_t,
                          uint32_t grid[3], uint32_t block[3]) {
    grid[0] = (N + 31) / 32;  // N = super-blocks
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// dequant_<fmt>_f16(w, out, nblocks)
// threads a decoder spends on one block of its format: a thread per eight weights
static uint32_t dequant_threads_per_block(uint32_t type) {
    const ojh_block_format *f = ojh_format(type);
    return f && f->weights == 32 ? 4 : 32;
}
static int check_dequant(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                         const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f = ojh_format(s->type);
    uint32_t nb = c[0];
    if (!f || nb == 0) return ojh_fail(OJH_ERR_ARG, "%s: nblocks must be positive", s->name);
    int rc = check_block(block, 256);
    if (rc) return rc;
    uint32_t tpb = dequant_threads_per_block(s->type);
    if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * 256 < (uint64_t)nb * tpb)
        return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover %u blocks", s->name, nb);
    need[0] = (size_t)nb * f->bytes;
    need[1] = (size_t)nb * f->weights * 2;
    align[0] = ojh_block_align(f);
    align[1] = 8;
    return OJH_OK;
}

// embed_q80(table, out, token, d) / embed_q80_g(table, out, ctl, d): a thread per weight, grid-stride
static int check_embed(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                       const uint32_t block[3], size_t need[16], size_t align[16]) {
    const uint32_t d = c[s->n_consts - 1];
    if (!d || d % 32) return ojh_fail(OJH_ERR_ARG, "%s: d=%u must be a positive multiple of 32", s->name, d);
    int rc = check_block(block, 0);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    need[0] = (size_t)(d / 32) * 34;      // one row; the dispatcher turns the extent into the row bound
    need[1] = (size_t)d * 4;
    need[2] = 4;
    align[0] = 2;
    align[1] = align[2] = 4;
    return OJH_OK;
}
static int shape_embed(const ojh_kernel_spec *, const ojh_device *, uint32_t K, uint32_t, uint32_t,
                       uint32_t grid[3], uint32_t block[3]) {   // K = d
    grid[0] = (K + 255) / 256;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// gemm_mm_<fmt>(xh, w, y, K, N, accum, M) and gemm_mm_<fmt>_sk(xh, w, y, K, N, M, nsplit);
// `rows_per_wave` = 1 marks the split-K form.
// `rows_per_wave` carries the variant: bit 0 = split-K entry; 0/1 the 256 x 128 tile of family
// "gemm", 2/3 the 256 x 256 tile and 4/5 the 128 x 256 tile of family "gemm_xl".
static void gemm_tile(const ojh_kernel_spec *s, uint32_t *bm, uint32_t *bn, bool *sk) {
    *sk = s->rows_per_wave & 1;
    *bn = (s->rows_per_wave >= 2 && s->rows_per_wave < 8) ? 256 : 128;
    *bm = (s->rows_per_wave >= 4 && s->rows_per_wave < 8) ? 128 : 256;
    if (s->rows_per_wave == 12 || s->rows_per_wave == 13) {   // 64 rows x 128 tokens, K over the workgroup's waves
        *bn = 64;
        *bm = 128;
    }
    if (s->rows_per_wave == 14 || s->rows_per_wave == 15) {   // 128 rows x 128 tokens (the `_m128` entries of family "gemm")
        *bn = 128;
        *bm = 128;
    }
}

static int check_gemm(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                      const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    bool sk;
    uint32_t bm, bn;
    gemm_tile(s, &bm, &bn, &sk);
    uint32_t K = c[0], N = c[1], M = sk ? c[2] : c[3], nsplit = sk ? c[3] : 1;
    static const ojh_block_format plain_f16 = {OJH_F16, 2, 1, "f16"};   // (rows of plain f16: the `gemm_mm_f16*` entries)
    int rc = OJH_OK;
    if (s->type == OJH_F16) {
        f = &plain_f16;
        if (!K || !N) rc = ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u", s->name, K, N);
    } else {
        rc = check_kn(s, K, N, &f);
    }
    if (rc) return rc;
    if (K % 64) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a multiple of 64", s->name, K);
    if (M == 0 || nsplit == 0) return ojh_fail(OJH_ERR_ARG, "%s: M and nsplit must be positive", s->name);
    if ((rc = check_block(block, 256))) return rc;
    if (grid[0] != (N + bn - 1) / bn || grid[1] != (M + bm - 1) / bm || grid[2] != nsplit)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,%u]", s->name, (N + bn - 1) / bn, (M + bm - 1) / bm, nsplit);
    // the 256-wide tiles address activations with 32-bit byte offsets
    if (bn != 128 && (uint64_t)M * K * 2 > 0xFFFFFFFFull)
        return ojh_fail(OJH_ERR_ARG, "%s: M*K=%llu exceeds 2^31 activations", s->name, (unsigned long long)M * K);
    if (bn != 128 && (uint64_t)N * (K / f->weights) * f->bytes > 0xFFFFFFFFull)
        return ojh_fail(OJH_ERR_ARG, "%s: the weight tensor exceeds 4 GiB", s->name);
    need[0] = (size_t)M * K * 2;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)M * N * 4;
    align[1] = s->type == OJH_F16 ? 16 : ojh_block_align(f);
    align[2] = 4;
    return OJH_OK;
}

// gemm_mm_q4kl_bd{,256}_sr(xh, w, y, part, cnt, K, N, M, nsplit, ACC): K slices that meet in `part` (one tile per
// slice, 4 bytes x tile outputs) under one counter per tile; `rows_per_wave` = tokens per tile.
uint32_t ojh_gemm_sr_slices(uint32_t K, uint32_t nsplit) {   // slices that hold at least one super-block
    const uint32_t nsb = K / 256, per = (nsb + nsplit - 1) / nsplit;
    return per ? (nsb + per - 1) / per : 0;
}
static int check_gemm_sr(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                         const uint32_t block[3], size_t need[16], size_t align[16]) {
    const ojh_block_format *f;
    const uint32_t bm = (uint32_t)s->rows_per_wave, bn = 256;
    uint32_t K = c[0], N = c[1], M = c[2], nsplit = c[3];
    int rc = check_kn(s, K, N, &f);
    if (rc) return rc;
    if (M == 0 || nsplit == 0 || nsplit > K / 256) return ojh_fail(OJH_ERR_ARG, "%s: M=%u and nsplit=%u (1 .. K/256) out of range", s->name, M, nsplit);
    if ((rc = check_block(block, 256))) return rc;
    if (grid[0] != (N + bn - 1) / bn || grid[1] != (M + bm - 1) / bm || grid[2] != nsplit)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,%u]", s->name, (N + bn - 1) / bn, (M + bm - 1) / bm, nsplit);
    if ((uint64_t)M * K * 2 > 0xFFFFFFFFull)
        return ojh_fail(OJH_ERR_ARG, "%s: M*K=%llu exceeds 2^31 activations", s->name, (unsigned long long)M * K);
    if ((uint64_t)N * (K / f->weights) * f->bytes > 0xFFFFFFFFull)
        return ojh_fail(OJH_ERR_ARG, "%s: the weight tensor exceeds 4 GiB", s->name);
    const size_t tiles = (size_t)grid[0] * grid[1];
    need[0] = (size_t)M * K * 2;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)M * N * 4;
    need[3] = tiles * ojh_gemm_sr_slices(K, nsplit) * bm * bn * 4;
    need[4] = tiles * 4;
    align[1] = ojh_block_align(f);
    align[2] = align[4] = 4;
    return OJH_OK;
}
static int shape_gemm_sr(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                         uint32_t grid[3], uint32_t block[3]) {
    const uint32_t bm = (uint32_t)s->rows_per_wave;
    grid[0] = (N + 255) / 256;
    grid[1] = (M + bm - 1) / bm;
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
    uint32_t tiles = grid[0] * grid[1], nsb = K / 256;
    uint32_t z = tiles ? cus / tiles : 1;
    if (z > nsb) z = nsb;
    if (z > 16) z = 16;
    grid[2] = z ? z : 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// gemm_mm_q4l(x f32, w4, y, qa, qb, K, N, accum, M), gemm_mm_q4l_hb(xh f16, ...), gemm_mm_q4l_sk(xh, w4, y, qa, qb, K, N, M, nsplit):
// the reference's argument lists (crates/ojas-cuda/src/kernels/gemm_q.rs:26-38).  `rows_per_wave`: 8 plain with f32
// activations, 9 split-K, 10 plain with f16 activations; all on the 256 x 128 tile.
static int check_gemm_q4l(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    const bool sk = s->rows_per_wave == 9, xf32 = s->rows_per_wave == 8;
    uint32_t K = c[0], N = c[1], M = sk ? c[2] : c[3], nsplit = sk ? c[3] : 1;
    if (!K || !N || K % 256) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u (Q4L is relaid Q4_K: K a positive multiple of 256)", s->name, K, N);
    if (M == 0 || nsplit == 0) return ojh_fail(OJH_ERR_ARG, "%s: M and nsplit must be positive", s->name);
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[0] != (N + 127) / 128 || grid[1] != (M + 255) / 256 || grid[2] != nsplit)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,%u,%u]", s->name, (N + 127) / 128, (M + 255) / 256, nsplit);
    need[0] = (size_t)M * K * (xf32 ? 4 : 2);
    need[1] = (size_t)N * (K / 2);
    need[2] = (size_t)M * N * 4;
    need[3] = need[4] = (size_t)N * (K / 32) * 2;
    align[2] = 4;
    align[3] = align[4] = 2;
    return OJH_OK;
}

static int shape_gemm(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                      uint32_t grid[3], uint32_t block[3]) {
    bool sk;
    uint32_t bm, bn;
    gemm_tile(s, &bm, &bn, &sk);
    grid[0] = (N + bn - 1) / bn;
    grid[1] = (M + bm - 1) / bm;
    grid[2] = 1;
    if (sk) {  // split K until every CU has a tile, at least 4 K-steps per slice
        uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
        uint32_t tiles = grid[0] * grid[1], steps = K / 64;
        uint32_t z = tiles ? cus / tiles : 1;  // floor: 224 tiles on 256 CUs are better left whole
        if (z > steps / 4) z = steps / 4;
        if (s->rows_per_wave == 13 && z > steps / 16) z = steps / 16;   // K over the waves: a super-block per wave and slice at least
        if (z > 16) z = 16;
        grid[2] = z ? z : 1;
    }
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// gemm_few_<fmt>{,_r4}_t{1,2,4}(xh, w, y, K, N, accum, M): grid [ceil(N / 16 RG),1,1] x 256 (or 512 where RG TG <= 4); K a
// multiple of 128 (and whole blocks of the format); up to 16 TG tokens (`rows_per_wave` = 16 RG + TG)
static int check_gemm_few(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                          const uint32_t block[3], size_t need[16], size_t align[16]) {
    const uint32_t K = c[0], N = c[1], M = c[3], TG = (uint32_t)s->rows_per_wave & 15u, RG = (uint32_t)s->rows_per_wave >> 4;
    static const ojh_block_format plain_f16 = {OJH_F16, 2, 1, "f16"};
    const ojh_block_format *f = &plain_f16;
    int rc;
    if (s->type == OJH_F16) {
        if (!K || !N) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u", s->name, K, N);
    } else if ((rc = check_kn(s, K, N, &f))) {
        return rc;
    }
    if (K % 128) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a multiple of 128", s->name, K);
    if (!M || M > 16 * TG) return ojh_fail(OJH_ERR_ARG, "%s: M=%u, takes 1 to %u tokens", s->name, M, 16 * TG);
    if (block[0] != 256 && !(block[0] == 512 && RG * TG <= 4))
        return ojh_fail(OJH_ERR_ARG, "%s: block must be 256%s threads", s->name, RG * TG <= 4 ? " or 512" : "");
    if (block[1] != 1 || block[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: block must be [x,1,1]", s->name);
    if (grid[0] != (N + 16 * RG - 1) / (16 * RG) || grid[1] != 1 || grid[2] != 1)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [%u,1,1]", s->name, (N + 16 * RG - 1) / (16 * RG));
    need[0] = (size_t)M * K * 2;
    need[1] = (size_t)N * (K / f->weights) * f->bytes;
    need[2] = (size_t)M * N * 4;
    align[0] = 16;
    align[1] = s->type == OJH_F16 ? 16 : ojh_block_align(f);
    align[2] = 4;
    return OJH_OK;
}
static int shape_gemm_few(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                          uint32_t grid[3], uint32_t block[3]) {
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
    const uint32_t TG = (uint32_t)s->rows_per_wave & 15u, RG = (uint32_t)s->rows_per_wave >> 4;
    grid[0] = (N + 16 * RG - 1) / (16 * RG);
    grid[1] = grid[2] = 1;
    block[0] = grid[0] < 2 * cus && RG * TG <= 4 ? 512 : 256;     // few workgroups: eight waves share their K
    block[1] = block[2] = 1;
    return OJH_OK;
}

// LDS of the moe_*_mt entries: 16 token rows, their scales and split sums, a block of zeros, the pass's assignments
uint64_t ojh_moe_mt_lds(uint32_t K) { return 16 * ((uint64_t)K + 32) + K / 4 + K + 256 + 64; }

// The MoE family; the number of tokens of the batched entries is read off the grid.
//   0 moe_topk(lg, idx, wgt, E, KSEL)            1 moe_topk_m(same)              grid [T,1,1] x 64
//   2 moe_group(idx, counts, offsets, list, NA, E)                                grid [1,1,1] x 256
//   3 moe_gu_q4k_m(xq, xs, wg, wu, act, offsets, list, K, N, KSEL, NA)            grid [ceil(N/8), E, 1]
//   4 moe_down_q4k_m(aq, as, wd, dv, offsets, list, K, N, NA)                     grid [ceil(N/16), E, 1]; ceil(N/32) for K <= 1024
//   5 moe_combine(dv, wgt, y, T, KSEL, D, ACC)                                    grid [ceil(T*D/256),1,1]
//   6 moe_gu_q4k_mm, 7 moe_down_q4k_mm: the arguments of 3 and 4, grid [ceil(N/16), E, 1]
//  12 moe_gu_q4k_mt, 13 moe_down_q4k_mt: the arguments of 3 and 4, grid [1 .. ceil(N/16), E, 1] x 512
//   8 moe_gu_q4k_dec(x, wg, wu, act, idx, K, N, KSEL, NA, E)                      grid [ceil(N/8), NA, 1]
//   9 moe_down_q4k_dec(act, wd, idx, wgt, y, K, N, KSEL, E, ACC)                  grid [ceil(N/8), T, 1]
//  14 moe_gu_q80(x, wg, wu, act, idx, K, N)                                     grid [ceil(N/8), KSEL, tokens]
//  15 moe_down_q80(act, wd, y, idx, wgt, K, N, KSEL)                            grid [1 .. ceil(N/4), tokens, 1]
//  14 / 15 also moe_{gu,down}_{iq4xs,iq4nl} of family "moe_iq", the same arguments
//  16 moe_gu_q80_slots(x, arena_g, arena_u, act, off_g, off_u, K, N)             grid [ceil(N/8), KSEL, tokens]
//  17 moe_down_q80_slots(act, arena, y, off_d, wgt, K, N, KSEL)                  grid [1 .. ceil(N/4), tokens, 1]
//     (the reference's Q8_0 expert kernels; the expert count is not an argument, so the weight buffers are
//     checked for one expert only)
//  10 moe_gu_q4k_slots, 11 moe_down_q4k_slots: 8 and 9 with a u64 byte offset per assignment into an arena
//     and LIM * 256 = the last offset at which an expert still fits, in place of idx and E
static int check_moe(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                     const uint32_t block[3], size_t need[16], size_t align[16]) {
    int rc;
    for (int i = 0; i < 8; i++) align[i] = 4;
    switch (s->rows_per_wave) {
    case 0: case 1: {
        uint32_t E = c[0], KS = c[1], T = grid[0];
        if ((rc = check_block(block, 64))) return rc;
        if (!E || E > 1024 || !KS || KS > E || KS > 64) return ojh_fail(OJH_ERR_ARG, "%s: E=%u KSEL=%u out of range", s->name, E, KS);
        if (grid[1] != 1 || grid[2] != 1 || (s->rows_per_wave == 0 && T != 1))
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [tokens,1,1]", s->name);
        need[0] = (size_t)T * E * 4;
        need[1] = need[2] = (size_t)T * KS * 4;
        return OJH_OK;
    }
    case 18: case 19: {  // moe_topk_nonorm(lg, idx, wgt, E, KSEL); moe_topk_v3(lg, bias, idx, wgt, E, KSEL, RSCALE, NORM)
        const bool v3 = s->rows_per_wave == 19;
        uint32_t E = c[0], KS = c[1], T = grid[0];
        if ((rc = check_block(block, 64))) return rc;
        if (!E || E > 1024 || !KS || KS > E || KS > 64) return ojh_fail(OJH_ERR_ARG, "%s: E=%u KSEL=%u out of range", s->name, E, KS);
        if (!T || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [tokens,1,1]", s->name);
        need[0] = (size_t)T * E * 4;
        if (v3) need[1] = (size_t)E * 4;
        need[v3 ? 2 : 1] = need[v3 ? 3 : 2] = (size_t)T * KS * 4;
        return OJH_OK;
    }
    case 20: {   // moe_quant_group(x, xq, xs, idx, counts, offsets, list, K, T, NA, E)   grid [T + 1,1,1]
        uint32_t K = c[0], T = c[1], NA = c[2], E = c[3];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || !T || !NA || !E || E > 1024) return ojh_fail(OJH_ERR_ARG, "%s: K=%u T=%u NA=%u E=%u out of range", s->name, K, T, NA, E);
        if (grid[0] != T + 1 || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [T + 1,1,1]", s->name);
        need[0] = (size_t)T * K * 4;
        need[1] = (size_t)T * K;
        need[2] = (size_t)T * (K / 256) * 4;
        need[3] = need[6] = (size_t)NA * 4;
        need[4] = (size_t)E * 4;
        need[5] = (size_t)(E + 1) * 4;
        align[0] = align[1] = 16;
        return OJH_OK;
    }
    case 2: {
        uint32_t NA = c[0], E = c[1];
        if ((rc = check_block(block, 256))) return rc;
        if (!NA || !E || E > 1024) return ojh_fail(OJH_ERR_ARG, "%s: NA=%u E=%u out of range", s->name, NA, E);
        if (grid[0] != 1 || grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [1,1,1]", s->name);
        need[0] = need[3] = (size_t)NA * 4;
        need[1] = (size_t)E * 4;
        need[2] = (size_t)(E + 1) * 4;
        return OJH_OK;
    }
    case 3: case 6: case 12: {
        uint32_t K = c[0], N = c[1], KS = c[2], NA = c[3], E = grid[1];
        const uint32_t per = s->rows_per_wave == 3 ? 8 : 16;   // rows per workgroup
        const bool mt = s->rows_per_wave == 12;
        if ((rc = check_block(block, mt ? 512 : 256))) return rc;
        if (!K || K % 256 || !N || !KS || !NA || NA % KS) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u KSEL=%u NA=%u", s->name, K, N, KS, NA);
        if (mt) {
            if (ojh_moe_mt_lds(K) > 81920) return ojh_fail(OJH_ERR_ARG, "%s: 16 tokens of K=%u do not fit its 80 KB of LDS", s->name, K);
            if (!grid[0] || grid[0] > (N + 15) / 16 || grid[2] != 1)
                return ojh_fail(OJH_ERR_ARG, "%s: grid must be [1 .. ceil(N/16), E, 1]", s->name);
        } else if (grid[0] != (N + per - 1) / per || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/%u), E, 1]", s->name, per);
        size_t rb = (size_t)(K / 256) * 144;
        need[0] = (size_t)(NA / KS) * K;
        need[1] = (size_t)(NA / KS) * (K / 256) * 4;
        need[2] = need[3] = (size_t)E * N * rb;
        need[4] = (size_t)NA * N * 4;
        need[5] = (size_t)(E + 1) * 4;
        need[6] = (size_t)NA * 4;
        align[0] = align[2] = align[3] = 16;
        return OJH_OK;
    }
    case 4: case 7: case 13: {
        uint32_t K = c[0], N = c[1], NA = c[2], E = grid[1];
        const uint32_t per = s->rows_per_wave == 4 && K <= 1024 ? 32 : 16;   // short rows: two row sets per wave
        const bool mt = s->rows_per_wave == 13;
        if ((rc = check_block(block, mt ? 512 : 256))) return rc;
        if (!K || K % 256 || !N || !NA) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u NA=%u", s->name, K, N, NA);
        if (mt) {
            if (ojh_moe_mt_lds(K) > 81920) return ojh_fail(OJH_ERR_ARG, "%s: 16 tokens of K=%u do not fit its 80 KB of LDS", s->name, K);
            if (!grid[0] || grid[0] > (N + 15) / 16 || grid[2] != 1)
                return ojh_fail(OJH_ERR_ARG, "%s: grid must be [1 .. ceil(N/16), E, 1]", s->name);
        } else if (grid[0] != (N + per - 1) / per || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/%u), E, 1]", s->name, per);
        need[0] = (size_t)NA * K;
        need[1] = (size_t)NA * (K / 256) * 4;
        need[2] = (size_t)E * N * (K / 256) * ojh_format(s->type)->bytes;
        need[3] = (size_t)NA * N * 4;
        need[4] = (size_t)(E + 1) * 4;
        need[5] = (size_t)NA * 4;
        align[0] = align[2] = 16;
        return OJH_OK;
    }
    case 22: {  // moe_down_{q6k,q5k}_gs(aq, as, wd, dv, offsets, list, K, N, NA)   grid [ceil(N/128), 1 .. , E]
        uint32_t K = c[0], N = c[1], NA = c[2], E = grid[2];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || !N || !NA) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u NA=%u", s->name, K, N, NA);
        if (grid[0] != (N + 127) / 128 || !grid[1] || grid[1] > 65535 || !E || E > 65535)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/128), token tiles (any, up to 65535), E]", s->name);
        need[0] = (size_t)NA * K;
        need[1] = (size_t)NA * (K / 256) * 4;
        need[2] = (size_t)E * N * (K / 256) * ojh_format(s->type)->bytes;
        need[3] = (size_t)NA * N * 4;
        need[4] = (size_t)(E + 1) * 4;
        need[5] = (size_t)NA * 4;
        align[0] = align[2] = 16;
        return OJH_OK;
    }
    case 8: {   // moe_gu_q4k_dec(x, wg, wu, act, idx, K, N, KSEL, NA, E)
        uint32_t K = c[0], N = c[1], KS = c[2], NA = c[3], E = c[4];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || !N || !KS || !NA || NA % KS || !E) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u KSEL=%u NA=%u E=%u", s->name, K, N, KS, NA, E);
        if (K > 8192) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: K=%u exceeds the 8192 activations staged in LDS", s->name, K);
        if (grid[0] != (N + 7) / 8 || grid[1] != NA || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), NA, 1]", s->name);
        need[0] = (size_t)(NA / KS) * K * 4;
        need[1] = need[2] = (size_t)E * N * (K / 256) * 144;
        need[3] = (size_t)NA * N * 4;
        need[4] = (size_t)NA * 4;
        align[0] = align[1] = align[2] = 16;
        return OJH_OK;
    }
    case 21: {  // moe_gu_q4k_decr(x, wg, wu, act, lg, idx, wgt, K, N, KSEL, NA, E): the decode form, router inside
        uint32_t K = c[0], N = c[1], KS = c[2], NA = c[3], E = c[4];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || !N || !KS || KS > 64 || !NA || NA % KS || !E || E > 1024 || KS > E)
            return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u KSEL=%u (<= 64, <= E) NA=%u E=%u (<= 1024)", s->name, K, N, KS, NA, E);
        if (K > 8192) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: K=%u exceeds the 8192 activations staged in LDS", s->name, K);
        if (grid[0] != (N + 7) / 8 || grid[1] != NA || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), NA, 1]", s->name);
        need[0] = (size_t)(NA / KS) * K * 4;
        need[1] = need[2] = (size_t)E * N * (K / 256) * 144;
        need[3] = (size_t)NA * N * 4;
        need[4] = (size_t)(NA / KS) * E * 4;
        need[5] = need[6] = (size_t)NA * 4;
        align[0] = align[1] = align[2] = 16;
        align[4] = align[5] = align[6] = 4;
        return OJH_OK;
    }
    case 9: {   // moe_down_q4k_dec(act, wd, idx, wgt, y, K, N, KSEL, E, ACC)
        uint32_t K = c[0], N = c[1], KS = c[2], E = c[3], T = grid[1];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || !N || !KS || KS > 64 || !E) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u KSEL=%u (<= 64) E=%u", s->name, K, N, KS, E);
        if (K > 2048) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: K=%u exceeds the 2048 (eight super-blocks) a wave takes side by side", s->name, K);
        if ((uint64_t)KS * K > 32768) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: KSEL * K = %llu activations exceed the 32768 staged in LDS", s->name, (unsigned long long)KS * K);
        if (grid[0] != (N + 7) / 8 || !T || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), tokens, 1]", s->name);
        need[0] = (size_t)T * KS * K * 4;
        need[1] = (size_t)E * N * (K / 256) * ojh_format(s->type)->bytes;
        need[2] = need[3] = (size_t)T * KS * 4;
        need[4] = (size_t)T * N * 4;
        align[0] = align[1] = 16;
        return OJH_OK;
    }
    case 14: {  // moe_gu_{q80,iq4xs,iq4nl}(x, wg, wu, act, idx, K, N)
        uint32_t K = c[0], N = c[1], KS = grid[1], T = grid[2];
        const ojh_block_format *f = ojh_format(s->type);
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % f->weights || !N || !KS || !T) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u slots=%u tokens=%u", s->name, K, N, KS, T);
        if (grid[0] != (N + 7) / 8) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), slots, tokens]", s->name);
        need[0] = (size_t)T * K * 4;
        need[1] = need[2] = (size_t)N * (K / f->weights) * f->bytes;
        need[3] = (size_t)T * KS * N * 4;
        need[4] = (size_t)T * KS * 4;
        align[0] = 16;
        align[1] = align[2] = ojh_block_align(f);
        return OJH_OK;
    }
    case 15: {  // moe_down_{q80,iq4xs,iq4nl}(act, wd, y, idx, wgt, K, N, KSEL): rows grid-stride, 4 per workgroup
        uint32_t K = c[0], N = c[1], KS = c[2], T = grid[1];
        const ojh_block_format *f = ojh_format(s->type);
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % f->weights || !N || !KS || !T) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u KSEL=%u tokens=%u", s->name, K, N, KS, T);
        if (!grid[0] || grid[0] > (N + 3) / 4 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [1 .. ceil(N/4), tokens, 1]", s->name);
        need[0] = (size_t)T * KS * K * 4;
        need[1] = (size_t)N * (K / f->weights) * f->bytes;
        need[2] = (size_t)T * N * 4;
        need[3] = need[4] = (size_t)T * KS * 4;
        align[0] = 16;
        align[1] = ojh_block_align(f);
        return OJH_OK;
    }
    case 16: {  // moe_gu_{q80,iq3s}_slots(x, arena_g, arena_u, act, off_g, off_u, K, N)
        uint32_t K = c[0], N = c[1], KS = grid[1], T = grid[2];
        const ojh_block_format *f = ojh_format(s->type);
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % f->weights || !N || !KS || !T) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u slots=%u tokens=%u", s->name, K, N, KS, T);
        if (grid[0] != (N + 7) / 8) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), slots, tokens]", s->name);
        need[0] = (size_t)T * K * 4;
        need[1] = need[2] = (size_t)N * (K / f->weights) * f->bytes;
        need[3] = (size_t)T * KS * N * 4;
        need[4] = need[5] = (size_t)T * KS * 4;
        align[0] = 16;
        align[1] = align[2] = 2;
        return OJH_OK;
    }
    case 17: {  // moe_down_q80_slots(act, arena, y, off_d, wgt, K, N, KSEL)
        uint32_t K = c[0], N = c[1], KS = c[2], T = grid[1];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 32 || !N || !KS || !T) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u KSEL=%u tokens=%u", s->name, K, N, KS, T);
        if (!grid[0] || grid[0] > (N + 3) / 4 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [1 .. ceil(N/4), tokens, 1]", s->name);
        need[0] = (size_t)T * KS * K * 4;
        need[1] = (size_t)N * (K / 32) * 34;
        need[2] = (size_t)T * N * 4;
        need[3] = need[4] = (size_t)T * KS * 4;
        align[0] = 16;
        align[1] = 2;
        return OJH_OK;
    }
    case 10: {  // moe_gu_q4k_slots(x, arena_g, arena_u, act, off_g, off_u, K, N, KSEL, NA, LIM_G, LIM_U)
        uint32_t K = c[0], N = c[1], KS = c[2], NA = c[3];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || K > 8192 || !N || !KS || !NA || NA % KS) return ojh_fail(OJH_ERR_ARG, "%s: K=%u (<= 8192) N=%u KSEL=%u NA=%u", s->name, K, N, KS, NA);
        if (grid[0] != (N + 7) / 8 || grid[1] != NA || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), NA, 1]", s->name);
        const size_t eb = (size_t)N * (K / 256) * 144;
        need[0] = (size_t)(NA / KS) * K * 4;
        need[1] = (size_t)c[4] * 256 + eb;
        need[2] = (size_t)c[5] * 256 + eb;
        need[3] = (size_t)NA * N * 4;
        need[4] = need[5] = (size_t)NA * 8;
        align[0] = align[1] = align[2] = 16;
        align[4] = align[5] = 8;
        return OJH_OK;
    }
    case 11: {  // moe_down_q4k_slots(act, arena, off_d, wgt, y, K, N, KSEL, LIM, ACC)
        uint32_t K = c[0], N = c[1], KS = c[2], T = grid[1];
        if ((rc = check_block(block, 256))) return rc;
        if (!K || K % 256 || K > 2048 || !N || !KS || KS > 64 || (uint64_t)KS * K > 32768)
            return ojh_fail(OJH_ERR_ARG, "%s: K=%u (<= 2048) N=%u KSEL=%u (<= 64, KSEL * K <= 32768)", s->name, K, N, KS);
        if (grid[0] != (N + 7) / 8 || !T || grid[2] != 1)
            return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/8), tokens, 1]", s->name);
        need[0] = (size_t)T * KS * K * 4;
        need[1] = (size_t)c[3] * 256 + (size_t)N * (K / 256) * 144;
        need[2] = (size_t)T * KS * 8;
        need[3] = (size_t)T * KS * 4;
        need[4] = (size_t)T * N * 4;
        align[0] = align[1] = 16;
        align[2] = 8;
        return OJH_OK;
    }
    default: {
        uint32_t T = c[0], KS = c[1], D = c[2];
        if ((rc = check_block(block, 256))) return rc;
        if (!T || !KS || !D) return ojh_fail(OJH_ERR_ARG, "%s: T=%u KSEL=%u D=%u", s->name, T, KS, D);
        if (grid[1] != 1 || grid[2] != 1 || (uint64_t)grid[0] * 256 < (uint64_t)T * D)
            return ojh_fail(OJH_ERR_ARG, "%s: grid does not cover %u x %u outputs", s->name, T, D);
        need[0] = (size_t)T * KS * D * 4;
        need[1] = (size_t)T * KS * 4;
        need[2] = (size_t)T * D * 4;
        return OJH_OK;
    }
    }
}

// K, N as named by the kernel; M = tokens (topk, combine) or assignments (group)
// Workgroups per expert for the moe_*_mt entries: about `per_cu` workgroups per CU over all experts (what
// is resident at once: one for the gate/up entry, which holds two tensors' blocks of four steps in
// registers, two for the down entry), fewer until the expert's tiles divide evenly over the workgroups'
// eight waves (or one workgroup is left).
uint32_t ojh_moe_mt_groups(const ojh_device *dev, uint32_t N, uint32_t E, uint32_t per_cu) {
    const uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, tiles = (N + 15) / 16;
    uint32_t rg = per_cu * cus / (E ? E : 1), cap = (tiles + 7) / 8;
    if (rg > cap) rg = cap;
    if (rg < 1) rg = 1;
    while (rg > 1 && tiles % (8 * rg)) rg--;
    return rg;
}
static int shape_moe(const ojh_kernel_spec *s, const ojh_device *dev, uint32_t K, uint32_t N, uint32_t M,
                     uint32_t grid[3], uint32_t block[3]) {
    grid[0] = grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    switch (s->rows_per_wave) {
    case 0: block[0] = 64; break;
    case 1: case 18: case 19: block[0] = 64; grid[0] = M ? M : 1; break;
    case 2: break;
    case 3: grid[0] = (N + 7) / 8; grid[1] = M ? M : 1; break;    // M = experts
    case 4: grid[0] = K <= 1024 ? (N + 31) / 32 : (N + 15) / 16; grid[1] = M ? M : 1; break;  // M = experts
    case 20: grid[0] = M + 1; break;  // M = tokens
    case 22: grid[0] = (N + 127) / 128; grid[2] = M ? M : 1; break;   // M = experts; grid[1]: the caller's token tiles per expert
    case 21: grid[0] = (N + 7) / 8; grid[1] = M ? M : 1; break;   // M = assignments
    case 6: case 7: grid[0] = (N + 15) / 16; grid[1] = M ? M : 1; break;
    case 14: case 16: grid[0] = (N + 7) / 8; grid[1] = M ? M : 1; break;    // M = slots, one token
    case 15: case 17: grid[0] = (N + 3) / 4; break;                           // one token
    case 12: case 13: grid[0] = ojh_moe_mt_groups(dev, N, M ? M : 1, s->rows_per_wave == 12 ? 1 : 2); grid[1] = M ? M : 1; block[0] = 512; break;  // M = experts
    case 8: case 10: grid[0] = (N + 7) / 8; grid[1] = M ? M : 1; break;    // M = assignments
    case 9: case 11: grid[0] = (N + 7) / 8; grid[1] = M ? M : 1; break;    // M = tokens
    default: grid[0] = (uint32_t)(((uint64_t)M * N + 255) / 256); break;  // N = D, M = tokens
    }
    return OJH_OK;
}

// moe_mm_<fmt>(xh, w0, w1, y0, y1, offsets, list, K, N, NA, E, DIV): grid [ceil(N/128), token tiles (any), E or 2 E];
// w1 / y1 may be NULL with a grid of E.  moe_act_half(g, u, act16, n): grid [x,1,1], grid-stride.
static int check_moe_mm(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                        const uint32_t block[3], size_t need[16], size_t align[16]) {
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (s->rows_per_wave == 1) {
        const size_t n = c[0];
        if (!n) return ojh_fail(OJH_ERR_ARG, "%s: n must be positive", s->name);
        if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
        need[0] = need[1] = n * 4;
        need[2] = n * 2;
        align[0] = align[1] = 4;
        align[2] = 2;
        return OJH_OK;
    }
    const uint32_t K = c[0], N = c[1], NA = c[2], E = c[3], DIV = c[4];
    static const ojh_block_format plain_f16 = {OJH_F16, 2, 1, "f16"};   // (rows of plain f16: `moe_mm_f16`)
    const ojh_block_format *f = &plain_f16;
    if (s->type == OJH_F16) {
        if (!K || !N) return ojh_fail(OJH_ERR_ARG, "%s: K=%u N=%u", s->name, K, N);
    } else if ((rc = check_kn(s, K, N, &f))) {
        return rc;
    }
    const uint32_t bn = s->rows_per_wave == 2 ? 64u : 128u, bk = s->rows_per_wave == 2 ? 128u : 64u;   // (2: the `moe_few_*` entries)
    if (K % bk) return ojh_fail(OJH_ERR_ARG, "%s: K=%u must be a multiple of %u", s->name, K, bk);
    if (!NA || !E || !DIV) return ojh_fail(OJH_ERR_ARG, "%s: NA=%u E=%u DIV=%u", s->name, NA, E, DIV);
    if (grid[0] != (N + bn - 1) / bn || !grid[1] || grid[1] > 65535 || (grid[2] != E && grid[2] != 2 * E) || grid[2] > 65535)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [ceil(N/%u), token tiles (any, up to 65535), E or 2 E]", s->name, bn);
    const bool pair = grid[2] == 2 * E;
    const size_t wbytes = (size_t)E * N * (K / f->weights) * f->bytes;
    need[0] = ((size_t)(NA - 1) / DIV + 1) * K * 2;
    need[1] = need[2] = wbytes;
    need[3] = need[4] = (size_t)NA * N * 4;
    need[5] = (size_t)(E + 1) * 4;
    need[6] = (size_t)NA * 4;
    align[0] = 16;
    const size_t wal = s->type == OJH_F16 ? 16 : ojh_block_align(f);
    align[1] = wal;
    align[2] = pair ? wal : 0;                     // 0: the buffer may be NULL (unused with a grid of E)
    align[3] = 4;
    align[4] = pair ? 4 : 0;
    align[5] = align[6] = 4;
    return OJH_OK;
}
static int shape_moe_mm(const ojh_kernel_spec *s, const ojh_device *, uint32_t, uint32_t N, uint32_t M,
                        uint32_t grid[3], uint32_t block[3]) {
    grid[0] = s->rows_per_wave == 1 ? (uint32_t)(((uint64_t)(N ? N : 1) + 1023) / 1024) : s->rows_per_wave == 2 ? (N + 63) / 64 : (N + 127) / 128;   // (act: N = elements)
    grid[1] = 1;
    grid[2] = s->rows_per_wave == 1 ? 1 : (M ? M : 1);     // M = experts
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

// copy_*(x, y, n) / fill_zero_u32(y, n): grid-stride, any positive grid of 256-thread blocks
static int check_elementwise(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                             const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t n = c[0];
    if (!n) return ojh_fail(OJH_ERR_ARG, "%s: n must be positive", s->name);
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    if (s->n_bufs == 1) {
        need[0] = (size_t)n * (s->type & 0xFF);
        align[0] = 4;
    } else {
        need[0] = (size_t)n * (s->type >> 8);
        need[1] = (size_t)n * (s->type & 0xFF);
        align[0] = s->type >> 8;
        align[1] = s->type & 0xFF;
    }
    return OJH_OK;
}

// copy_{bf16,f32}_half_zero(x, y, z, n, nz, CB): CB converting workgroups, the rest of the grid clears z
static int check_convert_zero(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                              const uint32_t block[3], size_t need[16], size_t align[16]) {
    uint32_t n = c[0], nz = c[1], cb = c[2];
    if (!n || !nz) return ojh_fail(OJH_ERR_ARG, "%s: n=%u and nz=%u must be positive", s->name, n, nz);
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1 || !cb || grid[0] <= cb)
        return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1] with x > CB=%u > 0 (CB workgroups convert, the others clear)", s->name, cb);
    need[0] = (size_t)n * (s->type >> 8);
    need[1] = (size_t)n * 2;
    need[2] = (size_t)nz * 4;
    align[0] = s->type >> 8;
    align[1] = 2;
    align[2] = 4;
    return OJH_OK;
}

// stream_copy_u32x4(x, y, n16) / stream_read_u32x4(x, y, n16): grid-stride over 16-byte units
static int check_stream(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                        const uint32_t block[3], size_t need[16], size_t align[16]) {
    (void)align;
    uint32_t n16 = c[0];
    if (!n16) return ojh_fail(OJH_ERR_ARG, "%s: n16 must be positive", s->name);
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    need[0] = (size_t)n16 * 16;
    need[1] = s->type == 1 ? (size_t)grid[0] * 16 : (size_t)n16 * 16;
    return OJH_OK;
}

// calib_mfma_f16(x, y, iters, mode): 32 KB of operands, one dword out per thread
static int check_calib_mfma(const ojh_kernel_spec *s, const uint32_t *c, const uint32_t grid[3],
                            const uint32_t block[3], size_t need[16], size_t align[16]) {
    (void)align;
    if (!c[0] || c[0] > (1u << 20)) return ojh_fail(OJH_ERR_ARG, "%s: iters=%u out of range (1 .. 2^20)", s->name, c[0]);
    if (c[1] > (strstr(s->name, "_i8") ? 1u : 2u)) return ojh_fail(OJH_ERR_ARG, "%s: mode=%u (0 = operands in registers, 1 = read from LDS, 2 = with a tile step's copies, LDS writes and vector ALU work)", s->name, c[1]);
    int rc = check_block(block, 256);
    if (rc) return rc;
    if (grid[1] != 1 || grid[2] != 1) return ojh_fail(OJH_ERR_ARG, "%s: grid must be [x,1,1]", s->name);
    need[0] = 8 * 256 * 16 + (c[1] == 2 ? (4u << 20) : 0u);
    need[1] = (size_t)grid[0] * 256 * 4;
    return OJH_OK;
}

// ---- launch shapes ---------------------------------------------------------------------------
static int shape_elementwise(const ojh_kernel_spec *, const ojh_device *, uint32_t, uint32_t N, uint32_t,
                             uint32_t grid[3], uint32_t block[3]) {
    grid[0] = (N / 8 + 255) / 256;  // N = element count; a thread takes 8 elements per trip
    if (!grid[0]) grid[0] = 1;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// N = activations to convert, M = dwords to clear, a thread takes 8 elements or 4 dwords; CB = ceil(N / 2048)
static int shape_convert_zero(const ojh_kernel_spec *, const ojh_device *, uint32_t, uint32_t N, uint32_t M,
                              uint32_t grid[3], uint32_t block[3]) {
    grid[0] = (N / 8 + 255) / 256 + 1 + (M / 4 + 255) / 256 + 1;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// decode_chain_q4k takes one argument block (kernels/ojk_chain.h), not buffers and constants: it is launched by
// ojh_decode_chain, which validates every stage, and cannot be dispatched by name.
static int check_chain(const ojh_kernel_spec *s, const uint32_t *, const uint32_t[3], const uint32_t[3], size_t[16], size_t[16]) {
    return ojh_fail(OJH_ERR_UNSUPPORTED, "%s takes an argument block, not a buffer list: call ojh_decode_chain", s->name);
}
static int shape_chain(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t, uint32_t, uint32_t grid[3],
                       uint32_t block[3]) {
    (void)dev;
    grid[0] = grid[1] = grid[2] = 1;   // the grid is the sum of the stages' workgroups: ojh_decode_chain computes it
    block[0] = 256; block[1] = block[2] = 1;
    return OJH_OK;
}

static int shape_calib_mfma(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t, uint32_t,
                            uint32_t grid[3], uint32_t block[3]) {
    grid[0] = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;   // one workgroup of four waves per CU
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
static int shape_stream(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                        uint32_t grid[3], uint32_t block[3]) {
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u;
    uint32_t want = cus * 8u, cover = (N + 255) / 256;  // N = 16-byte units
    grid[0] = cover < want ? cover : want;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
static int shape_mx(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                    uint32_t grid[3], uint32_t block[3]) {
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, cover = (N + 7) / 8;
    grid[0] = cover < 2 * cus ? cover : 2 * cus;   // two resident workgroups per CU, rows grid-stride
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// 4 waves x 16 rows per workgroup trip; two workgroups per CU are resident (68 KB of LDS each) and a
// grid that is a whole multiple of the CU count measured up to 20 % faster than an evenly divided one
static int shape_mf(const ojh_kernel_spec *, const ojh_device *dev, uint32_t, uint32_t N, uint32_t,
                    uint32_t grid[3], uint32_t block[3]) {
    uint32_t cus = dev ? (uint32_t)dev->prop.multiProcessorCount : 256u, trips = (N + 63) / 64;
    grid[0] = trips < 2 * cus ? trips : 2 * cus;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
static int shape_rows(const ojh_kernel_spec *s, const ojh_device *, uint32_t, uint32_t N, uint32_t,
                      uint32_t grid[3], uint32_t block[3]) {
    uint32_t rows_per_block = 4u * (uint32_t)s->rows_per_wave;
    grid[0] = (N + rows_per_block - 1) / rows_per_block;
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
static int shape_quantize(const ojh_kernel_spec *s, const ojh_device *, uint32_t K, uint32_t, uint32_t M,
                          uint32_t grid[3], uint32_t block[3]) {
    grid[0] = (K + 255) / 256;
    grid[1] = M ? M : 1;
    grid[2] = 1;
    if (s->rows_per_wave == 1) {
        grid[0] = (uint32_t)(((uint64_t)grid[0] * grid[1] + 3) / 4);
        grid[1] = 1;
    }
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}
// dequant: N is the number of blocks
static int shape_dequant(const ojh_kernel_spec *s, const ojh_device *, uint32_t, uint32_t N, uint32_t,
                         uint32_t grid[3], uint32_t block[3]) {
    uint32_t tpb = dequant_threads_per_block(s->type);
    grid[0] = (uint32_t)(((uint64_t)N * tpb + 255) / 256);
    grid[1] = grid[2] = 1;
    block[0] = 256;
    block[1] = block[2] = 1;
    return OJH_OK;
}

static std::vector<ojh_kernel_spec> build_manifest() {
    std::vector<ojh_kernel_spec> m;
    // `names` must outlive the table: keep them in a static pool.
    static std::deque<std::string> pool;
    auto add = [&](const std::string &name, const char *family, int nb, int nc, uint32_t type, int rpw,
                   ojh_check_fn chk, ojh_shape_fn shp) {
        pool.push_back(name);
        m.push_back({pool.back().c_str(), family, nb, nc, type, rpw, chk, shp});
    };
    for (const auto &f : kFormats) {
        std::string t = f.tag;
        // the grid-codebook formats keep decoder and matvecs in one code object of their own
        const bool grid_fmt = ojh_grid_type(f.type);
        const char *fam_nat = grid_fmt ? "iq_grid" : "gemv", *fam_q8k = grid_fmt ? "iq_grid" : "gemv_q8k";
        add("dequant_" + t + "_f16", grid_fmt ? "iq_grid" : "dequant", 2, 1, f.type, 0, check_dequant, shape_dequant);
        if (f.type == OJH_Q5_K) {   // Q5_K: the decoder, the CPU path's int8-activation matvec
            std::string q5 = "gemv_q8k_" + t;
            add(q5, "gemv_q8k", 4, 2, f.type, 4, check_gemv_q8k, shape_rows);
            add(q5 + "_r1", "gemv_q8k", 4, 2, f.type, 1, check_gemv_q8k, shape_rows);
            add(q5 + "_r2", "gemv_q8k", 4, 2, f.type, 2, check_gemv_q8k, shape_rows);
            add(q5 + "_wide", "gemv_q8k", 4, 2, f.type, 2, check_gemv_q8k, shape_rows);
            add(q5 + "_accum", "gemv_q8k", 4, 2, f.type, 1, check_gemv_q8k, shape_rows);
            add(q5 + "_bias", "gemv_q8k", 5, 2, f.type, 1, check_gemv_q8k, shape_rows);
            add(q5 + "_m", "gemv_q8k", 4, 4, f.type, 1, check_gemv_q8k_m, shape_rows);
            // ... and the f32-activation matvecs of the reference's GPU path (no MFMA tile)
            std::string n5 = "gemv_nat_" + t;
            add(n5, "gemv", 3, 2, f.type, 4, check_gemv_nat, shape_rows);
            add(n5 + "_r1", "gemv", 3, 2, f.type, 1, check_gemv_nat, shape_rows);
            add(n5 + "_r2", "gemv", 3, 2, f.type, 2, check_gemv_nat, shape_rows);
            add(n5 + "_accum", "gemv", 3, 2, f.type, 4, check_gemv_nat, shape_rows);
            add(n5 + "_bias", "gemv", 4, 2, f.type, 4, check_gemv_nat, shape_rows);
            add(n5 + "_m", "gemv", 3, 4, f.type, 1, check_gemv_nat_m, shape_rows);
            add(n5 + "_px", "gemv", 3, 2, f.type, 2, check_gemv_nat_px, shape_px);
            continue;
        }
        std::string g = "gemv_nat_" + t;
        add(g, fam_nat, 3, 2, f.type, 4, check_gemv_nat, shape_rows);
        add(g + "_r1", fam_nat, 3, 2, f.type, 1, check_gemv_nat, shape_rows);
        add(g + "_r2", fam_nat, 3, 2, f.type, 2, check_gemv_nat, shape_rows);
        add(g + "_accum", fam_nat, 3, 2, f.type, 4, check_gemv_nat, shape_rows);
        add(g + "_bias", fam_nat, 4, 2, f.type, 4, check_gemv_nat, shape_rows);
        add(g + "_m", fam_nat, 3, 4, f.type, 1, check_gemv_nat_m, shape_rows);
        if (f.type != OJH_Q8_0) add(g + "_px", fam_nat, 3, 2, f.type, 2, check_gemv_nat_px, shape_px);
        if (ojh_float_only(f.type)) continue;   // f32 activations only, no MFMA tile
        if (f.type == OJH_Q8_0) {
            add(g + "_lds", fam_nat, 3, 3, f.type, 1, check_gemv_q80_lds, shape_q80_lds);
            add(g + "_lds_accum", fam_nat, 3, 3, f.type, 1, check_gemv_q80_lds, shape_q80_lds);
            add(g + "_lds_bias", fam_nat, 4, 3, f.type, 1, check_gemv_q80_lds, shape_q80_lds);
            continue;  // the CPU path keeps f32 activations for Q8_0
        }
        std::string q = "gemv_q8k_" + t;
        add(q, fam_q8k, 4, 2, f.type, 4, check_gemv_q8k, shape_rows);
        add(q + "_r1", fam_q8k, 4, 2, f.type, 1, check_gemv_q8k, shape_rows);
        add(q + "_r2", fam_q8k, 4, 2, f.type, 2, check_gemv_q8k, shape_rows);
        add(q + "_wide", fam_q8k, 4, 2, f.type, 2, check_gemv_q8k, shape_rows);
        add(q + "_accum", fam_q8k, 4, 2, f.type, 1, check_gemv_q8k, shape_rows);
        add(q + "_bias", fam_q8k, 5, 2, f.type, 1, check_gemv_q8k, shape_rows);
        add(q + "_m", fam_q8k, 4, 4, f.type, 1, check_gemv_q8k_m, shape_rows);
        if (f.type == OJH_Q6_K) add(q + "_mx", "gemv_q8k", 4, 4, f.type, 0, check_gemv_q8k_m, shape_mx);
        if (f.type == OJH_Q6_K) add(q + "_mf", "gemv_q8k", 4, 4, f.type, -1, check_gemv_q8k_m, shape_mf);
        if (f.type == OJH_Q6_K) add(q + "_ml", "gemv_q8k", 4, 4, f.type, -2, check_gemv_q8k_m, shape_ml);
        if (f.type == OJH_Q6_K) add(q + "_mk", "gemv_q8k", 4, 4, f.type, -3, check_gemv_q8k_m, shape_mk);
        if (f.type == OJH_Q6_K) add(q + "_px", "gemv_q8k", 4, 2, f.type, 2, check_gemv_q8k_px, shape_px);
        if (f.type == OJH_Q4_K) {
            std::string fq = "gemv_fq8k_" + t;
            add(q + "_x4_r1", "gemv_q8k", 10, 5, f.type, 1, check_gemv_q8k_x4, shape_rows);
            add(q + "_x4_r2", "gemv_q8k", 10, 5, f.type, 2, check_gemv_q8k_x4, shape_rows);
            add(fq + "_r1", "gemv_q8k", 3, 3, f.type, 1, check_gemv_fq8k, shape_rows);
            add(fq + "_r2", "gemv_q8k", 3, 3, f.type, 2, check_gemv_fq8k, shape_rows);
            add(fq + "_wide", "gemv_q8k", 3, 3, f.type, 2, check_gemv_fq8k, shape_rows);
            add(fq + "_x4_r1", "gemv_q8k", 9, 7, f.type, 1, check_gemv_fq8k_x4, shape_rows);
            add(fq + "_x4_r2", "gemv_q8k", 9, 7, f.type, 2, check_gemv_fq8k_x4, shape_rows);
        }
    }
    add("gemm_q8k_q4k_mf", "gemm_q8k", 4, 6, OJH_Q4_K, 1, check_gemm_q8k, shape_gemm_q8k);
    add("gemm_q8k_q4k_ml", "gemm_q8k", 4, 4, OJH_Q4_K, 1, check_gemm_q8k_ml, shape_ml);
    add("q8k_token_sides", "gemm_q8k", 4, 3, 0, 0, check_gemm_q8k_xt, shape_gemm_q8k_xt);
    add("quantize_q8k_sides", "gemm_q8k", 5, 3, 0, 0, check_quantize_sides, shape_quantize_sides);
    add("quantize_q8k_bf16_sides", "gemm_q8k", 5, 3, 0, 0, check_quantize_sides, shape_quantize_sides);
    add("gemm_q8k_q4k_xt", "gemm_q8k", 5, 5, OJH_Q4_K, 1, check_gemm_q8k_xt, shape_gemm_q8k_xt);
    add("gemm_q8k_q4k_xt64", "gemm_q8k", 5, 5, OJH_Q4_K, 2, check_gemm_q8k_xt, shape_gemm_q8k_xt);
    add("gemm_q8k_q4k_xt64_sr", "gemm_q8k", 7, 6, OJH_Q4_K, 2, check_gemm_q8k_xt_sr, shape_gemm_q8k_xt_sr);
    add("gemv_q8", "gemv_q8", 4, 2, 0, 0, check_gemv_q8, shape_gemv_q8);
    add("gemv_q8_accum", "gemv_q8", 4, 2, 0, 0, check_gemv_q8, shape_gemv_q8);
    add("gemv_q8_bias", "gemv_q8", 5, 2, 0, 2, check_gemv_q8, shape_gemv_q8);
    add("gemv_q8_ksplit", "gemv_q8", 4, 2, 0, 3, check_gemv_q8, shape_gemv_q8);
    add("ffn_gu_q8", "gemv_q8", 6, 3, 0, 4, check_gemv_q8, shape_gemv_q8);
    add("qkv_q8", "gemv_q8", 13, 3, 0, 5, check_gemv_q8, shape_gemv_q8);
    add("embed_q8", "gemv_q8", 3, 2, 0, 6, check_gemv_q8, shape_gemv_q8);
    add("quantize_q8_pertoken", "gemv_q8", 3, 1, 0, 7, check_gemv_q8, shape_gemv_q8);
    add("gemm_q8k_q6k_gs", "gemm_q8k", 4, 4, OJH_Q6_K, 0, check_gemm_q8k_gs, shape_gemm_q8k_gs);
    add("gemm_q8k_q6k_gs_sr", "gemm_q8k", 6, 5, OJH_Q6_K, 1, check_gemm_q8k_gs, shape_gemm_q8k_gs);
    add("gemm_q8k_q5k_gs", "gemm_q8k", 4, 4, OJH_Q5_K, 0, check_gemm_q8k_gs, shape_gemm_q8k_gs);
    add("gemm_q8k_q5k_gs_sr", "gemm_q8k", 6, 5, OJH_Q5_K, 1, check_gemm_q8k_gs, shape_gemm_q8k_gs);
    add("gemm_q8k_q4k_mk", "gemm_q8k", 4, 4, OJH_Q4_K, 2, check_gemm_q8k_ml, shape_mk);
    add("relayout_q4k_q4l", "dequant", 4, 1, OJH_Q4_K, 0, check_relayout, shape_relayout);
    add("embed_q80", "dequant", 2, 2, OJH_Q8_0, 0, check_embed, shape_embed);
    m.back().expert_bufs = 1;
    m.back().bound_first = 0;
    add("embed_q80_g", "dequant", 3, 1, OJH_Q8_0, 0, check_embed, shape_embed);
    m.back().expert_bufs = 1;
    m.back().bound_first = 0;
    add("quantize_q8_1", "q80_dp4a", 4, 1, OJH_Q8_0, 0, check_q80_dp4a, shape_q80_dp4a);
    add("gemv_q80_dp4a", "q80_dp4a", 4, 2, OJH_Q8_0, 1, check_q80_dp4a, shape_q80_dp4a);
    add("gemv_q80_dp4a_bias", "q80_dp4a", 5, 2, OJH_Q8_0, 2, check_q80_dp4a, shape_q80_dp4a);
    add("gemv_q80_dp4a_accum", "q80_dp4a", 4, 2, OJH_Q8_0, 3, check_q80_dp4a, shape_q80_dp4a);
    add("qkv_q80_dp4a", "q80_dp4a", 9, 3, OJH_Q8_0, 4, check_q80_dp4a, shape_q80_dp4a);
    add("ffn_gu_q80_dp4a", "q80_dp4a", 5, 3, OJH_Q8_0, 5, check_q80_dp4a, shape_q80_dp4a);
    add("rows_q8_from_f16", "rowq8", 3, 2, 0, 0, check_rowq8, shape_rowq8);
    add("quant_rows_i8", "rowq8", 3, 2, 0, 1, check_rowq8, shape_rowq8);
    add("matmul_q8row", "rowq8", 5, 3, 0, 2, check_rowq8, shape_rowq8);
    add("matmul_q8row_bias", "rowq8", 6, 3, 0, 3, check_rowq8, shape_rowq8);
    add("matmul_q8row_mt", "rowq8", 6, 3, 0, 4, check_rowq8, shape_rowq8);
    add("matmul_q8row_mt_sr", "rowq8", 8, 4, 0, 5, check_rowq8, shape_rowq8);
    add("matmul_q8row_mt128", "rowq8", 6, 3, 0, 6, check_rowq8, shape_rowq8);
    add("matmul_q8row_dec", "rowq8", 6, 3, 0, 7, check_rowq8, shape_rowq8);
    add("matmul_q8row_dec_l", "rowq8", 6, 3, 0, 8, check_rowq8, shape_rowq8);
    add("ffn_gu_q8k_q4k", "gemv_q8k", 5, 3, OJH_Q4_K, 1, check_ffn_gu, shape_rows);
    add("ffn_gu_q8k_kq", "gemv_q8k", 5, 4, 0, 1, check_ffn_gu_kq, shape_rows);
    add("gemv_q8k_kq_x4", "gemv_q8k", 10, 6, 0, 1, check_gemv_q8k_kq_x4, shape_rows);
    add("rmsnorm_q8k", "gemv_q8k", 5, 4, 0, 0, check_rmsnorm_q8k, shape_rmsnorm);
    add("quantize_q8k", "gemv_q8k", 3, 2, 0, 0, check_quantize, shape_quantize);
    add("quantize_q8k_bf16", "gemv_q8k", 3, 2, 0, 0, check_quantize, shape_quantize);
    add("quantize_q8k_w", "gemv_q8k", 3, 2, 0, 1, check_quantize, shape_quantize);
    add("quantize_q8k_bf16_w", "gemv_q8k", 3, 2, 0, 1, check_quantize, shape_quantize);
    // prefill / verify MFMA tiles: "q8_0" is the reference's spelling for this family
    for (const auto &f : kFormats) {
        if (ojh_float_only(f.type) || ojh_grid_type(f.type)) continue;
        std::string g = std::string("gemm_mm_") + (f.type == OJH_Q8_0 ? "q8_0" : f.tag);
        add(g, "gemm", 3, 4, f.type, 0, check_gemm, shape_gemm);
        add(g + "_sk", "gemm", 3, 4, f.type, 1, check_gemm, shape_gemm);
        add(g + "_m128", "gemm", 3, 4, f.type, 14, check_gemm, shape_gemm);
        add(g + "_m128_sk", "gemm", 3, 4, f.type, 15, check_gemm, shape_gemm);
    }
    // IQ4_NL / IQ4_XS, the legacy 32-weight blocks, MXFP4 and Q2_K / Q3_K (f32-activation formats on the decode path) have loaders
    // in the same tile; the IQ4 pair also in its grouped form
    for (uint32_t t : {(uint32_t)OJH_IQ4_NL, (uint32_t)OJH_IQ4_XS, (uint32_t)OJH_Q4_0, (uint32_t)OJH_Q4_1, (uint32_t)OJH_Q5_0,
                       (uint32_t)OJH_Q5_1, (uint32_t)OJH_MXFP4, (uint32_t)OJH_Q2_K, (uint32_t)OJH_Q3_K}) {
        std::string g = std::string("gemm_mm_") + ojh_format(t)->tag;
        add(g, "gemm", 3, 4, t, 0, check_gemm, shape_gemm);
        add(g + "_sk", "gemm", 3, 4, t, 1, check_gemm, shape_gemm);
        add(g + "_m128", "gemm", 3, 4, t, 14, check_gemm, shape_gemm);
        add(g + "_m128_sk", "gemm", 3, 4, t, 15, check_gemm, shape_gemm);
        if (t == OJH_IQ4_NL || t == OJH_IQ4_XS)
            add(std::string("moe_mm_") + ojh_format(t)->tag, "gemm", 7, 5, t, 0, check_moe_mm, shape_moe_mm);
    }
    // a few tokens: 16 rows per workgroup, the weights decoded straight into the matrix operand
    for (uint32_t t : {(uint32_t)OJH_Q8_0, (uint32_t)OJH_F16, (uint32_t)OJH_IQ4_NL, (uint32_t)OJH_IQ4_XS, (uint32_t)OJH_Q4_0,
                       (uint32_t)OJH_Q4_1, (uint32_t)OJH_Q5_0, (uint32_t)OJH_Q5_1, (uint32_t)OJH_MXFP4, (uint32_t)OJH_Q2_K,
                       (uint32_t)OJH_Q3_K}) {
        const std::string g = std::string("gemm_few_") + (t == OJH_Q8_0 ? "q8_0" : t == OJH_F16 ? "f16" : ojh_format(t)->tag);
        for (int tg : {1, 2, 4}) {
            add(g + "_t" + std::to_string(tg), "gemm", 3, 4, t, 16 + tg, check_gemm_few, shape_gemm_few);
            add(g + "_r4_t" + std::to_string(tg), "gemm", 3, 4, t, 64 + tg, check_gemm_few, shape_gemm_few);
        }
    }
    // plain f16 rows on the same tile: what every format without a tile of its own is decoded into ahead of a batch
    add("gemm_mm_f16", "gemm", 3, 4, OJH_F16, 0, check_gemm, shape_gemm);
    add("gemm_mm_f16_sk", "gemm", 3, 4, OJH_F16, 1, check_gemm, shape_gemm);
    add("gemm_mm_f16_m128", "gemm", 3, 4, OJH_F16, 14, check_gemm, shape_gemm);
    add("gemm_mm_f16_m128_sk", "gemm", 3, 4, OJH_F16, 15, check_gemm, shape_gemm);
    // Q4L (relaid Q4_K + side arrays) under the reference's names and argument lists
    add("gemm_mm_q4l", "gemm", 5, 4, 0, 8, check_gemm_q4l, shape_gemm);
    add("gemm_mm_q4l_sk", "gemm", 5, 4, 0, 9, check_gemm_q4l, shape_gemm);
    add("gemm_mm_q4l_hb", "gemm", 5, 4, 0, 10, check_gemm_q4l, shape_gemm);
    // Q4_K with the arithmetic of the reference's `gemm_mm_q4l` (f16 qa*q + qb), 256-wide tiles
    add("gemm_mm_q4kl_bdk", "gemm_xl", 3, 4, OJH_Q4_K, 12, check_gemm, shape_gemm);
    add("gemm_mm_q4kl_bdk_sk", "gemm_xl", 3, 4, OJH_Q4_K, 13, check_gemm, shape_gemm);
    add("gemm_mm_q4kl_bd_sr", "gemm_xl", 5, 5, OJH_Q4_K, 128, check_gemm_sr, shape_gemm_sr);
    add("gemm_mm_q4kl_bd256_sr", "gemm_xl", 5, 5, OJH_Q4_K, 256, check_gemm_sr, shape_gemm_sr);
    add("gemm_mm_q4kl", "gemm_xl", 3, 4, OJH_Q4_K, 2, check_gemm, shape_gemm);
    add("gemm_mm_q4kl_sk", "gemm_xl", 3, 4, OJH_Q4_K, 3, check_gemm, shape_gemm);
    add("gemm_mm_q4kl_bd", "gemm_xl", 3, 4, OJH_Q4_K, 6, check_gemm, shape_gemm);      // 128 x 256, weights dequantized into B registers
    add("gemm_mm_q4kl_bd_sk", "gemm_xl", 3, 4, OJH_Q4_K, 7, check_gemm, shape_gemm);
    add("gemm_mm_q4kl_bd256", "gemm_xl", 3, 4, OJH_Q4_K, 2, check_gemm, shape_gemm);   // ... 256 x 256
    add("gemm_mm_q4kl_bd256_sk", "gemm_xl", 3, 4, OJH_Q4_K, 3, check_gemm, shape_gemm);
    // MoE: `rows_per_wave` selects the kernel inside check_moe / shape_moe
    add("moe_topk", "moe", 3, 2, 0, 0, check_moe, shape_moe);
    add("moe_topk_nonorm", "moe", 3, 2, 0, 18, check_moe, shape_moe);
    add("moe_topk_v3", "moe", 4, 4, 0, 19, check_moe, shape_moe);
    add("moe_topk_m", "moe", 3, 2, 0, 1, check_moe, shape_moe);
    add("moe_group", "moe", 4, 2, 0, 2, check_moe, shape_moe);
    add("moe_quant_group", "moe", 7, 4, 0, 20, check_moe, shape_moe);
    add("moe_gu_q4k_m", "moe", 7, 4, OJH_Q4_K, 3, check_moe, shape_moe);
    add("moe_down_q4k_m", "moe", 6, 3, OJH_Q4_K, 4, check_moe, shape_moe);
    add("moe_combine", "moe", 3, 4, 0, 5, check_moe, shape_moe);
    add("moe_gu_q4k_mm", "moe", 7, 4, OJH_Q4_K, 6, check_moe, shape_moe);
    add("moe_down_q4k_mm", "moe", 6, 3, OJH_Q4_K, 7, check_moe, shape_moe);
    add("moe_gu_q4k_mt", "moe", 7, 4, OJH_Q4_K, 12, check_moe, shape_moe);
    add("moe_down_q4k_mt", "moe", 6, 3, OJH_Q4_K, 13, check_moe, shape_moe);
    add("moe_gu_q4k_dec", "moe", 5, 5, OJH_Q4_K, 8, check_moe, shape_moe);
    add("moe_gu_q4k_decr", "moe", 7, 5, OJH_Q4_K, 21, check_moe, shape_moe);
    add("moe_down_q4k_dec", "moe", 5, 5, OJH_Q4_K, 9, check_moe, shape_moe);
    add("moe_gu_q4k_slots", "moe", 6, 6, OJH_Q4_K, 10, check_moe, shape_moe);
    add("moe_down_q4k_slots", "moe", 5, 5, OJH_Q4_K, 11, check_moe, shape_moe);
    add("moe_down_q5k_m", "moe", 6, 3, OJH_Q5_K, 4, check_moe, shape_moe);
    add("moe_down_q5k_gs", "gemm_q8k", 6, 3, OJH_Q5_K, 22, check_moe, shape_moe);
    add("moe_down_q6k_gs", "gemm_q8k", 6, 3, OJH_Q6_K, 22, check_moe, shape_moe);
    add("moe_down_q5k_dec", "moe", 5, 5, OJH_Q5_K, 9, check_moe, shape_moe);
    add("moe_gu_q80", "moe", 5, 2, OJH_Q8_0, 14, check_moe, shape_moe);
    m.back().expert_bufs = 2;
    add("moe_down_q80", "moe", 5, 3, OJH_Q8_0, 15, check_moe, shape_moe);
    m.back().expert_bufs = 1;
    add("moe_gu_q80_slots", "moe", 6, 2, OJH_Q8_0, 16, check_moe, shape_moe);
    m.back().arena_bufs = 2;
    add("moe_down_q80_slots", "moe", 5, 3, OJH_Q8_0, 17, check_moe, shape_moe);
    m.back().arena_bufs = 1;
    // the reference keeps the IQ expert kernels in a family of their own (crates/ojas-cuda/src/kernels/mod.rs:111-145)
    for (uint32_t ty : {(uint32_t)OJH_IQ4_XS, (uint32_t)OJH_IQ4_NL}) {
        std::string tag = ojh_format(ty)->tag;
        add("moe_gu_" + tag, "moe_iq", 5, 2, ty, 14, check_moe, shape_moe);
        m.back().expert_bufs = 2;
        add("moe_down_" + tag, "moe_iq", 5, 3, ty, 15, check_moe, shape_moe);
        m.back().expert_bufs = 1;
    }
    // ... and the grid-codebook rows of the expert table (crates/ojas-core/src/quant_src.rs:180-190)
    for (uint32_t ty : {(uint32_t)OJH_IQ3_S, (uint32_t)OJH_IQ2_XXS, (uint32_t)OJH_IQ2_S}) {
        add(std::string("moe_gu_") + ojh_format(ty)->tag, "moe_iq", 5, 2, ty, 14, check_moe, shape_moe);
        m.back().expert_bufs = 2;
    }
    for (uint32_t ty : {(uint32_t)OJH_IQ2_XXS, (uint32_t)OJH_IQ3_XXS}) {
        add(std::string("moe_down_") + ojh_format(ty)->tag, "moe_iq", 5, 3, ty, 15, check_moe, shape_moe);
        m.back().expert_bufs = 1;
    }
    add("moe_gu_iq3s_slots", "moe_iq", 6, 2, OJH_IQ3_S, 16, check_moe, shape_moe);
    m.back().arena_bufs = 2;
    // K-quant experts on f32 activations, the reference's names (crates/ojas-core/src/quant_src.rs:174-179)
    add("moe_gu_q4k", "moe", 5, 2, OJH_Q4_K, 14, check_moe, shape_moe);
    m.back().expert_bufs = 2;
    for (uint32_t ty : {(uint32_t)OJH_Q4_K, (uint32_t)OJH_Q5_K, (uint32_t)OJH_Q6_K}) {
        add(std::string("moe_down_") + ojh_format(ty)->tag, "moe", 5, 3, ty, 15, check_moe, shape_moe);
        m.back().expert_bufs = 1;
    }
    add("moe_down_q6k_m", "moe", 6, 3, OJH_Q6_K, 4, check_moe, shape_moe);
    add("moe_down_q6k_dec", "moe", 5, 5, OJH_Q6_K, 9, check_moe, shape_moe);
    add("copy_bf16_half", "glue", 2, 1, (2u << 8) | 2u, 0, check_elementwise, shape_elementwise);
    // glue: `type` carries (input element bytes << 8 | output element bytes)
    add("moe_mm_q8_0", "gemm", 7, 5, OJH_Q8_0, 0, check_moe_mm, shape_moe_mm);
    add("moe_mm_f16", "gemm", 7, 5, OJH_F16, 0, check_moe_mm, shape_moe_mm);
    add("moe_few_q8_0", "gemm", 7, 5, OJH_Q8_0, 2, check_moe_mm, shape_moe_mm);
    add("moe_few_iq4nl", "gemm", 7, 5, OJH_IQ4_NL, 2, check_moe_mm, shape_moe_mm);
    add("moe_few_iq4xs", "gemm", 7, 5, OJH_IQ4_XS, 2, check_moe_mm, shape_moe_mm);
    add("moe_act_half", "gemm", 3, 1, 0, 1, check_moe_mm, shape_moe_mm);
    add("copy_f32_half", "glue", 2, 1, (4u << 8) | 2u, 0, check_elementwise, shape_elementwise);
    add("copy_f32_bf16", "glue", 2, 1, (4u << 8) | 2u, 0, check_elementwise, shape_elementwise);
    add("copy_bf16_f32", "glue", 2, 1, (2u << 8) | 4u, 0, check_elementwise, shape_elementwise);
    add("fill_zero_u32", "glue", 1, 1, 4u, 0, check_elementwise, shape_elementwise);
    add("copy_bf16_half_zero", "glue", 3, 3, (2u << 8) | 2u, 0, check_convert_zero, shape_convert_zero);
    add("copy_f32_half_zero", "glue", 3, 3, (4u << 8) | 2u, 0, check_convert_zero, shape_convert_zero);
    add("stream_copy_u32x4", "glue", 2, 1, 0, 0, check_stream, shape_stream);
    add("stream_read_u32x4", "glue", 2, 1, 1, 0, check_stream, shape_stream);
    add("calib_mfma_f16", "glue", 2, 2, 0, 0, check_calib_mfma, shape_calib_mfma);
    add("calib_mfma_i8", "glue", 2, 2, 0, 0, check_calib_mfma, shape_calib_mfma);
    add("decode_chain_q4k", "chain", 0, 0, OJH_Q4_K, 2, check_chain, shape_chain);
    return m;
}

const std::vector<ojh_kernel_spec> &ojh_manifest_table() {
    static const std::vector<ojh_kernel_spec> table = build_manifest();
    return table;
}

const ojh_kernel_spec *ojh_find_kernel(const char *name) {
    if (!name) return nullptr;
    for (const auto &s : ojh_manifest_table())
        if (!strcmp(s.name, name)) return &s;
    return nullptr;
}

extern "C" const char *ojh_kernel_family(const char *name) {
    const ojh_kernel_spec *s = ojh_find_kernel(name);
    return s ? s->family : nullptr;
}

extern "C" int ojh_manifest(int i, const char **name, const char **family, int *n_bufs, int *n_consts) {
    const auto &t = ojh_manifest_table();
    if (i >= 0 && i < (int)t.size()) {
        if (name) *name = t[i].name;
        if (family) *family = t[i].family;
        if (n_bufs) *n_bufs = t[i].n_bufs;
        if (n_consts) *n_consts = t[i].n_consts;
    }
    return (int)t.size();
}

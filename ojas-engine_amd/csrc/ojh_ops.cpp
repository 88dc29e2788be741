// Host side of the op seam: weight handles that keep GGUF block bytes in place, and the matmul
// router that picks a kernel per call — the role `Lin::load` and `CudaSsm::mm` play in the
// reference (crates/ojas-cuda/src/qwen35.rs:174-201, :644-702; Metal twin
// crates/ojas-models/src/decoder/dispatch.rs:288-626).
#include <cstdlib>
#include <cstring>

#include "ojh_internal.h"

static int ensure(ojh_device *dev, const char *family) {
    return dev->modules.count(family) ? OJH_OK : ojh_ensure_family(dev, family);
}

static int span_ok(const char *what, const ojh_buf *b, size_t off, size_t bytes, size_t align) {
    if (!b) return ojh_fail(OJH_ERR_ARG, "%s: NULL buffer", what);
    if (off > b->bytes || bytes > b->bytes - off)
        return ojh_fail(OJH_ERR_BOUNDS, "%s needs %zu bytes at offset %zu, buffer has %zu", what, bytes, off,
                        b->bytes);
    if (((uintptr_t)b->ptr + off) % align)
        return ojh_fail(OJH_ERR_ARG, "%s (+%zu) must be %zu-byte aligned", what, off, align);
    return OJH_OK;
}

static inline void *at(const ojh_buf *b, size_t off) { return (char *)b->ptr + off; }

// ---- Lin ---------------------------------------------------------------------------------------
static int lin_check(uint32_t type, uint32_t n, uint32_t k, size_t *row_bytes) {
    const ojh_block_format *f = ojh_format(type);
    if (!f) return ojh_fail(OJH_ERR_UNSUPPORTED, "GGUF type %u has no kernel on this backend", type);
    if (!n || !k || k % f->weights)
        return ojh_fail(OJH_ERR_ARG, "Lin %ux%u: K must be a positive multiple of %u for %s", n, k, f->weights,
                        f->tag);
    *row_bytes = (size_t)(k / f->weights) * f->bytes;
    return OJH_OK;
}

extern "C" int ojh_lin_create(ojh_device *dev, uint32_t type, uint32_t n, uint32_t k, const void *raw,
                              ojh_lin **out) {
    if (!dev || !raw || !out) return ojh_fail(OJH_ERR_ARG, "ojh_lin_create: NULL argument");
    *out = nullptr;
    size_t rb;
    int rc = lin_check(type, n, k, &rb);
    if (rc) return rc;
    ojh_buf *buf = nullptr;
    // up to the next multiple of 16: kernels that copy whole aligned 16-byte pieces may read that far
    if ((rc = ojh_alloc(dev, (rb * n + 15) & ~(size_t)15, &buf))) return rc;
    if ((rc = ojh_upload(dev, buf, 0, raw, rb * n))) {
        ojh_free(dev, buf);
        return rc;
    }
    ojh_lin *l = new ojh_lin();
    l->type = type; l->n = n; l->k = k; l->row_bytes = rb; l->raw = buf; l->off = 0; l->owns_raw = true;
    *out = l;
    return OJH_OK;
}

extern "C" int ojh_lin_wrap(ojh_device *dev, uint32_t type, uint32_t n, uint32_t k, ojh_buf *raw, size_t off,
                            ojh_lin **out) {
    if (!dev || !raw || !out) return ojh_fail(OJH_ERR_ARG, "ojh_lin_wrap: NULL argument");
    *out = nullptr;
    size_t rb;
    int rc = lin_check(type, n, k, &rb);
    if (rc) return rc;
    const ojh_block_format *f = ojh_format(type);
    if ((rc = span_ok("ojh_lin_wrap: raw", raw, off, rb * n, ojh_block_align(f)))) return rc;
    ojh_lin *l = new ojh_lin();
    l->type = type; l->n = n; l->k = k; l->row_bytes = rb; l->raw = raw; l->off = off; l->owns_raw = false;
    *out = l;
    return OJH_OK;
}

extern "C" int ojh_lin_free(ojh_device *dev, ojh_lin *lin) {
    if (!lin) return OJH_OK;
    int rc = OJH_OK;
    if (lin->owns_raw) rc = ojh_free(dev, lin->raw);
    delete lin;
    return rc;
}

// ---- dequant -----------------------------------------------------------------------------------
extern "C" int ojh_dequant_f16(ojh_device *dev, uint32_t type, const ojh_buf *raw, size_t raw_off,
                               size_t n_weights, ojh_buf *out, size_t out_off) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_dequant_f16: NULL device");
    const ojh_block_format *f = ojh_format(type);
    if (!f) return ojh_fail(OJH_ERR_UNSUPPORTED, "GGUF type %u has no decoder on this backend", type);
    if (!n_weights || n_weights % f->weights)
        return ojh_fail(OJH_ERR_ARG, "dequant: %zu weights is not a positive multiple of %u", n_weights, f->weights);
    size_t nb = n_weights / f->weights;
    if (nb > 0x7FFFFFFFu / 64) return ojh_fail(OJH_ERR_ARG, "dequant: too many blocks in one call (%zu)", nb);
    int rc;
    if ((rc = span_ok("dequant: raw", raw, raw_off, nb * f->bytes, ojh_block_align(f)))) return rc;
    if ((rc = span_ok("dequant: out", out, out_off, n_weights * 2, 2))) return rc;
    if ((rc = ensure(dev, ojh_grid_type(type) ? "iq_grid" : "dequant"))) return rc;
    std::string name = std::string("dequant_") + f->tag + "_f16";
    uint32_t grid[3], block[3];
    if ((rc = ojh_launch_shape(dev, name.c_str(), 0, (uint32_t)nb, 0, grid, block))) return rc;
    return ojh_launch(dev, name.c_str(), {at(raw, raw_off), at(out, out_off)}, {(uint32_t)nb}, grid, block);
}

extern "C" int ojh_relayout_q4k_q4l(ojh_device *dev, const ojh_buf *raw, size_t raw_off, uint32_t n, uint32_t k,
                                    ojh_buf *nib, ojh_buf *qa, ojh_buf *qb) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_relayout_q4k_q4l: NULL device");
    if (!n || !k || k % 256) return ojh_fail(OJH_ERR_ARG, "relayout_q4k_q4l: %u rows of %u weights (K must be a multiple of 256)", n, k);
    size_t nb = (size_t)n * (k / 256);
    if (nb > 0x0FFFFFFFu) return ojh_fail(OJH_ERR_ARG, "relayout_q4k_q4l: too many super-blocks (%zu)", nb);
    int rc;
    if ((rc = span_ok("relayout: raw", raw, raw_off, nb * 144, 16))) return rc;
    if ((rc = span_ok("relayout: nib", nib, 0, nb * 128, 16))) return rc;
    if ((rc = span_ok("relayout: qa", qa, 0, nb * 16, 2))) return rc;
    if ((rc = span_ok("relayout: qb", qb, 0, nb * 16, 2))) return rc;
    if ((rc = ensure(dev, "dequant"))) return rc;
    uint32_t grid[3] = {(uint32_t)((nb + 31) / 32), 1, 1}, block[3] = {256, 1, 1};
    return ojh_launch(dev, "relayout_q4k_q4l", {at(raw, raw_off), nib->ptr, qa->ptr, qb->ptr}, {(uint32_t)nb}, grid, block);
}

// ---- activation quantizer ----------------------------------------------------------------------
int ojh_quant_q8k_launch(ojh_device *dev, const void *x, int x_dtype, uint32_t m, uint32_t k, void *q,
                            void *scales) {
    const char *name = x_dtype == OJH_X_BF16 ? "quantize_q8k_bf16" : "quantize_q8k";
    uint32_t grid[3] = {(k + 255) / 256, m, 1}, block[3] = {256, 1, 1};
    // many segments (a batch): a segment per wave, four to a workgroup
    const uint64_t segs = (uint64_t)grid[0] * m;
    if (segs >= 1024) {
        uint32_t gw[3] = {(uint32_t)((segs + 3) / 4), 1, 1};
        return ojh_launch(dev, x_dtype == OJH_X_BF16 ? "quantize_q8k_bf16_w" : "quantize_q8k_w", {(void *)x, q, scales}, {k, m}, gw, block);
    }
    return ojh_launch(dev, name, {(void *)x, q, scales}, {k, m}, grid, block);
}

extern "C" int ojh_quant_q8k(ojh_device *dev, const ojh_buf *x, size_t x_off, int x_dtype, uint32_t m,
                             uint32_t k, ojh_buf *q, ojh_buf *scales) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_quant_q8k: NULL device");
    if (x_dtype != OJH_X_F32 && x_dtype != OJH_X_BF16)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "quant_q8k takes f32 or bf16 activations");
    if (!m || !k || m > 65535) return ojh_fail(OJH_ERR_ARG, "quant_q8k: m=%u k=%u out of range", m, k);
    size_t esz = x_dtype == OJH_X_BF16 ? 2 : 4, nsb = (k + 255) / 256;
    int rc;
    if ((rc = span_ok("quant_q8k: x", x, x_off, (size_t)m * k * esz, esz))) return rc;
    if ((rc = span_ok("quant_q8k: q", q, 0, (size_t)m * nsb * 256, 16))) return rc;
    if ((rc = span_ok("quant_q8k: scales", scales, 0, (size_t)m * nsb * 4, 4))) return rc;
    if ((rc = ensure(dev, "gemv_q8k"))) return rc;
    return ojh_quant_q8k_launch(dev, at(x, x_off), x_dtype, m, k, q->ptr, scales->ptr);
}

// ---- mm ----------------------------------------------------------------------------------------
// Rows per wave for the row-parallel matvecs: enough waves to put several on every SIMD, while
// reusing each activation fragment across as many rows as that allows.
static int pick_rows(const ojh_device *dev, uint32_t n) {
    if (dev->gemv_rows_override == 1 || dev->gemv_rows_override == 2 || dev->gemv_rows_override == 4)
        return dev->gemv_rows_override;
    uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
    // Measured on MI355X (Q4_K, K=4096): two rows per wave streams fastest once N gives every CU
    // several workgroups; four rows per wave loses to it at every size.
    return n >= cus * 32u ? 2 : 1;
}

// y (=,+=,+bias) quantized-x . W^T for K-quant weights: the matvec (m = 1) and its batched form.
// Whether a Q4_K product of m tokens takes the 128-token int8 tile (when its tiles cover at least half of the CUs: a
// 4096-row matrix against 128 tokens stays below).
// K slices the 64-row int8 tile is launched over (measured on 4096 / 14336-wide matrices at 128 .. 2048 tokens): two
// workgroups per CU is the aim, with at most eight slices of at least four super-blocks each (two, where four would
// leave more than half the CUs idle); a grid that already covers more than half the CUs is sliced only when a slice
// keeps sixteen super-blocks.  1 = unsliced; 0 = even sliced, most CUs would idle: another kernel takes the product.
static uint32_t q4k_xt_slices(const ojh_device *dev, uint32_t K, uint32_t N, uint32_t m) {
    const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount, nsb = K / 256;
    const uint64_t tiles = (uint64_t)((N + 63) / 64) * ((m + 127) / 128);
    const uint32_t whole = tiles * 2 >= cus ? 1u : 0u;
    if (dev->q4k_xt_split == 0 || (tiles > cus && dev->q4k_xt_split == 1)) return whole;
    uint32_t z = (uint32_t)(2 * (uint64_t)cus / tiles);
    if (z > 8) z = 8;
    uint32_t cap = nsb / 4;
    if (tiles * (z < cap ? z : cap) * 2 < cus) cap = nsb / 2;
    if (z > cap) z = cap;
    if (tiles * 2 > cus && z > 1 && nsb / z < 16) z = 1;
    if (dev->q4k_xt_split > 1) z = dev->q4k_xt_split <= nsb ? dev->q4k_xt_split : nsb;
    if (z < 2 || tiles * z * 2 < cus) return whole;
    return ojh_gemm_sr_slices(K, z);
}
// Tokens from which that tile is taken (measured with the rows streamed from HBM, K = 2048 .. 14336): the tile costs
// the same from 1 to 128 tokens, the matrix-core kernel below it doubles past 32 tokens.  So from 33 tokens; from 17
// where K is at least twice the row count (few tiles, each a long walk: 4096 x 14336 takes 38 us here against 45);
// and only from 65 for a matrix of more than one and a half 64-row tiles per CU, where two 32-token passes of the
// other kernel are still ahead (32000 x 4096 at 64 tokens: 56 us against 62).
static uint32_t q4k_xt_min_tokens(const ojh_device *dev, uint32_t K, uint32_t N) {
    if (dev->q4k_xt_min_m != 1) return dev->q4k_xt_min_m;
    const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
    if (2 * (uint64_t)((N + 63) / 64) > 3ull * cus) return 65;
    return K >= 2ull * N ? 17 : 33;
}
bool ojh_q4k_xt_taken(const ojh_device *dev, const ojh_lin *w, uint32_t m, const void *wp) {
    const uint32_t K = w->k, N = w->n;
    return w->type == OJH_Q4_K && dev->q4k_xt_min_m && m >= q4k_xt_min_tokens(dev, K, N) && !dev->no_scratch &&
           q4k_xt_slices(dev, K, N, m) >= 1 &&
           (uint64_t)m * K <= 0xFFFFFFFFull && (uint64_t)w->row_bytes * N <= 0xFFFFFFFFull && (uintptr_t)wp % 16 == 0;
}

int ojh_mm_q8k_launch(ojh_device *dev, void *xq, void *xs, const ojh_lin *w, const ojh_block_format *f, void *yp,
                         const ojh_buf *bias, uint32_t m, int accum, bool sides_ready) {
    const uint32_t K = w->k, N = w->n;
    void *wp = at(w->raw, w->off);
    uint32_t grid[3] = {1, 1, 1}, block[3] = {256, 1, 1};
    std::string base = std::string("gemv_q8k_") + f->tag;
    // an output head: rows grid-stride, activations in registers
    if (m == 1 && w->type == OJH_Q6_K && dev->px && !accum && !bias && N >= 32768u && K <= 8192u) {
        uint32_t sg[3], sb[3];
        const std::string name = base + "_px";
        int rc = ojh_launch_shape(dev, name.c_str(), K, N, 1, sg, sb);
        if (rc) return rc;
        return ojh_launch(dev, name.c_str(), {xq, xs, wp, yp}, {K, N}, sg, sb);
    }
    if (m == 1) {
        int r = (accum || bias) ? 1 : pick_rows(dev, N);
        bool wide = !accum && !bias && r == 2 && N >= 32768u;
        std::string name = base + (accum ? "_accum" : bias ? "_bias" : wide ? "_wide" : r == 4 ? "" : r == 2 ? "_r2" : "_r1");
        grid[0] = (N + 4 * r - 1) / (4 * r);
        std::vector<void *> p = {xq, xs, wp, yp};
        if (bias) p.push_back(bias->ptr);
        return ojh_launch(dev, name.c_str(), p, {K, N}, grid, block);
    }
    // Q4_K rows against a prefill-sized batch: 128 x 128 tiles, the tokens copied into LDS by the memory system
    // (needs two side arrays, built by one small launch into the library's scratch — or by the quantizer itself when
    // ojh_mm quantizes: it then comes here with the side arrays ready)
    if (ojh_q4k_xt_taken(dev, w, m, wp)) {
        int rc = ensure(dev, "gemm_q8k");
        if (rc) return rc;
        const uint32_t mp = (m + 127) / 128 * 128;
        const size_t nsb = K / 256;
        ojh_buf *xst, *sums;
        if ((rc = ojh_scratch_get(dev, "xt_xst", nsb * mp * 4, &xst))) return rc;
        if ((rc = ojh_scratch_get(dev, "xt_sums", nsb * mp * 32, &sums))) return rc;
        uint32_t sg[3], sb[3];
        if (!sides_ready) {
            if ((rc = ojh_launch_shape(dev, "q8k_token_sides", K, N, m, sg, sb))) return rc;
            if ((rc = ojh_launch(dev, "q8k_token_sides", {xq, xs, xst->ptr, sums->ptr}, {K, m, mp}, sg, sb))) return rc;
        }
        // too few 64-row tiles for the chip: K slices of them, summed in slice order by the last to finish
        if (const uint32_t z = q4k_xt_slices(dev, K, N, m); z > 1) {
            const size_t tiles = (size_t)((N + 63) / 64) * (mp / 128);
            ojh_buf *part, *cnt;
            if ((rc = ojh_scratch_get(dev, "xt_part", tiles * z * 32768, &part))) return rc;
            if ((rc = ojh_scratch_get_zeroed(dev, "xt_cnt", tiles * 4, &cnt))) return rc;
            sg[0] = (N + 63) / 64; sg[1] = mp / 128; sg[2] = z;
            sb[0] = 512; sb[1] = sb[2] = 1;
            return ojh_launch(dev, "gemm_q8k_q4k_xt64_sr", {xq, xst->ptr, sums->ptr, wp, yp, part->ptr, cnt->ptr},
                              {K, N, m, (uint32_t)(accum != 0), mp, z}, sg, sb);
        }
        // 128-row tiles when they give every CU one, 64-row tiles otherwise
        const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
        const char *xt = (uint64_t)((N + 127) / 128) * (mp / 128) >= cus && !dev->q4k_xt64 ? "gemm_q8k_q4k_xt" : "gemm_q8k_q4k_xt64";
        if ((rc = ojh_launch_shape(dev, xt, K, N, m, sg, sb))) return rc;
        return ojh_launch(dev, xt, {xq, xst->ptr, sums->ptr, wp, yp}, {K, N, m, (uint32_t)(accum != 0), mp}, sg, sb);
    }
    // Q4_K rows against several tokens: the int8 matrix cores, in the shape measured fastest on K = 4096 and 14336.
    // A long matrix (six 16-row tiles per CU and wave: 24576 rows on this GPU) against 2 .. 16 tokens: a wave
    // per tile, rows copied through LDS.
    if (w->type == OJH_Q4_K && dev->q4k_ml_min_m && m >= dev->q4k_ml_min_m && m <= 16 &&
        (N + 15) / 16 >= 6u * (uint32_t)dev->prop.multiProcessorCount && ojh_gemm_q8k_ml_lds(K) <= 163840 &&
        (uint64_t)w->row_bytes * N <= 0xFFFFFFFFull && (uintptr_t)wp % 16 == 0) {
        int rc = ensure(dev, "gemm_q8k");
        if (rc) return rc;
        uint32_t sg[3], sb[3];
        if ((rc = ojh_launch_shape(dev, "gemm_q8k_q4k_ml", K, N, m, sg, sb))) return rc;
        return ojh_launch(dev, "gemm_q8k_q4k_ml", {xq, xs, wp, yp}, {K, N, m, (uint32_t)(accum != 0)}, sg, sb);
    }
    // Few rows (up to a tile and a half per CU: 6144 rows) against 5 .. 16 tokens that fit LDS whole: a
    // workgroup per tile, its eight waves splitting K (a third faster than the general tiling at K = 14336).
    if (w->type == OJH_Q4_K && m >= dev->q4k_mf_min_m && m <= 16 && 2 * ((N + 15) / 16) <= 3u * (uint32_t)dev->prop.multiProcessorCount &&
        ojh_gemm_q8k_mk_lds(K, m) <= 163840 && (uintptr_t)wp % 16 == 0) {
        int rc = ensure(dev, "gemm_q8k");
        if (rc) return rc;
        uint32_t sg[3], sb[3];
        if ((rc = ojh_launch_shape(dev, "gemm_q8k_q4k_mk", K, N, m, sg, sb))) return rc;
        return ojh_launch(dev, "gemm_q8k_q4k_mk", {xq, xs, wp, yp}, {K, N, m, (uint32_t)(accum != 0)}, sg, sb);
    }
    // (from 5 tokens; from 3 on an output head, where the per-token loop of the dot kernel costs most)
    if (w->type == OJH_Q4_K && (m >= dev->q4k_mf_min_m || (m >= 3 && m + 2 >= dev->q4k_mf_min_m && N >= 32768u))) {
        int rc = ensure(dev, "gemm_q8k");
        if (rc) return rc;
        uint32_t sg[3], sb[3];
        if ((rc = ojh_launch_shape(dev, "gemm_q8k_q4k_mf", K, N, m, sg, sb))) return rc;
        uint32_t rw, rt;
        ojh_gemm_q8k_tiles(dev, K, N, m, &rw, &rt);
        return ojh_launch(dev, "gemm_q8k_q4k_mf", {xq, xs, wp, yp}, {K, N, m, (uint32_t)(accum != 0), rw, rt}, sg, sb);
    }
    const size_t w_bytes = w->row_bytes * N;
    const bool dwords_ok = (uintptr_t)wp % 4 == 0 && (w_bytes % 4 == 0 || w->off + w_bytes + 2 <= w->raw->bytes);
    // Q6_K / Q5_K rows against a batch: 128-row x 64-token tiles, one matrix instruction per scale group;
    // over K slices where the tiles alone would leave CUs idle (partial tiles in library scratch, added in slice order)
    // (from where it was measured ahead of what it replaces, rows streamed from HBM.  Q6_K: from 17 tokens on large
    // matrices — 14336 x 4096 at 24 tokens 28.6 against 39 us for two launches of 16, 4096 x 14336 32.6 against 50 — and
    // from 33 on small ones, where two launches still win (4096 x 4096: 18 against 19.4).  Q5_K, whose few-token form is
    // the integer-dot kernel: from 5 tokens on large matrices (14336 x 4096 at 8 tokens 25.5 against 31.8), from 9 on
    // small ones (4096 x 4096 at 12 tokens 17.8 against 20.5).)
    const bool gs_large = N >= 8192 || K > 8192;
    const uint32_t gs_min = dev->kq_gs_min_m != 1 ? dev->kq_gs_min_m
                            : w->type == OJH_Q6_K ? (gs_large ? 17u : 33u) : (gs_large ? 5u : 9u);
    if ((w->type == OJH_Q6_K || w->type == OJH_Q5_K) && gs_min && m >= gs_min && K % 256 == 0 &&
        (uintptr_t)xq % 16 == 0 && (w->type == OJH_Q6_K ? dwords_ok : (uintptr_t)wp % 16 == 0)) {
        int rc = ensure(dev, "gemm_q8k");
        if (rc) return rc;
        const std::string gs = std::string("gemm_q8k_") + f->tag + "_gs";
        uint32_t sg[3] = {(N + 127) / 128, (m + 63) / 64, 1}, sb[3] = {256, 1, 1};
        const uint32_t z = dev->no_scratch ? 1 : ojh_gemm_q8k_gs_slices(dev, K, N, m);
        if (z > 1) {
            const size_t tiles = (size_t)sg[0] * sg[1];
            ojh_buf *part, *cnt;
            if ((rc = ojh_scratch_get(dev, "gs_part", tiles * z * 32768, &part))) return rc;
            if ((rc = ojh_scratch_get_zeroed(dev, "gs_cnt", tiles * 4, &cnt))) return rc;
            sg[2] = z;
            return ojh_launch(dev, (gs + "_sr").c_str(), {xq, xs, wp, yp, part->ptr, cnt->ptr},
                              {K, N, m, (uint32_t)(accum != 0), z}, sg, sb);
        }
        return ojh_launch(dev, gs.c_str(), {xq, xs, wp, yp}, {K, N, m, (uint32_t)(accum != 0)}, sg, sb);
    }
    // Q6_K rows against 2 or more tokens on the int8 matrix cores (beyond 16 tokens as launches of 16 or 8:
    // each streams the rows once, which the per-token loop of the general entry does sixteen times
    // over).  Three shapes of the same tile arithmetic, picked by what was measured on K = 4096 and 14336:
    //   many rows (eight tiles per CU and wave, 32768 rows on this GPU): a wave per tile, rows copied
    //     through LDS, ahead of everything from 2 tokens;
    //   few rows (up to two tiles per CU, 8192 rows): a workgroup per tile, its waves splitting K, ahead of
    //     the integer-dot entry from 5 tokens (from 3 when K is long) and the only one that holds 8 tokens
    //     of K = 14336;
    //   between: a wave per tile with direct loads, ahead of the integer-dot entry from 5 tokens.
    if (w->type == OJH_Q6_K && m >= 2) {
        const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount, tiles = (N + 15) / 16;
        const uint32_t mc16 = m <= 8 ? m : 16;
        const bool ml_fits = dev->q6k_ml && (uint64_t)w_bytes <= 0xFFFFFFFFull && ojh_q6k_ml_lds(K, mc16) <= 163840 &&
                             (uintptr_t)wp % 16 == 0 && w->off + ((w_bytes + 15) & ~(size_t)15) <= w->raw->bytes;
        const bool mf_fits = dwords_ok && (uint64_t)(m <= 8 ? 8 : 16) * (K + 32) + K / 4 + 256 <= 69632;
        const bool mk16 = dwords_ok && ojh_q6k_mk_lds(K, mc16) <= 163840, mk8 = dwords_ok && ojh_q6k_mk_lds(K, 8) <= 163840;
        const bool mx_fits = m <= 16 && (uint64_t)m * ((K + 4095) / 4096) <= 19;
        const char *entry = nullptr;
        uint32_t step = 16;
        if (ml_fits && m >= dev->q6k_ml_min_m && tiles >= 8 * cus) {
            entry = "gemv_q8k_q6k_ml";
        } else if (tiles <= 2 * cus && (mk16 || mk8) && (m >= dev->q6k_mf_min_m || (m >= 3 && K > 8192) || !mx_fits)) {
            entry = "gemv_q8k_q6k_mk";
            step = mk16 ? 16 : 8;
        } else if (mf_fits && (m >= dev->q6k_mf_min_m || !mx_fits)) {
            entry = "gemv_q8k_q6k_mf";
        } else if (!mx_fits && (mk16 || mk8)) {
            entry = "gemv_q8k_q6k_mk";
            step = mk16 ? 16 : 8;
        } else if (!mx_fits && ml_fits) {
            entry = "gemv_q8k_q6k_ml";
        }
        if (entry) {
            const size_t nsb = K / 256;
            for (uint32_t t0 = 0; t0 < m; t0 += step) {
                const uint32_t mc = m - t0 < step ? m - t0 : step;
                uint32_t sg[3], sb[3];
                int rc = ojh_launch_shape(dev, entry, K, N, mc, sg, sb);
                if (rc) return rc;
                if ((rc = ojh_launch(dev, entry,
                                     {(char *)xq + (size_t)t0 * nsb * 256, (char *)xs + (size_t)t0 * nsb * 4, wp,
                                      (char *)yp + (size_t)t0 * N * 4},
                                     {K, N, mc, (uint32_t)(accum != 0)}, sg, sb)))
                    return rc;
            }
            return OJH_OK;
        }
    }
    // few tokens on Q6_K rows: activations staged in LDS once per workgroup, rows grid-stride
    if (w->type == OJH_Q6_K && m <= 16 && (uint64_t)m * ((K + 4095) / 4096) <= 19) {
        uint32_t sg[3], sb[3];
        int rc = ojh_launch_shape(dev, "gemv_q8k_q6k_mx", K, N, m, sg, sb);
        if (rc) return rc;
        return ojh_launch(dev, "gemv_q8k_q6k_mx", {xq, xs, wp, yp}, {K, N, m, (uint32_t)(accum != 0)}, sg, sb);
    }
    grid[0] = (N + 3) / 4;
    return ojh_launch(dev, (base + "_m").c_str(), {xq, xs, wp, yp}, {K, N, m, (uint32_t)(accum != 0)}, grid, block);
}

int ojh_mm_checks(const char *who, const ojh_lin *w, ojh_buf *y, size_t y_off, const ojh_buf *bias,
                            uint32_t m, int accum, const ojh_block_format **fmt) {
    if (!w) return ojh_fail(OJH_ERR_ARG, "%s: NULL weights", who);
    if (!m || m > 65535) return ojh_fail(OJH_ERR_ARG, "%s: m=%u out of range", who, m);
    const ojh_block_format *f = ojh_format(w->type);
    if (!f) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: GGUF type %u", who, w->type);
    if (bias && accum) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: bias and accum together", who);
    if (bias && m != 1) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: bias is a matvec (m=1) epilogue", who);
    int rc;
    if ((rc = span_ok("y", y, y_off, (size_t)m * w->n * 4, 4))) return rc;
    if (bias && (rc = span_ok("bias", bias, 0, (size_t)w->n * 4, 4))) return rc;
    if ((rc = span_ok("w", w->raw, w->off, w->row_bytes * w->n, ojh_block_align(f)))) return rc;
    *fmt = f;
    return OJH_OK;
}

extern "C" int ojh_mm_q8k(ojh_device *dev, const ojh_buf *xq, const ojh_buf *xscales, const ojh_lin *w, ojh_buf *y,
                          size_t y_off, const ojh_buf *bias, uint32_t m, int accum) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_mm_q8k: NULL device");
    const ojh_block_format *f;
    int rc = ojh_mm_checks("ojh_mm_q8k", w, y, y_off, bias, m, accum, &f);
    if (rc) return rc;
    if (ojh_float_rows(w->type))
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm_q8k: %s rows take f32 activations, as their CPU dot does", f->tag);
    size_t nsb = w->k / 256;
    if ((rc = span_ok("xq", xq, 0, (size_t)m * nsb * 256, 16))) return rc;
    if ((rc = span_ok("xscales", xscales, 0, (size_t)m * nsb * 4, 4))) return rc;
    if ((rc = ensure(dev, "gemv_q8k")) || (ojh_grid_type(w->type) && (rc = ensure(dev, "iq_grid")))) return rc;
    return ojh_mm_q8k_launch(dev, xq->ptr, xscales->ptr, w, f, at(y, y_off), bias, m, accum);
}

extern "C" int ojh_mm_q8k_multi(ojh_device *dev, const ojh_buf *xq, const ojh_buf *xscales, int count,
                                const ojh_lin *const *ws, ojh_buf *const *ys, const size_t *y_offs) {
    if (!dev || !ws || !ys) return ojh_fail(OJH_ERR_ARG, "ojh_mm_q8k_multi: NULL argument");
    if (count < 1 || count > 4) return ojh_fail(OJH_ERR_ARG, "ojh_mm_q8k_multi: count=%d, takes 1 to 4 projections", count);
    int rc;
    bool grouped = true;
    uint64_t total = 0;
    for (int i = 0; i < count; i++) {
        const ojh_block_format *fi;
        if ((rc = ojh_mm_checks("ojh_mm_q8k_multi", ws[i], ys[i], y_offs ? y_offs[i] : 0, nullptr, 1, 0, &fi))) return rc;
        if (ojh_float_rows(ws[i]->type))
            return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm_q8k_multi: %s rows take f32 activations, as their CPU dot does", fi->tag);
        if (ws[i]->k != ws[0]->k)
            return ojh_fail(OJH_ERR_ARG, "ojh_mm_q8k_multi: projection %d has K=%u, the first has K=%u", i, ws[i]->k, ws[0]->k);
        if (ws[i]->type != OJH_Q4_K) grouped = false;
        total += ws[i]->n;
    }
    if (total > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_mm_q8k_multi: too many rows");
    size_t nsb = ws[0]->k / 256;
    if ((rc = span_ok("xq", xq, 0, nsb * 256, 16))) return rc;
    if ((rc = span_ok("xscales", xscales, 0, nsb * 4, 4))) return rc;
    if ((rc = ensure(dev, "gemv_q8k"))) return rc;
    for (int i = 0; i < count; i++)
        if (ojh_grid_type(ws[i]->type) && (rc = ensure(dev, "iq_grid"))) return rc;
    // a stage that mixes Q4_K, Q5_K and Q6_K tensors (a Q4_K_M file does): still one launch, every row in its own
    // format's arithmetic
    bool kquants = count > 1;
    for (int i = 0; i < count; i++)
        if (ws[i]->type != OJH_Q4_K && ws[i]->type != OJH_Q5_K && ws[i]->type != OJH_Q6_K) kquants = false;
    if (!grouped && kquants) {
        std::vector<void *> p = {xq->ptr, xscales->ptr};
        uint32_t ends[4], run = 0, types = 0;
        for (int i = 0; i < 4; i++) {
            int j = i < count ? i : count - 1;
            p.push_back(at(ws[j]->raw, ws[j]->off));
            if (i < count) run += ws[i]->n;
            ends[i] = run;
            types |= ws[j]->type << (8 * i);
        }
        for (int i = 0; i < 4; i++) {
            int j = i < count ? i : count - 1;
            p.push_back(at(ys[j], y_offs ? y_offs[j] : 0));
        }
        uint32_t grid[3] = {(run + 3) / 4, 1, 1}, block[3] = {256, 1, 1};
        return ojh_launch(dev, "gemv_q8k_kq_x4", p, {ws[0]->k, ends[0], ends[1], ends[2], ends[3], types}, grid, block);
    }
    if (!grouped || count == 1) {   // formats without a grouped entry: one launch per projection
        for (int i = 0; i < count; i++) {
            const ojh_block_format *fi = ojh_format(ws[i]->type);
            if ((rc = ojh_mm_q8k_launch(dev, xq->ptr, xscales->ptr, ws[i], fi, at(ys[i], y_offs ? y_offs[i] : 0), nullptr, 1, 0)))
                return rc;
        }
        return OJH_OK;
    }
    std::vector<void *> p = {xq->ptr, xscales->ptr};
    uint32_t ends[4], run = 0;
    for (int i = 0; i < 4; i++) {
        int j = i < count ? i : count - 1;
        p.push_back(at(ws[j]->raw, ws[j]->off));
        if (i < count) run += ws[i]->n;
        ends[i] = run;
    }
    for (int i = 0; i < 4; i++) {
        int j = i < count ? i : count - 1;
        p.push_back(at(ys[j], y_offs ? y_offs[j] : 0));
    }
    int r = pick_rows(dev, run);
    if (r == 4) r = 2;
    uint32_t grid[3] = {(run + 4 * r - 1) / (4 * r), 1, 1}, block[3] = {256, 1, 1};
    return ojh_launch(dev, r == 2 ? "gemv_q8k_q4k_x4_r2" : "gemv_q8k_q4k_x4_r1", p,
                      {ws[0]->k, ends[0], ends[1], ends[2], ends[3]}, grid, block);
}

// One stage of a decode layer in ONE launch: 1 to 4 projections of one f32 vector, the vector quantized inside the launch.
extern "C" int ojh_mm_multi(ojh_device *dev, const ojh_buf *x, size_t x_off, int count, const ojh_lin *const *ws,
                            ojh_buf *const *ys, const size_t *y_offs, int accum) {
    if (!dev || !ws || !ys) return ojh_fail(OJH_ERR_ARG, "ojh_mm_multi: NULL argument");
    if (count < 1 || count > 4) return ojh_fail(OJH_ERR_ARG, "ojh_mm_multi: count=%d, takes 1 to 4 projections", count);
    int rc;
    bool fused = true;
    uint64_t total = 0;
    for (int i = 0; i < count; i++) {
        const ojh_block_format *fi;
        if ((rc = ojh_mm_checks("ojh_mm_multi", ws[i], ys[i], y_offs ? y_offs[i] : 0, nullptr, 1, accum, &fi))) return rc;
        if (ojh_float_rows(ws[i]->type))
            return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm_multi: %s rows take f32 activations and need no quantizer: call ojh_mm", fi->tag);
        if (ws[i]->k != ws[0]->k)
            return ojh_fail(OJH_ERR_ARG, "ojh_mm_multi: projection %d has K=%u, the first has K=%u", i, ws[i]->k, ws[0]->k);
        if (ws[i]->type != OJH_Q4_K) fused = false;
        total += ws[i]->n;
    }
    if (total > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_mm_multi: too many rows");
    const uint32_t K = ws[0]->k;
    if ((rc = span_ok("ojh_mm_multi: x", x, x_off, (size_t)K * 4, 16))) return rc;
    if ((rc = ensure(dev, "gemv_q8k"))) return rc;
    for (int i = 0; i < count; i++)
        if (ojh_grid_type(ws[i]->type) && (rc = ensure(dev, "iq_grid"))) return rc;
    // Measured on MI355X (weights streamed from HBM): the single launch wins on a small stage (q/k/v of an 8B model:
    // 6.6 against 7.7 us), ties on 4096 x 4096 and loses from there on — few large workgroups cannot keep as many bytes
    // in flight as the plain matvec's thousands of small ones, and many small ones repeat the quantization too often.
    // OJAS_HIP_FQ_MULTI = 0 never takes it, 2 takes it at every size.
    const bool small_stage = total * K <= 32u * 1024u * 1024u && K <= 4096u;
    if (!fused || K > 16384 || dev->fq_multi == 0 || (dev->fq_multi == 1 && !small_stage)) {   // quantize once, then the per-format launches
        size_t nsb = K / 256;
        ojh_buf *xq, *xs;
        if ((rc = ojh_scratch_get(dev, "xq", nsb * 256, &xq))) return rc;
        if ((rc = ojh_scratch_get(dev, "xs", nsb * 4, &xs))) return rc;
        if ((rc = ojh_quant_q8k_launch(dev, at(x, x_off), OJH_X_F32, 1, K, xq->ptr, xs->ptr))) return rc;
        if (!accum) return ojh_mm_q8k_multi(dev, xq, xs, count, ws, ys, y_offs);
        for (int i = 0; i < count; i++)
            if ((rc = ojh_mm_q8k_launch(dev, xq->ptr, xs->ptr, ws[i], ojh_format(ws[i]->type), at(ys[i], y_offs ? y_offs[i] : 0),
                                        nullptr, 1, 1)))
                return rc;
        return OJH_OK;
    }
    std::vector<void *> p = {at(x, x_off)};
    uint32_t ends[4], run = 0;
    for (int i = 0; i < 4; i++) {
        int j = i < count ? i : count - 1;
        p.push_back(at(ws[j]->raw, ws[j]->off));
        if (i < count) run += ws[i]->n;
        ends[i] = run;
    }
    for (int i = 0; i < 4; i++) {
        int j = i < count ? i : count - 1;
        p.push_back(at(ys[j], y_offs ? y_offs[j] : 0));
    }
    // Every workgroup repeats the quantization (as many vector instructions as the dots of some twenty rows), so the
    // launch takes few, large workgroups — `fq_blocks_per_cu` per CU, `fq_threads` threads each — and deals the rows
    // evenly between them.
    const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
    int r = dev->fq_rows ? dev->fq_rows : 2;
    uint32_t want = cus * dev->fq_multi_blocks;
    uint32_t nrb = (run + want - 1) / want;
    nrb = (nrb + (uint32_t)r - 1) / (uint32_t)r * (uint32_t)r;
    uint32_t grid[3] = {(run + nrb - 1) / nrb, 1, 1}, block[3] = {dev->fq_threads, 1, 1};
    return ojh_launch(dev, r == 2 ? "gemv_fq8k_q4k_x4_r2" : "gemv_fq8k_q4k_x4_r1", p,
                      {K, ends[0], ends[1], ends[2], ends[3], nrb, (uint32_t)(accum != 0)}, grid, block);
}

extern "C" int ojh_mm(ojh_device *dev, const ojh_buf *x, size_t x_off, int x_dtype, const ojh_lin *w, ojh_buf *y,
                      size_t y_off, const ojh_buf *bias, uint32_t m, int accum, int act_mode) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_mm: NULL device");
    const ojh_block_format *f;
    int rc = ojh_mm_checks("ojh_mm", w, y, y_off, bias, m, accum, &f);
    if (rc) return rc;
    if (x_dtype != OJH_X_F32 && x_dtype != OJH_X_BF16)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm: activations must be f32 or bf16");
    const uint32_t K = w->k, N = w->n;
    size_t esz = x_dtype == OJH_X_BF16 ? 2 : 4;
    if ((rc = span_ok("ojh_mm: x", x, x_off, (size_t)m * K * esz, 16))) return rc;

    void *wp = at(w->raw, w->off), *yp = at(y, y_off);
    uint32_t grid[3] = {1, 1, 1}, block[3] = {256, 1, 1};

    // Q8_0 rows on the reference GPU decode path's arithmetic: activations quantized per 32 (quantize_q8_1), integer
    // dots against the blocks as the file stores them (crates/ojas-cuda/src/kernels/gemv_q8.rs:152-215), token by token.
    if (act_mode == OJH_ACT_Q8_1) {
        if (w->type != OJH_Q8_0) return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm: OJH_ACT_Q8_1 serves Q8_0 rows, not %s", f->tag);
        if (x_dtype != OJH_X_F32) return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm: OJH_ACT_Q8_1 takes f32 activations");
        if ((rc = ensure(dev, "q80_dp4a"))) return rc;
        const size_t nblk = K / 32;
        ojh_buf *q8, *d8, *d8s;
        if ((rc = ojh_scratch_get(dev, "q81_q", (size_t)m * K, &q8))) return rc;
        if ((rc = ojh_scratch_get(dev, "q81_d", (size_t)m * nblk * 4, &d8))) return rc;
        if ((rc = ojh_scratch_get(dev, "q81_s", (size_t)m * nblk * 4, &d8s))) return rc;
        const char *name = accum ? "gemv_q80_dp4a_accum" : bias ? "gemv_q80_dp4a_bias" : "gemv_q80_dp4a";
        if (accum && bias) return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm: OJH_ACT_Q8_1 adds a bias or accumulates, not both");
        uint32_t qg[3] = {(K + 255) / 256, 1, 1}, gg[3] = {(N + 7) / 8, 1, 1};
        for (uint32_t t = 0; t < m; t++) {
            void *tq = (char *)q8->ptr + (size_t)t * K, *td = (char *)d8->ptr + (size_t)t * nblk * 4;
            if ((rc = ojh_launch(dev, "quantize_q8_1", {(char *)at(x, x_off) + (size_t)t * K * 4, tq, td, (char *)d8s->ptr + (size_t)t * nblk * 4},
                                 {K}, qg, block)))
                return rc;
            std::vector<void *> p = {wp, tq, td, (char *)yp + (size_t)t * N * 4};
            if (bias && !accum) p.push_back(bias->ptr);
            if ((rc = ojh_launch(dev, name, p, {K, N}, gg, block))) return rc;
        }
        return OJH_OK;
    }

    // Q5_K: the CPU path's arithmetic (dot_q5k over int8 activations) unless floating-point activations are
    // asked for, which run on the f32-activation matvecs; from the tile crossover both that request and
    // OJH_ACT_AUTO take the f16 tile (dequant_to_f16 bits), as Q6_K and Q8_0 do.
    // Where OJH_ACT_AUTO hands over from the int8 kernels to the f16 tile: 32 tokens (OJAS_HIP_GEMM_MIN_M); for Q6_K and
    // Q5_K rows later — their int8 tile is ahead of their f16 tile up to 128 / 64 tokens (measured, 14336 x 4096 at 64
    // tokens: Q6_K 34.5 against 45.9 us, Q5_K 31.9 against 38.7; a 151936-row head at 32 tokens 164 against 341).
    uint32_t tile_min = dev->gemm_min_m;
    if (act_mode == OJH_ACT_AUTO && dev->kq_gs_min_m && K % 256 == 0 && (w->type == OJH_Q6_K || w->type == OJH_Q5_K)) {
        const uint32_t later = w->type == OJH_Q6_K ? 129u : 65u;
        if (tile_min < later) tile_min = later;
    }
    // Q8_0 rows have no few-token kernel on the matrix cores: their f32-activation matvec walks the rows once per token
    // (14336 x 4096 at 8 tokens 84 us, a 128256-row head 810), and the 128-token f16 tile — the contract the reference's
    // own GPU path switches to from 8 rows (crates/ojas-models/src/decoder/dispatch.rs:70-75) — takes 38 and 251: under
    // OJH_ACT_AUTO from 4 tokens on large matrices, 6 on small ones (4096 x 4096: 12.3 against 17.0 at 4, 21.4 at 8).
    if (act_mode == OJH_ACT_AUTO && w->type == OJH_Q8_0 && dev->q80_tile_min_m) {
        const uint32_t early = dev->q80_tile_min_m != 1 ? dev->q80_tile_min_m : (uint64_t)N * K >= (32ull << 20) ? 4u : 6u;
        if (tile_min > early) tile_min = early;
    }
    const bool q5_tile = w->type == OJH_Q5_K && act_mode != OJH_ACT_Q8K && m >= tile_min && K % 64 == 0 &&
                         (uint64_t)m * K < 0x7FFFFFFFull && (uint64_t)m * N < 0x7FFFFFFFull;
    const bool q5_float = w->type == OJH_Q5_K && !q5_tile && (act_mode == OJH_ACT_FLOAT || act_mode == OJH_ACT_FLOAT_EXACT);
    if (w->type == OJH_Q5_K && !q5_float && !q5_tile) act_mode = OJH_ACT_Q8K;

    // IQ4_NL / IQ4_XS (dot_iq4nl / dot_iq4xs), Q4_0 / Q4_1 / Q5_0 / Q5_1 and Q2_K / Q3_K: f32 activations against the raw
    // rows at every token count; no int8-activation form and no MFMA tile read them.
    // The grid-codebook formats likewise have no MFMA tile; IQ2_XXS and IQ3_XXS take int8 activations unless f32
    // ones are asked for (dot_iq2xxs_q8k / dot_iq3xxs_q8k under matvec_kq, dot_iq2xxs / dot_iq3xxs under dot_iq).
    const bool grid_fmt = ojh_grid_type(w->type);
    const bool iq4 = ojh_float_only(w->type) || q5_float;   // (the IQ4 types, the legacy 32-weight blocks, Q2_K, Q3_K, ...)
    if (iq4 && act_mode == OJH_ACT_Q8K)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm: %s rows take f32 activations only (OJH_ACT_FLOAT or OJH_ACT_AUTO)", f->tag);

    // Above the crossover the MFMA tile wins over streaming the weights once per few tokens
    // (the reference switches at 8 rows, crates/ojas-models/src/decoder/dispatch.rs:70-75).
    const int act_asked = act_mode;
    if (grid_fmt && !iq4 && act_mode == OJH_ACT_AUTO) act_mode = OJH_ACT_Q8K;
    if (grid_fmt && (rc = ensure(dev, "iq_grid"))) return rc;
    // Formats without a tile of their own (the IQ4 types, the legacy 32-weight blocks, Q2_K / Q3_K, MXFP4, the grid
    // codebooks) against a batch: their matvec walks the rows once per token (14336 x 4096: 8 us a token, 1 ms at 128
    // tokens).  From `deq_min_m` tokens the rows are decoded once into library scratch (`dequant_<fmt>_f16`:
    // dequant_to_f16's bits) and the batch runs on the f16 tile — what the reference does at load time for every
    // tensor it cannot keep in place (crates/ojas-cuda/src/qwen35.rs:174-201), without holding the f16 copy.
    // (from where the decode pass plus the tile beat the matvec that walks the rows once per four tokens: measured with
    // the decoders at 22 - 31 us for 14336 x 4096, pass + tile 50 - 56 us flat against 37 - 41 / 66 / 98 us at 4 / 8 / 12
    // tokens; on 4096 x 4096 28 against 13 / 22 / 31 / 39 at 4 / 8 / 12 / 16)
    const uint32_t deq_min = dev->deq_min_m != 1 ? dev->deq_min_m : (uint64_t)N * K >= (32ull << 20) ? 5u : 9u;
    // Q6_K rows against a long prefill batch likewise: the tile that dequantizes them on the way into LDS spends a fifth
    // of its time on that (14336 x 4096 at 2048 tokens 399 us against 288 for plain f16 rows), and the decode pass costs
    // 29 us — the same weights, dequant_to_f16's bits, either way (OJAS_HIP_DEQ_BIG_M: tokens from which, 0 = never).
    // (Q5_K and Q8_0 rows, whose loaders are lighter, from twice as many tokens: 14336 x 4096 at 2048 tokens 368 / 352 us
    // against 327)
    const uint32_t big_from = w->type == OJH_Q6_K ? dev->deq_big_m : w->type == OJH_Q5_K || w->type == OJH_Q8_0 ? 2 * dev->deq_big_m : 0u;
    const bool deq_big = big_from && m >= big_from && m >= tile_min && act_mode != OJH_ACT_Q8K && (uint64_t)N * K >= (32ull << 20);
    // IQ4_NL / IQ4_XS rows have loaders in the tile: short of the long batches they skip the decode pass (14336 x 4096:
    // 53 - 62 -> 32 - 42 us up to 128 tokens, 114 -> 93 at 512; 4096 x 4096 at 16 tokens 29 -> 14; from 1024 tokens
    // the pass pays for itself as it does for Q6_K) and take the tile from 5 tokens on every shape (the matvec that
    // walks the rows once per four tokens: 13 / 22 us at 4 / 8 tokens on 4096 x 4096)
    // (the legacy 32-weight blocks, MXFP4, Q2_K and Q3_K likewise)
    const bool own_loader = w->type == OJH_IQ4_NL || (w->type == OJH_IQ4_XS && K % 256 == 0) || w->type == OJH_Q4_0 ||
                            w->type == OJH_Q4_1 || w->type == OJH_Q5_0 || w->type == OJH_Q5_1 || w->type == OJH_MXFP4 ||
                            ((w->type == OJH_Q2_K || w->type == OJH_Q3_K) && K % 256 == 0);
    const bool iq4_own = dev->iq4_tile && own_loader &&
                         act_asked != OJH_ACT_Q8K && m >= dev->iq4_tile && (!dev->deq_big_m || m < dev->deq_big_m) &&
                         (w->type != OJH_Q3_K || m <= dev->iq4_tile_cap) &&   // (Q3_K: eight loads at 2-byte alignment per thread and step, 55 against 68 us at 128 tokens, 86 against 82 at 256)
                         K % 64 == 0;
    const bool deq_tile = ((iq4 || grid_fmt) && !iq4_own && !q5_float && act_asked != OJH_ACT_Q8K && deq_min && m >= deq_min || deq_big) &&
                          !dev->no_scratch && K % 64 == 0 && (uint64_t)N * K / f->weights <= 0x7FFFFFFFu / 64;
    void *tile_w = wp;
    if (deq_tile) {
        ojh_buf *wdeq;
        if ((rc = ojh_scratch_get(dev, "wdeq", (size_t)N * K * 2, &wdeq))) return rc;
        if ((rc = ensure(dev, grid_fmt ? "iq_grid" : "dequant"))) return rc;
        const std::string dq = std::string("dequant_") + f->tag + "_f16";
        const uint32_t nb = (uint32_t)((uint64_t)N * K / f->weights);
        uint32_t dg[3], db[3];
        if ((rc = ojh_launch_shape(dev, dq.c_str(), 0, nb, 0, dg, db))) return rc;
        if ((rc = ojh_launch(dev, dq.c_str(), {wp, wdeq->ptr}, {nb}, dg, db))) return rc;
        tile_w = wdeq->ptr;
    }
    if ((deq_tile || iq4_own || (m >= tile_min && act_mode != OJH_ACT_Q8K && !iq4 && !grid_fmt)) && K % 64 == 0 &&
        (uint64_t)m * K < 0x7FFFFFFFull && (uint64_t)m * N < 0x7FFFFFFFull) {
        // Q4_K takes the 256-wide tile with the reference GPU kernel's arithmetic (f16 qa*q + qb)
        // unless the tile that reproduces dequant_to_f16 bit for bit is asked for.
        const bool xl = w->type == OJH_Q4_K && !dev->gemm_exact && act_mode != OJH_ACT_FLOAT_EXACT &&
                        (uint64_t)w->row_bytes * N <= 0xFFFFFFFFull;  // 32-bit row offsets in that tile
        if ((rc = ensure(dev, "glue")) || (rc = ensure(dev, xl ? "gemm_xl" : "gemm"))) return rc;
        ojh_buf *xh;
        if ((rc = ojh_scratch_get(dev, "xh", (size_t)m * K * 2, &xh))) return rc;
        const uint32_t n_el = m * K, conv_blocks = (n_el / 8 + 255) / 256 + 1;
        std::string base = std::string("gemm_mm_") + (deq_tile ? "f16" : w->type == OJH_Q8_0 ? "q8_0" : f->tag);
        // (the tile that shares the dequantized weights through LDS is 256 tokens tall; its 128-token form up to 128 tokens
        // and wherever the taller one would give at most half of the CUs a tile — 14336 x 4096 at 256 tokens: Q8_0 78 ->
        // 55 us, Q6_K 100 -> 77; plain f16 rows take it at every size, 322 -> 288 us at 2048 tokens)
        const uint64_t t256 = (uint64_t)((N + 127) / 128) * ((m + 255) / 256);
        if (!xl && dev->gemm_m128 && (m <= (uint32_t)dev->gemm_m128 || 2 * t256 <= (uint32_t)dev->prop.multiProcessorCount || deq_tile))
            base += "_m128";
        if (xl) {
            // 256-token tiles when they give every CU a tile, or half of them with a K long enough
            // to split in two without the slices' fixed costs showing (measured on MI355X);
            // 128-token tiles, which dequantize every weight for half as many MFMAs, otherwise — in the form that
            // dequantizes straight into the B registers (5-17 % ahead of the form that shares the f16 tile through LDS).
            uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
            uint32_t t256 = ((N + 255) / 256) * ((m + 255) / 256);
            bool tall = m > 128 && (t256 >= cus || (2 * t256 >= cus && K >= 8192));
            base = tall ? "gemm_mm_q4kl" : "gemm_mm_q4kl_bd";
            // 128-token tiles of 256 rows too few to fill the chip: 64-row tiles whose four waves split K between them
            // and meet in LDS — four times the tiles before any K slice has to meet another through atomics
            // (measured: gate/up at 128 tokens 26 against 42 us, down at 512 tokens 74 against 88, 4096 x 4096 at 512
            // tokens 33 against 51 with the conversion)
            // — wherever the 256-row tiles would have to split K in two or more (from four slices when K is long: there
            // the longer loop pays more for the waves' separate activation copies than two slices' atomics cost)
            const uint32_t t_bd = ((N + 255) / 256) * ((m + 127) / 128), z_bd = t_bd ? cus / t_bd : 0;
            if (!tall && K >= 1024 && (dev->gemm_bdk == 2 || (dev->gemm_bdk == 1 && z_bd >= 2 && (K <= 8192 || z_bd >= 4))))
                base = "gemm_mm_q4kl_bdk";
        }
        // A few tokens on the formats whose 32 weights per thread come out of one or two wide loads: 16 (or 64) rows per
        // workgroup with the weights decoded straight into the matrix operand, no LDS staging, no barrier per K step
        // (`gemm_few_*`; 14336 x 4096 at 8 / 16 / 32 tokens, kernel alone: IQ4_XS 14 / 15 / 23 us against 30 of the tile,
        // Q8_0 26 / 28 / 32 against 36; 4096 x 4096 IQ4_XS 7 / 9 / 11 against 12 .. 14).  Four row groups per workgroup where
        // that still gives most CUs a workgroup: the tokens' bytes, re-read by every workgroup, are most of its traffic.
        // (with 16 rows per workgroup a long K costs more: up to 16 tokens there; Q8_0, twice the bytes per weight, only
        // where the tile is no better — 4096 x 14336 at 32 tokens: IQ4_XS 34 against 31 us, Q8_0 48 against 36)
        const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
        const bool r4 = (uint64_t)(N + 63) / 64 * 4 >= 3ull * cus;
        const uint32_t few_cap = r4 ? dev->gemm_few : K > 4096 ? (w->type == OJH_Q8_0 ? 0u : 16u) : w->type == OJH_Q8_0 ? 16u : dev->gemm_few;
        if (dev->gemm_few && !xl && !deq_tile && (own_loader || w->type == OJH_Q8_0) && m <= few_cap && m <= 64 && K % 128 == 0) {
            const std::string few = std::string("gemm_few_") + (w->type == OJH_Q8_0 ? "q8_0" : f->tag) + (r4 ? "_r4" : "") +
                                    (m <= 16 ? "_t1" : m <= 32 ? "_t2" : "_t4");
            uint32_t fg[3], fb[3], eg[3] = {conv_blocks, 1, 1};
            if ((rc = ojh_launch_shape(dev, few.c_str(), K, N, m, fg, fb))) return rc;
            if ((rc = ojh_launch(dev, x_dtype == OJH_X_BF16 ? "copy_bf16_half" : "copy_f32_half", {at(x, x_off), xh->ptr},
                                 {n_el}, eg, block)))
                return rc;
            return ojh_launch(dev, few.c_str(), {xh->ptr, wp, yp}, {K, N, (uint32_t)(accum != 0), m}, fg, fb);
        }
        uint32_t sg[3], sb[3];
        if ((rc = ojh_launch_shape(dev, (base + "_sk").c_str(), K, N, m, sg, sb))) return rc;
        // (a forced split counts before the tile is chosen, so that what follows sees the split that will run)
        if (dev->gemm_split_override > 0) sg[2] = (uint32_t)dev->gemm_split_override;
        if (dev->gemm_sr && base == "gemm_mm_q4kl_bdk" && sg[2] > 1) {   // reproducible bits asked for: its K slices meet in atomics
            base = "gemm_mm_q4kl_bd";
            if ((rc = ojh_launch_shape(dev, (base + "_sk").c_str(), K, N, m, sg, sb))) return rc;
            if (dev->gemm_split_override > 0) sg[2] = (uint32_t)dev->gemm_split_override;
        }
        // ... and tiles without a slice-ordered form (the LDS-shared Q4_K tile, Q6_K, Q8_0) keep K whole under that request:
        // their slices could only meet in f32 atomics, in arrival order
        if (dev->gemm_sr && sg[2] > 1 && !(xl && (base == "gemm_mm_q4kl_bd" || (base == "gemm_mm_q4kl" &&
                (uint64_t)sg[0] * sg[1] * sg[2] >= (uint32_t)dev->prop.multiProcessorCount))))
            sg[2] = 1;
        // 256-token tiles that fill the chip: the form that dequantizes into the B registers (same grid).  Its step
        // time does not grow with the number of busy CUs as the LDS-shared tile's does (measured: 2.2 us per K step
        // at 224 and at 448 workgroups against 2.0 and 2.4).
        if (xl && base == "gemm_mm_q4kl" && (uint64_t)sg[0] * sg[1] * sg[2] >= (uint32_t)dev->prop.multiProcessorCount)
            base = "gemm_mm_q4kl_bd256";
        // On request (OJAS_HIP_GEMM_SR=1) the K slices of the tiles that dequantize into the B registers meet in
        // scratch, the last slice of a tile to finish adding them in slice order: bits that do not depend on arrival, no
        // zero fill.  Measured slower than the atomics (one workgroup per tile reads every slice back from behind the
        // L2: gate/up at 128 tokens 60 against 45 us, down 142 against 46), so it is not the default.
        if (sg[2] > 1 && xl && (base == "gemm_mm_q4kl_bd" || base == "gemm_mm_q4kl_bd256") && dev->gemm_sr && !dev->no_scratch) {
            uint32_t eg[3] = {conv_blocks, 1, 1};
            if ((rc = ojh_launch(dev, x_dtype == OJH_X_BF16 ? "copy_bf16_half" : "copy_f32_half", {at(x, x_off), xh->ptr},
                                 {n_el}, eg, block)))
                return rc;
            const size_t tiles = (size_t)sg[0] * sg[1], bm = base == "gemm_mm_q4kl_bd256" ? 256 : 128;
            ojh_buf *part, *cnt;
            if ((rc = ojh_scratch_get(dev, "gemm_part", tiles * ojh_gemm_sr_slices(K, sg[2]) * bm * 256 * 4, &part))) return rc;
            if ((rc = ojh_scratch_get_zeroed(dev, "gemm_cnt", tiles * 4, &cnt))) return rc;
            return ojh_launch(dev, (base + "_sr").c_str(), {xh->ptr, wp, yp, part->ptr, cnt->ptr},
                              {K, N, m, sg[2], (uint32_t)(accum != 0)}, sg, sb);
        }
        // activations to f16 — and, ahead of K slices that add into y, the zero fill of y in the same launch
        if (sg[2] > 1 && !accum) {
            uint32_t n_y = m * N, cg[3] = {conv_blocks + (n_y / 4 + 255) / 256 + 1, 1, 1};
            if ((rc = ojh_launch(dev, x_dtype == OJH_X_BF16 ? "copy_bf16_half_zero" : "copy_f32_half_zero",
                                 {at(x, x_off), xh->ptr, yp}, {n_el, n_y, conv_blocks}, cg, block)))
                return rc;
        } else {
            uint32_t eg[3] = {conv_blocks, 1, 1};
            if ((rc = ojh_launch(dev, x_dtype == OJH_X_BF16 ? "copy_bf16_half" : "copy_f32_half", {at(x, x_off), xh->ptr},
                                 {n_el}, eg, block)))
                return rc;
        }
        if (sg[2] > 1) return ojh_launch(dev, (base + "_sk").c_str(), {xh->ptr, tile_w, yp}, {K, N, m, sg[2]}, sg, sb);
        sg[2] = 1;
        return ojh_launch(dev, base.c_str(), {xh->ptr, tile_w, yp}, {K, N, (uint32_t)(accum != 0), m}, sg, sb);
    }

    bool q8k = !ojh_float_rows(w->type) && act_mode != OJH_ACT_FLOAT && act_mode != OJH_ACT_FLOAT_EXACT;
    if (grid_fmt && act_mode == OJH_ACT_FLOAT_EXACT)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm: %s rows have no MFMA tile; OJH_ACT_FLOAT runs their f32-activation matvec", f->tag);
    // Opt-in: one token, f32 in, plain store through the launch that quantizes x itself
    // (bit-identical results).  Measured slower than quantize + matvec at every decode shape on
    // MI355X — each block repeats the quantization and reads x through LDS — so it is off by default.
    if (q8k && m == 1 && !accum && !bias && x_dtype == OJH_X_F32 && w->type == OJH_Q4_K && K <= 16384 &&
        dev->fused_quant) {
        if ((rc = ensure(dev, "gemv_q8k"))) return rc;
        int r = pick_rows(dev, N);
        if (r > 2) r = 2;
        const char *name = (r == 2 && N >= 32768u) ? "gemv_fq8k_q4k_wide" : r == 2 ? "gemv_fq8k_q4k_r2" : "gemv_fq8k_q4k_r1";
        // rows per block: every block re-quantizes x, so give it enough rows that this stays a
        // small share, but keep several blocks per CU
        uint32_t unit = 4u * (uint32_t)r, cus = (uint32_t)dev->prop.multiProcessorCount;
        uint32_t nrb = (N + cus * dev->fq_blocks_per_cu - 1) / (cus * dev->fq_blocks_per_cu);
        nrb = ((nrb + unit - 1) / unit) * unit;
        if (nrb < unit) nrb = unit;
        grid[0] = (N + nrb - 1) / nrb;
        return ojh_launch(dev, name, {at(x, x_off), wp, yp}, {K, N, nrb}, grid, block);
    }
    if (q8k) {
        if ((rc = ensure(dev, "gemv_q8k"))) return rc;
        size_t nsb = K / 256;
        ojh_buf *xq, *xs;
        if ((rc = ojh_scratch_get(dev, "xq", (size_t)m * nsb * 256, &xq))) return rc;
        if ((rc = ojh_scratch_get(dev, "xs", (size_t)m * nsb * 4, &xs))) return rc;
        // ahead of the 128-token int8 tile the quantizer writes that tile's side arrays too (one launch less)
        if (ojh_q4k_xt_taken(dev, w, m, wp) && K % 256 == 0 && (uintptr_t)at(x, x_off) % (x_dtype == OJH_X_BF16 ? 8 : 16) == 0) {
            if ((rc = ensure(dev, "gemm_q8k"))) return rc;
            const uint32_t mp = (m + 127) / 128 * 128;
            ojh_buf *xst, *sums;
            if ((rc = ojh_scratch_get(dev, "xt_xst", nsb * mp * 4, &xst))) return rc;
            if ((rc = ojh_scratch_get(dev, "xt_sums", nsb * mp * 32, &sums))) return rc;
            uint32_t qg[3] = {K / 256 * (mp / 4), 1, 1};
            if ((rc = ojh_launch(dev, x_dtype == OJH_X_BF16 ? "quantize_q8k_bf16_sides" : "quantize_q8k_sides",
                                 {at(x, x_off), xq->ptr, xs->ptr, xst->ptr, sums->ptr}, {K, m, mp}, qg, block)))
                return rc;
            return ojh_mm_q8k_launch(dev, xq->ptr, xs->ptr, w, f, yp, bias, m, accum, true);
        }
        if ((rc = ojh_quant_q8k_launch(dev, at(x, x_off), x_dtype, m, K, xq->ptr, xs->ptr))) return rc;
        return ojh_mm_q8k_launch(dev, xq->ptr, xs->ptr, w, f, yp, bias, m, accum);
    }

    // floating-point activations: the matvec kernels read f32
    void *xp = at(x, x_off);
    if (x_dtype == OJH_X_BF16) {
        if ((rc = ensure(dev, "glue"))) return rc;
        ojh_buf *xf;
        if ((uint64_t)m * K > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_mm: %u x %u bf16 activations exceed 2^32 elements", m, K);
        if ((rc = ojh_scratch_get(dev, "xf", (size_t)m * K * 4, &xf))) return rc;
        uint32_t n_el = m * K, eg[3] = {(n_el / 8 + 255) / 256 + 1, 1, 1};
        if ((rc = ojh_launch(dev, "copy_bf16_f32", {xp, xf->ptr}, {n_el}, eg, block))) return rc;
        xp = xf->ptr;
    }
    if (!grid_fmt && (rc = ensure(dev, "gemv"))) return rc;
    std::string base = std::string("gemv_nat_") + f->tag;
    // Q8_0 rows from a few thousand up: activations in registers, rows copied into LDS by the
    // memory system (needs 16-byte aligned rows and a K that chunks)
    if (m == 1 && w->type == OJH_Q8_0 && dev->q80_lds && N >= dev->q80_lds_min_n && ojh_q80_lds_kc(K) &&
        (uintptr_t)wp % 16 == 0 && (uintptr_t)xp % 16 == 0) {
        uint32_t sg[3], sb[3];
        if ((rc = ojh_launch_shape(dev, "gemv_nat_q80_lds", K, N, 1, sg, sb))) return rc;
        std::vector<void *> p = {xp, wp, yp};
        if (bias) p.push_back(bias->ptr);
        return ojh_launch(dev, accum ? "gemv_nat_q80_lds_accum" : bias ? "gemv_nat_q80_lds_bias" : "gemv_nat_q80_lds", p,
                          {K, N, ojh_q80_lds_kc(K)}, sg, sb);
    }
    // an output head (K-quant or IQ4 rows): rows grid-stride, the wave's f32 activations in registers
    if (m == 1 && w->type != OJH_Q8_0 && dev->px && !accum && !bias && N >= 32768u && K <= 4096u) {
        uint32_t sg[3], sb[3];
        if ((rc = ojh_launch_shape(dev, (base + "_px").c_str(), K, N, 1, sg, sb))) return rc;
        return ojh_launch(dev, (base + "_px").c_str(), {xp, wp, yp}, {K, N}, sg, sb);
    }
    // the sub-block-per-lane form of IQ2_XXS / IQ2_S / IQ3_XXS / IQ3_S also wins on mid-sized projections, with fewer
    // workgroups (a wave needs a few row pairs to pay for the 64 activations it keeps): 14336 x 4096 IQ3_S 17.1 -> 15.9 us,
    // IQ2_XXS 17.4 -> 13.2 us at 512 workgroups
    if (m == 1 && dev->px && !accum && !bias && N >= 8192u && K <= 4096u &&
        (w->type == OJH_IQ2_XXS || w->type == OJH_IQ2_S || w->type == OJH_IQ3_XXS || w->type == OJH_IQ3_S)) {
        uint32_t sg[3] = {std::min(std::max(N / 28u / 64u * 64u, 256u), 2048u), 1, 1};
        return ojh_launch(dev, (base + "_px").c_str(), {xp, wp, yp}, {K, N}, sg, block);
    }
    if (m == 1) {
        // rows per wave for the f32-activation kernels (measured on Q4_K and Q6_K, K = 4096 and 14336): the
        // activation fragment is 4 bytes per weight, so sharing it pays earlier than for int8 activations —
        // two rows everywhere, four from 8192 Q4_K rows; one row only when told to
        int r = (accum || bias) ? 4 : dev->gemv_rows_override ? pick_rows(dev, N) : (w->type == OJH_Q4_K && N >= 8192u) ? 4 : 2;
        std::string name = base + (accum ? "_accum" : bias ? "_bias" : r == 4 ? "" : r == 2 ? "_r2" : "_r1");
        grid[0] = (N + 4 * r - 1) / (4 * r);
        std::vector<void *> p = {xp, wp, yp};
        if (bias) p.push_back(bias->ptr);
        return ojh_launch(dev, name.c_str(), p, {K, N}, grid, block);
    }
    grid[0] = (N + 3) / 4;
    return ojh_launch(dev, (base + "_m").c_str(), {xp, wp, yp}, {K, N, m, (uint32_t)(accum != 0)}, grid, block);
}

// ---- row-int8 path -------------------------------------------------------------------------------
extern "C" int ojh_q8rows_from_f16(ojh_device *dev, const ojh_buf *w16, size_t w_off, uint32_t n, uint32_t k,
                                   ojh_buf *q, ojh_buf *scale) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_q8rows_from_f16: NULL device");
    if (!n || !k) return ojh_fail(OJH_ERR_ARG, "ojh_q8rows_from_f16: n=%u k=%u", n, k);
    int rc;
    if ((rc = span_ok("q8rows: w16", w16, w_off, (size_t)n * k * 2, 2))) return rc;
    if ((rc = span_ok("q8rows: q", q, 0, (size_t)n * k, 16))) return rc;
    if ((rc = span_ok("q8rows: scale", scale, 0, (size_t)n * 4, 4))) return rc;
    if ((rc = ensure(dev, "rowq8"))) return rc;
    uint32_t grid[3] = {n, 1, 1}, block[3] = {256, 1, 1};
    return ojh_launch(dev, "rows_q8_from_f16", {at(w16, w_off), q->ptr, scale->ptr}, {k, n}, grid, block);
}

extern "C" int ojh_matmul_q8(ojh_device *dev, const ojh_buf *x, size_t x_off, const ojh_buf *wq, const ojh_buf *wscale,
                             const ojh_buf *bias, ojh_buf *y, size_t y_off, uint32_t n, uint32_t k, uint32_t m) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_matmul_q8: NULL device");
    if (!n || !k || !m || m > 65535) return ojh_fail(OJH_ERR_ARG, "ojh_matmul_q8: n=%u k=%u m=%u out of range", n, k, m);
    if (k % 16) return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_matmul_q8: K=%u must be a multiple of 16", k);
    int rc;
    if ((rc = span_ok("matmul_q8: x", x, x_off, (size_t)m * k * 4, 4))) return rc;
    if ((rc = span_ok("matmul_q8: wq", wq, 0, (size_t)n * k, 16))) return rc;
    if ((rc = span_ok("matmul_q8: wscale", wscale, 0, (size_t)n * 4, 4))) return rc;
    if (bias && (rc = span_ok("matmul_q8: bias", bias, 0, (size_t)n * 4, 4))) return rc;
    if ((rc = span_ok("matmul_q8: y", y, y_off, (size_t)m * n * 4, 4))) return rc;
    if ((rc = ensure(dev, "rowq8"))) return rc;
    ojh_buf *xq, *sx;
    if ((rc = ojh_scratch_get(dev, "q8_xq", (size_t)m * k, &xq))) return rc;
    if ((rc = ojh_scratch_get(dev, "q8_sx", (size_t)m * 4, &sx))) return rc;
    uint32_t block[3] = {256, 1, 1}, gq[3], bq[3], gm[3] = {(n + 3) / 4, 1, 1};
    if ((rc = ojh_launch_shape(dev, "quant_rows_i8", k, 0, m, gq, bq))) return rc;
    if ((rc = ojh_launch(dev, "quant_rows_i8", {at(x, x_off), xq->ptr, sx->ptr}, {k, m}, gq, bq))) return rc;
    // a batch: the integer sums on the int8 matrix instruction (the same bits; the per-row kernel reads a row once per
    // 8 tokens, so its time grows with the tokens)
    const uint32_t mt_min = dev->q8row_mt_min_m != 1 ? dev->q8row_mt_min_m : 9u;
    if (mt_min && m >= mt_min) {
        uint32_t gt[3] = {(n + 127) / 128, (m + 63) / 64, 1};
        void *bp = bias ? bias->ptr : nullptr;
        // 128 tokens a tile where that still leaves a tile and a half per CU
        const bool many = (uint64_t)gt[0] * ((m + 127) / 128) * 2 >= (uint64_t)3 * dev->prop.multiProcessorCount;
        const uint32_t t128 = dev->q8row_t128_min_m != 1 ? dev->q8row_t128_min_m : many ? 129u : 0u;
        if (t128 && m >= t128) {
            gt[1] = (m + 127) / 128;
            return ojh_launch(dev, "matmul_q8row_mt128", {xq->ptr, sx->ptr, wq->ptr, wscale->ptr, at(y, y_off), bp}, {k, n, m}, gt, block);
        }
        const uint32_t z = dev->no_scratch ? 1 : ojh_matmul_q8row_slices(dev, k, n, m);
        if (z > 1) {
            const size_t tiles = (size_t)gt[0] * gt[1];
            ojh_buf *part, *cnt;
            if ((rc = ojh_scratch_get(dev, "q8r_part", tiles * z * 32768, &part))) return rc;
            if ((rc = ojh_scratch_get_zeroed(dev, "q8r_cnt", tiles * 4, &cnt))) return rc;
            gt[2] = z;
            return ojh_launch(dev, "matmul_q8row_mt_sr", {xq->ptr, sx->ptr, wq->ptr, wscale->ptr, at(y, y_off), bp, part->ptr, cnt->ptr},
                              {k, n, m, z}, gt, block);
        }
        return ojh_launch(dev, "matmul_q8row_mt", {xq->ptr, sx->ptr, wq->ptr, wscale->ptr, at(y, y_off), bp}, {k, n, m}, gt, block);
    }
    if (dev->q8row_dec && m <= 8 && (size_t)m * k <= 131072) {
        const char *name = (size_t)m * k <= 65536 ? "matmul_q8row_dec" : "matmul_q8row_dec_l";
        uint32_t gd[3], bd[3];
        if ((rc = ojh_launch_shape(dev, name, k, n, m, gd, bd))) return rc;
        return ojh_launch(dev, name, {xq->ptr, sx->ptr, wq->ptr, wscale->ptr, at(y, y_off), bias ? bias->ptr : nullptr}, {k, n, m}, gd, bd);
    }
    if (bias)
        return ojh_launch(dev, "matmul_q8row_bias", {xq->ptr, sx->ptr, wq->ptr, wscale->ptr, at(y, y_off), bias->ptr},
                          {k, n, m}, gm, block);
    return ojh_launch(dev, "matmul_q8row", {xq->ptr, sx->ptr, wq->ptr, wscale->ptr, at(y, y_off)}, {k, n, m}, gm, block);
}

// ---- decode-layer epilogues around the matvec ----------------------------------------------------
extern "C" int ojh_rmsnorm_quant_q8k(ojh_device *dev, const ojh_buf *x, size_t x_off, const ojh_buf *gamma, float eps,
                                     uint32_t m, uint32_t k, ojh_buf *q, ojh_buf *scales, ojh_buf *xn) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_rmsnorm_quant_q8k: NULL device");
    if (!m || !k || k > 16384 || m > 65535) return ojh_fail(OJH_ERR_ARG, "rmsnorm_quant_q8k: m=%u k=%u out of range (k <= 16384)", m, k);
    size_t nsb = (k + 255) / 256;
    int rc;
    if ((rc = span_ok("rmsnorm_quant_q8k: x", x, x_off, (size_t)m * k * 4, 4))) return rc;
    if ((rc = span_ok("rmsnorm_quant_q8k: gamma", gamma, 0, (size_t)k * 4, 4))) return rc;
    if ((rc = span_ok("rmsnorm_quant_q8k: q", q, 0, (size_t)m * nsb * 256, 16))) return rc;
    if ((rc = span_ok("rmsnorm_quant_q8k: scales", scales, 0, (size_t)m * nsb * 4, 4))) return rc;
    if (xn && (rc = span_ok("rmsnorm_quant_q8k: xn", xn, 0, (size_t)m * k * 4, 4))) return rc;
    if ((rc = ensure(dev, "gemv_q8k"))) return rc;
    uint32_t eps_bits;
    memcpy(&eps_bits, &eps, 4);
    // a few rows: sixteen waves, a segment each up to 4096 values (the launch is one dependent chain of latencies);
    // many rows: four, so that several rows share a CU
    uint32_t grid[3] = {m, 1, 1}, block[3] = {dev->rms_threads ? dev->rms_threads : (m <= 64 ? 1024u : 256u), 1, 1};
    return ojh_launch(dev, "rmsnorm_q8k", {at(x, x_off), gamma->ptr, q->ptr, scales->ptr, xn ? xn->ptr : q->ptr},
                      {k, m, eps_bits, (uint32_t)(xn != nullptr)}, grid, block);
}

extern "C" int ojh_ffn_gu_q8k(ojh_device *dev, const ojh_buf *xq, const ojh_buf *xscales, const ojh_lin *gate,
                              const ojh_lin *up, ojh_buf *out, size_t out_off, int act) {
    if (!dev || !gate || !up) return ojh_fail(OJH_ERR_ARG, "ojh_ffn_gu_q8k: NULL argument");
    auto kq = [](uint32_t t) { return t == OJH_Q4_K || t == OJH_Q5_K || t == OJH_Q6_K; };
    if (!kq(gate->type) || !kq(up->type))
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_ffn_gu_q8k: gate and up must be Q4_K, Q5_K or Q6_K (got %u, %u)", gate->type, up->type);
    if (gate->n != up->n || gate->k != up->k)
        return ojh_fail(OJH_ERR_ARG, "ojh_ffn_gu_q8k: gate is %ux%u, up is %ux%u", gate->n, gate->k, up->n, up->k);
    if (act != 0 && act != 1) return ojh_fail(OJH_ERR_ARG, "ojh_ffn_gu_q8k: act=%d (0 = SiLU, 1 = GELU)", act);
    const uint32_t N = gate->n, K = gate->k;
    size_t nsb = K / 256;
    int rc;
    if ((rc = span_ok("ffn_gu: xq", xq, 0, nsb * 256, 16))) return rc;
    if ((rc = span_ok("ffn_gu: xscales", xscales, 0, nsb * 4, 4))) return rc;
    if ((rc = span_ok("ffn_gu: out", out, out_off, (size_t)N * 4, 4))) return rc;
    if ((rc = span_ok("ffn_gu: gate", gate->raw, gate->off, gate->row_bytes * N, ojh_block_align(ojh_format(gate->type))))) return rc;
    if ((rc = span_ok("ffn_gu: up", up->raw, up->off, up->row_bytes * N, ojh_block_align(ojh_format(up->type))))) return rc;
    if ((rc = ensure(dev, "gemv_q8k"))) return rc;
    uint32_t grid[3] = {(N + 3) / 4, 1, 1}, block[3] = {256, 1, 1};
    if (gate->type != OJH_Q4_K || up->type != OJH_Q4_K)   // every row in its own format's arithmetic
        return ojh_launch(dev, "ffn_gu_q8k_kq", {xq->ptr, xscales->ptr, at(gate->raw, gate->off), at(up->raw, up->off), at(out, out_off)},
                          {K, N, (uint32_t)act, gate->type | (up->type << 8)}, grid, block);
    return ojh_launch(dev, "ffn_gu_q8k_q4k", {xq->ptr, xscales->ptr, at(gate->raw, gate->off), at(up->raw, up->off), at(out, out_off)},
                      {K, N, (uint32_t)act}, grid, block);
}

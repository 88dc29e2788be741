// MoE op seam: router and grouped expert FFN (the host side of the "moe" kernel family).
// Stands in for the reference's MoE layer drivers (decode crates/ojas-models/src/decoder/
// graph_decode.rs:441-499, prefill graph_chunk.rs:564-628; CPU crates/ojas-cpu/src/cpu_glm.rs:519-597):
// router -> group assignments by expert -> gate/up (+SiLU*mul) -> quantize -> down -> weighted sum.
#include "ojh_internal.h"
#include <cstring>
#include <string>

static int ensure(ojh_device *dev, const char *family) {
    return dev->modules.count(family) ? OJH_OK : ojh_ensure_family(dev, family);
}

static int span(const char *what, const ojh_buf *b, size_t bytes, size_t align) {
    if (!b) return ojh_fail(OJH_ERR_ARG, "%s: NULL buffer", what);
    if (bytes > b->bytes) return ojh_fail(OJH_ERR_BOUNDS, "%s needs %zu bytes, buffer has %zu", what, bytes, b->bytes);
    if ((uintptr_t)b->ptr % align) return ojh_fail(OJH_ERR_ARG, "%s must be %zu-byte aligned", what, align);
    return OJH_OK;
}

extern "C" int ojh_moe_route(ojh_device *dev, const ojh_buf *logits, uint32_t n_tokens, uint32_t n_expert,
                             uint32_t ksel, ojh_buf *idx, ojh_buf *wgt) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_moe_route: NULL device");
    if (!n_tokens || !n_expert || n_expert > 1024 || !ksel || ksel > n_expert || ksel > 64)
        return ojh_fail(OJH_ERR_ARG, "moe_route: tokens=%u experts=%u (<= 1024) ksel=%u (<= 64, <= experts)", n_tokens,
                        n_expert, ksel);
    int rc;
    if ((rc = span("moe_route: logits", logits, (size_t)n_tokens * n_expert * 4, 4))) return rc;
    if ((rc = span("moe_route: idx", idx, (size_t)n_tokens * ksel * 4, 4))) return rc;
    if ((rc = span("moe_route: wgt", wgt, (size_t)n_tokens * ksel * 4, 4))) return rc;
    if ((rc = ensure(dev, "moe"))) return rc;
    uint32_t grid[3] = {n_tokens, 1, 1}, block[3] = {64, 1, 1};
    return ojh_launch(dev, "moe_topk_m", {logits->ptr, idx->ptr, wgt->ptr}, {n_expert, ksel}, grid, block);
}

// Router + expert FFN.  A few tokens over Q4_K gate / up experts: the router runs inside the gate/up launch of the
// decode form (every workgroup routes its token itself; idx / wgt are written for the down launch and for the
// caller) — two launches per layer instead of three; otherwise ojh_moe_route, then ojh_moe_ffn.
extern "C" int ojh_moe_ffn_routed(ojh_device *dev, const ojh_buf *x, uint32_t T, uint32_t d, uint32_t n_ff, uint32_t E,
                                  uint32_t ksel, const ojh_buf *logits, ojh_buf *idx, ojh_buf *wgt, const ojh_lin *gate,
                                  const ojh_lin *up, const ojh_lin *down, ojh_buf *y, int accum, int act_mode) {
    if (!dev || !gate || !up || !down) return ojh_fail(OJH_ERR_ARG, "ojh_moe_ffn_routed: NULL argument");
    if (!T || !E || E > 1024 || !ksel || ksel > E || ksel > 64 || T > 65535u / ksel)
        return ojh_fail(OJH_ERR_ARG, "moe_ffn_routed: tokens=%u experts=%u (<= 1024) ksel=%u (<= 64, <= experts) out of range", T, E, ksel);
    const bool kq = gate->type == OJH_Q4_K && up->type == OJH_Q4_K &&
                    (down->type == OJH_Q4_K || down->type == OJH_Q5_K || down->type == OJH_Q6_K);
    const bool dec_fits = d && n_ff && d % 256 == 0 && n_ff % 256 == 0 && d <= 8192 && n_ff <= 2048 && (uint64_t)ksel * n_ff <= 32768;
    const bool fused = kq && act_mode != OJH_ACT_FLOAT && act_mode != OJH_ACT_FLOAT_EXACT && dec_fits &&
                       (dev->moe_mode == 3 || (dev->moe_mode == 0 && T <= dev->moe_dec_tokens)) && dev->moe_route_fuse;
    int rc;
    if (!fused) {
        if ((rc = ojh_moe_route(dev, logits, T, E, ksel, idx, wgt))) return rc;
        return ojh_moe_ffn(dev, x, T, d, n_ff, E, ksel, idx, wgt, gate, up, down, y, accum, act_mode);
    }
    if (gate->k != d || up->k != d || gate->n != (uint64_t)E * n_ff || up->n != gate->n || down->k != n_ff ||
        down->n != (uint64_t)E * d)
        return ojh_fail(OJH_ERR_ARG, "moe_ffn_routed: expert tensor shapes do not match E=%u d=%u n_ff=%u", E, d, n_ff);
    const uint32_t NA = T * ksel;
    if ((rc = span("moe_ffn_routed: x", x, (size_t)T * d * 4, 16))) return rc;
    if ((rc = span("moe_ffn_routed: logits", logits, (size_t)T * E * 4, 4))) return rc;
    if ((rc = span("moe_ffn_routed: idx", idx, (size_t)NA * 4, 4))) return rc;
    if ((rc = span("moe_ffn_routed: wgt", wgt, (size_t)NA * 4, 4))) return rc;
    if ((rc = span("moe_ffn_routed: y", y, (size_t)T * d * 4, 4))) return rc;
    if ((rc = ensure(dev, "moe"))) return rc;
    ojh_buf *act;
    if ((rc = ojh_scratch_get(dev, "moe_act", (size_t)NA * n_ff * 4, &act))) return rc;
    uint32_t b256[3] = {256, 1, 1}, g1[3] = {(n_ff + 7) / 8, NA, 1}, g2[3] = {(d + 7) / 8, T, 1};
    if ((rc = ojh_launch(dev, "moe_gu_q4k_decr",
                         {x->ptr, (char *)gate->raw->ptr + gate->off, (char *)up->raw->ptr + up->off, act->ptr, logits->ptr,
                          idx->ptr, wgt->ptr},
                         {d, n_ff, ksel, NA, E}, g1, b256)))
        return rc;
    const std::string down_dec = std::string("moe_down_") + ojh_format(down->type)->tag + "_dec";
    return ojh_launch(dev, down_dec.c_str(), {act->ptr, (char *)down->raw->ptr + down->off, idx->ptr, wgt->ptr, y->ptr},
                      {n_ff, d, ksel, E, (uint32_t)(accum != 0)}, g2, b256);
}

extern "C" int ojh_moe_ffn(ojh_device *dev, const ojh_buf *x, uint32_t T, uint32_t d, uint32_t n_ff, uint32_t E,
                           uint32_t ksel, const ojh_buf *idx, const ojh_buf *wgt, const ojh_lin *gate,
                           const ojh_lin *up, const ojh_lin *down, ojh_buf *y, int accum, int act_mode) {
    if (!dev || !gate || !up || !down) return ojh_fail(OJH_ERR_ARG, "ojh_moe_ffn: NULL argument");
    if (!T || !E || E > 1024 || !ksel || ksel > E || T > 65535u / ksel)
        return ojh_fail(OJH_ERR_ARG, "moe_ffn: tokens=%u experts=%u ksel=%u out of range", T, E, ksel);
    // Experts in a format whose rows meet f32 activations (Q8_0, IQ4_XS, IQ4_NL; gate and up alike, down
    // any of the three): the reference's own expert kernels moe_gu_<fmt> / moe_down_<fmt>, one launch for
    // gate/up and one for down over all tokens; the down launch accumulates onto y, so a plain store
    // starts from zeros
    // K-quant experts take the same two launches when floating-point activations are asked for (OJH_ACT_FLOAT):
    // moe_gu_q4k / moe_down_{q4k,q5k,q6k}, the reference's GPU expert kernels for those formats.
    // The grid-codebook rows of the reference's expert table (crates/ojas-core/src/quant_src.rs:180-190) join them:
    // IQ3_S, IQ2_XXS, IQ2_S gate/up and IQ2_XXS, IQ3_XXS down, on f32 activations like the reference's GPU kernels.
    auto float_gu = [](uint32_t t) {
        return t == OJH_Q8_0 || t == OJH_IQ4_XS || t == OJH_IQ4_NL || t == OJH_IQ3_S || t == OJH_IQ2_XXS || t == OJH_IQ2_S;
    };
    auto float_down = [](uint32_t t) {
        return t == OJH_Q8_0 || t == OJH_IQ4_XS || t == OJH_IQ4_NL || t == OJH_IQ2_XXS || t == OJH_IQ3_XXS;
    };
    const bool kq_float = act_mode == OJH_ACT_FLOAT && gate->type == OJH_Q4_K && up->type == OJH_Q4_K &&
                          (down->type == OJH_Q4_K || down->type == OJH_Q5_K || down->type == OJH_Q6_K);
    if (kq_float || (gate->type == up->type && float_gu(gate->type) && float_down(down->type))) {
        if (act_mode == OJH_ACT_Q8K)
            return ojh_fail(OJH_ERR_UNSUPPORTED, "moe_ffn: %s / %s experts take f32 activations, as their CPU dots do",
                            ojh_format(gate->type)->tag, ojh_format(down->type)->tag);
        int rc;
        const ojh_block_format *fg = ojh_format(gate->type), *fd = ojh_format(down->type);
        if (d % fg->weights || n_ff % fd->weights || d % 32 || n_ff % 32)
            return ojh_fail(OJH_ERR_ARG, "moe_ffn: d=%u and n_ff=%u must be whole blocks of the expert formats", d, n_ff);
        if (gate->k != d || up->k != d || down->k != n_ff || (uint64_t)gate->n != (uint64_t)E * n_ff ||
            (uint64_t)up->n != (uint64_t)E * n_ff || (uint64_t)down->n != (uint64_t)E * d)
            return ojh_fail(OJH_ERR_ARG, "moe_ffn: expert tensor shapes do not match E=%u d=%u n_ff=%u", E, d, n_ff);
        const uint32_t NA8 = T * ksel;
        if ((rc = span("moe_ffn: x", x, (size_t)T * d * 4, 16))) return rc;
        if ((rc = span("moe_ffn: idx", idx, (size_t)NA8 * 4, 4))) return rc;
        if ((rc = span("moe_ffn: wgt", wgt, (size_t)NA8 * 4, 4))) return rc;
        if ((rc = span("moe_ffn: y", y, (size_t)T * d * 4, 4))) return rc;
        // A batch of such experts under OJH_ACT_AUTO: the per-assignment kernels below read an expert's matrices once
        // per assignment, so their time grows with the tokens; from a few assignments per expert the products run
        // grouped by expert on the f16 matrix tile (f16 activations, f32 accumulate: the contract of the dense f16
        // tile): gate and up in one launch, silu * up rounded to f16, down, the router-weighted sum.  Q8_0, IQ4_NL and
        // IQ4_XS rows are read by the tile's own loaders; the other formats are decoded into f16 scratch first (2 bytes
        // per weight of the tensors concerned), which pays from more assignments per expert.
        auto tile_of = [](uint32_t t) -> const char * {
            return t == OJH_Q8_0 ? "moe_mm_q8_0" : t == OJH_IQ4_NL ? "moe_mm_iq4nl" : t == OJH_IQ4_XS ? "moe_mm_iq4xs" : nullptr;
        };
        const char *tile_gu = tile_of(gate->type), *tile_dn = tile_of(down->type);
        const uint32_t mm_from = dev->moe_mm_tile != 1 ? dev->moe_mm_tile : tile_gu && tile_dn ? 4u : 8u;
        const uint64_t w_gu = (uint64_t)E * n_ff * d, w_dn = (uint64_t)E * d * n_ff;
        if (act_mode == OJH_ACT_AUTO && !kq_float && mm_from && (uint64_t)NA8 >= (uint64_t)mm_from * E && d % 64 == 0 &&
            n_ff % 64 == 0 && (uint64_t)NA8 * (d > n_ff ? d : n_ff) <= 0xFFFFFFFFull && w_gu / fg->weights <= 0x7FFFFFFFu / 64 &&
            w_dn / fd->weights <= 0x7FFFFFFFu / 64) {
            if ((rc = ensure(dev, "moe")) || (rc = ensure(dev, "gemm")) || (rc = ensure(dev, "glue"))) return rc;
            ojh_buf *xh, *gv, *uv, *a16, *dv, *grp;
            if ((rc = ojh_scratch_get(dev, "moe_xh", (size_t)T * d * 2, &xh))) return rc;
            if ((rc = ojh_scratch_get(dev, "moe_g", (size_t)NA8 * n_ff * 4, &gv))) return rc;
            if ((rc = ojh_scratch_get(dev, "moe_u", (size_t)NA8 * n_ff * 4, &uv))) return rc;
            if ((rc = ojh_scratch_get(dev, "moe_a16", (size_t)NA8 * n_ff * 2, &a16))) return rc;
            if ((rc = ojh_scratch_get(dev, "moe_dv", (size_t)NA8 * d * 4, &dv))) return rc;
            if ((rc = ojh_scratch_get(dev, "moe_grp", ((size_t)2 * E + 1 + NA8) * 4, &grp))) return rc;
            void *wg = (char *)gate->raw->ptr + gate->off, *wu = (char *)up->raw->ptr + up->off, *wd = (char *)down->raw->ptr + down->off;
            {
                ojh_buf *dq[3];
                const ojh_lin *ls[3] = {gate, up, down};
                const char *names[3] = {"moe_wg16", "moe_wu16", "moe_wd16"};
                void **outs[3] = {&wg, &wu, &wd};
                for (int i = 0; i < 3; i++) {
                    if (i < 2 ? tile_gu != nullptr : tile_dn != nullptr) continue;
                    const ojh_block_format *fi = ojh_format(ls[i]->type);
                    const uint64_t nw = i < 2 ? w_gu : w_dn;
                    if ((rc = ojh_scratch_get(dev, names[i], (size_t)nw * 2, &dq[i]))) return rc;
                    if ((rc = ensure(dev, ojh_grid_type(ls[i]->type) ? "iq_grid" : "dequant"))) return rc;
                    const std::string k = std::string("dequant_") + fi->tag + "_f16";
                    const uint32_t nb = (uint32_t)(nw / fi->weights);
                    uint32_t dg[3], db[3];
                    if ((rc = ojh_launch_shape(dev, k.c_str(), 0, nb, 0, dg, db))) return rc;
                    if ((rc = ojh_launch(dev, k.c_str(), {*outs[i], dq[i]->ptr}, {nb}, dg, db))) return rc;
                    *outs[i] = dq[i]->ptr;
                }
                if (!tile_gu) tile_gu = "moe_mm_f16";
                if (!tile_dn) tile_dn = "moe_mm_f16";
            }
            uint32_t *counts = (uint32_t *)grp->ptr, *offsets = counts + E, *list = offsets + E + 1;
            uint32_t b256[3] = {256, 1, 1}, g1[3] = {1, 1, 1};
            if ((rc = ojh_launch(dev, "moe_group", {idx->ptr, counts, offsets, list}, {NA8, E}, g1, b256))) return rc;
            const uint32_t n_x = T * d, n_a = NA8 * n_ff;
            uint32_t gc[3] = {(n_x / 8 + 255) / 256 + 1, 1, 1};
            if ((rc = ojh_launch(dev, "copy_f32_half", {x->ptr, xh->ptr}, {n_x}, gc, b256))) return rc;
            uint32_t tiles = (T + 127) / 128;
            // experts that received a few dozen tokens: 32 assignments per pass on the few-token kernel, 64 rows per
            // workgroup (two passes in the grid, the rest by its loop)
            const bool few_gu = dev->moe_few && (uint64_t)NA8 <= (uint64_t)dev->moe_few * E && d % 128 == 0 && !strncmp(tile_gu, "moe_mm_", 7) && strcmp(tile_gu, "moe_mm_f16");
            const bool few_dn = dev->moe_few && (uint64_t)NA8 <= (uint64_t)dev->moe_few * E && n_ff % 128 == 0 && !strncmp(tile_dn, "moe_mm_", 7) && strcmp(tile_dn, "moe_mm_f16");
            const std::string few_gu_name = std::string("moe_few_") + (tile_gu + 7), few_dn_name = std::string("moe_few_") + (tile_dn + 7);
            if (few_gu) tile_gu = few_gu_name.c_str();
            if (few_dn) tile_dn = few_dn_name.c_str();
            const uint32_t passes = T < 32 ? 1u : 2u;
            uint32_t gg[3] = {few_gu ? (n_ff + 63) / 64 : (n_ff + 127) / 128, few_gu ? passes : tiles, 2 * E};
            if ((rc = ojh_launch(dev, tile_gu, {xh->ptr, wg, wu, gv->ptr, uv->ptr, offsets, list}, {d, n_ff, NA8, E, ksel}, gg, b256)))
                return rc;
            uint32_t ga[3] = {(n_a / 8 + 255) / 256 + 1, 1, 1};
            if ((rc = ojh_launch(dev, "moe_act_half", {gv->ptr, uv->ptr, a16->ptr}, {n_a}, ga, b256))) return rc;
            uint32_t gd[3] = {few_dn ? (d + 63) / 64 : (d + 127) / 128, few_dn ? passes : tiles, E};
            if ((rc = ojh_launch(dev, tile_dn, {a16->ptr, wd, nullptr, dv->ptr, nullptr, offsets, list}, {n_ff, d, NA8, E, 1u}, gd, b256)))
                return rc;
            uint64_t n = (uint64_t)T * d;
            uint32_t gs[3] = {(uint32_t)((n + 255) / 256), 1, 1};
            return ojh_launch(dev, "moe_combine", {dv->ptr, wgt->ptr, y->ptr}, {T, ksel, d, (uint32_t)(accum != 0)}, gs, b256);
        }
        const std::string gu_name = std::string("moe_gu_") + fg->tag, down_name = std::string("moe_down_") + fd->tag;
        auto family_of = [](uint32_t t) { return t == OJH_IQ4_XS || t == OJH_IQ4_NL || ojh_grid_type(t) ? "moe_iq" : "moe"; };
        if ((rc = ensure(dev, family_of(gate->type)))) return rc;
        if ((rc = ensure(dev, family_of(down->type)))) return rc;
        ojh_buf *act8;
        if ((rc = ojh_scratch_get(dev, "moe_act", (size_t)NA8 * n_ff * 4, &act8))) return rc;
        uint32_t b256[3] = {256, 1, 1};
        if (!accum) {
            if ((rc = ensure(dev, "glue"))) return rc;
            if ((uint64_t)T * d > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "moe_ffn: %u tokens of %u outputs exceed 2^32 elements", T, d);
            uint32_t n_y = T * d, zg[3] = {(n_y / 4 + 255) / 256 + 1, 1, 1};
            if ((rc = ojh_launch(dev, "fill_zero_u32", {y->ptr}, {n_y}, zg, b256))) return rc;
        }
        uint32_t g1[3] = {(n_ff + 7) / 8, ksel, T};
        if ((rc = ojh_launch(dev, gu_name.c_str(), {x->ptr, (char *)gate->raw->ptr + gate->off, (char *)up->raw->ptr + up->off, act8->ptr, idx->ptr},
                             {d, n_ff, E}, g1, b256)))
            return rc;
        uint32_t g2[3] = {(d + 3) / 4, T, 1};
        return ojh_launch(dev, down_name.c_str(), {act8->ptr, (char *)down->raw->ptr + down->off, y->ptr, idx->ptr, wgt->ptr},
                          {n_ff, d, ksel, E}, g2, b256);
    }
    if (gate->type != OJH_Q4_K || up->type != OJH_Q4_K || (down->type != OJH_Q4_K && down->type != OJH_Q5_K && down->type != OJH_Q6_K))
        return ojh_fail(OJH_ERR_UNSUPPORTED, "moe_ffn: gate and up must be Q4_K with down Q4_K, Q5_K or Q6_K, or gate/up among Q8_0, IQ4_XS, IQ4_NL, IQ3_S, IQ2_XXS, IQ2_S with down among Q8_0, IQ4_XS, IQ4_NL, IQ2_XXS, IQ3_XXS (gate %u, up %u, down %u)",
                        gate->type, up->type, down->type);
    const bool down5 = down->type != OJH_Q4_K;   // Q5_K or Q6_K down tensors: integer dots at every batch size
    const std::string down_dec = std::string("moe_down_") + ojh_format(down->type)->tag + "_dec";
    const std::string down_m = std::string("moe_down_") + ojh_format(down->type)->tag + "_m";
    if (d % 256 || n_ff % 256) return ojh_fail(OJH_ERR_ARG, "moe_ffn: d=%u and n_ff=%u must be multiples of 256", d, n_ff);
    if (gate->k != d || up->k != d || gate->n != (uint64_t)E * n_ff || up->n != gate->n || down->k != n_ff ||
        down->n != (uint64_t)E * d)
        return ojh_fail(OJH_ERR_ARG, "moe_ffn: expert tensor shapes do not match E=%u d=%u n_ff=%u", E, d, n_ff);
    const uint32_t NA = T * ksel;
    int rc;
    if ((rc = span("moe_ffn: x", x, (size_t)T * d * 4, 16))) return rc;
    if ((rc = span("moe_ffn: idx", idx, (size_t)NA * 4, 4))) return rc;
    if ((rc = span("moe_ffn: wgt", wgt, (size_t)NA * 4, 4))) return rc;
    if ((rc = span("moe_ffn: y", y, (size_t)T * d * 4, 4))) return rc;
    if ((rc = ensure(dev, "moe")) || (rc = ensure(dev, "gemv_q8k"))) return rc;

    const uint32_t nsb_d = d / 256, nsb_f = n_ff / 256;
    uint32_t b256[3] = {256, 1, 1};
    // A few tokens: two launches addressed by assignment, activations quantized in registers,
    // weighted sum inside the down launch (bit-identical to the grouped integer-dot pipeline).
    // Measured on MI355X the grouped pipeline takes over once tokens start sharing experts.
    // what the two launches stage in LDS; the down launch keeps one partial sum per slot and lane group for up to 64 slots
    const bool dec_fits = d <= 8192 && n_ff <= 2048 && ksel <= 64 && (uint64_t)ksel * n_ff <= 32768;
    if (dev->moe_mode == 3 || (dev->moe_mode == 0 && T <= dev->moe_dec_tokens && dec_fits)) {
        if (!dec_fits)
            return ojh_fail(OJH_ERR_UNSUPPORTED, "moe_ffn: the decode form serves d <= 8192, n_ff <= 2048, ksel <= 64 and ksel * n_ff <= 32768");
        ojh_buf *act;
        if ((rc = ojh_scratch_get(dev, "moe_act", (size_t)NA * n_ff * 4, &act))) return rc;
        uint32_t g1[3] = {(n_ff + 7) / 8, NA, 1};
        if ((rc = ojh_launch(dev, "moe_gu_q4k_dec",
                             {x->ptr, (char *)gate->raw->ptr + gate->off, (char *)up->raw->ptr + up->off, act->ptr, idx->ptr},
                             {d, n_ff, ksel, NA, E}, g1, b256)))
            return rc;
        uint32_t g2[3] = {(d + 7) / 8, T, 1};
        return ojh_launch(dev, down_dec.c_str(), {act->ptr, (char *)down->raw->ptr + down->off, idx->ptr, wgt->ptr, y->ptr},
                          {n_ff, d, ksel, E, (uint32_t)(accum != 0)}, g2, b256);
    }
    ojh_buf *xq, *xs, *act, *aq, *as_, *dv, *grp;
    if ((rc = ojh_scratch_get(dev, "moe_xq", (size_t)T * d, &xq))) return rc;
    if ((rc = ojh_scratch_get(dev, "moe_xs", (size_t)T * nsb_d * 4, &xs))) return rc;
    if ((rc = ojh_scratch_get(dev, "moe_act", (size_t)NA * n_ff * 4, &act))) return rc;
    if ((rc = ojh_scratch_get(dev, "moe_aq", (size_t)NA * n_ff, &aq))) return rc;
    if ((rc = ojh_scratch_get(dev, "moe_as", (size_t)NA * nsb_f * 4, &as_))) return rc;
    if ((rc = ojh_scratch_get(dev, "moe_dv", (size_t)NA * d * 4, &dv))) return rc;
    // counts[E] | offsets[E+1] | list[NA]
    if ((rc = ojh_scratch_get(dev, "moe_grp", ((size_t)2 * E + 1 + NA) * 4, &grp))) return rc;
    uint32_t *counts = (uint32_t *)grp->ptr, *offsets = counts + E, *list = offsets + E + 1;

    // Expert products: on the matrix cores once experts see a few tokens each (measured crossover on
    // MI355X, 128 experts of 2048 x 768: 4 assignments per expert — 48 tokens of top-8 take 105 us on dots and 115 on
    // the matrix cores, 64 tokens 120 and 116), on integer dots below that.  The two
    // forms round their f32 sums in different orders (last ulp).
    const bool mm = dev->moe_mode == 1 || dev->moe_mode == 4 ||
                    (dev->moe_mode == 0 && (uint64_t)NA >= (uint64_t)4 * E);
    // ... a wave per row tile where 16 tokens of K fit the workgroup's LDS (OJAS_HIP_MOE=4 keeps the workgroup-per-tile form)
    const bool mt_gu = mm && dev->moe_mode != 4 && ojh_moe_mt_lds(d) <= 81920;
    const bool mt_down = mm && dev->moe_mode != 4 && !down5 && ojh_moe_mt_lds(n_ff) <= 81920;
    const uint32_t b512[3] = {512, 1, 1};
    // 1. quantize the tokens once, 2. group the (token, slot) assignments by expert: one launch where a token is one
    //    workgroup's work (the grouping rides along as an extra workgroup), two otherwise
    if (dev->moe_fuse && d <= 8192) {
        uint32_t g[3] = {T + 1, 1, 1};
        if ((rc = ojh_launch(dev, "moe_quant_group", {x->ptr, xq->ptr, xs->ptr, idx->ptr, counts, offsets, list}, {d, T, NA, E}, g, b256)))
            return rc;
    } else {
        if ((rc = ojh_quant_q8k_launch(dev, x->ptr, OJH_X_F32, T, d, xq->ptr, xs->ptr))) return rc;
        uint32_t g1[3] = {1, 1, 1};
        if ((rc = ojh_launch(dev, "moe_group", {idx->ptr, counts, offsets, list}, {NA, E}, g1, b256))) return rc;
    }
    // 3. gate/up + SiLU*mul, one launch over all experts
    {
        uint32_t g[3] = {mt_gu ? ojh_moe_mt_groups(dev, n_ff, E, 1) : mm ? (n_ff + 15) / 16 : (n_ff + 7) / 8, E, 1};
        if ((rc = ojh_launch(dev, mt_gu ? "moe_gu_q4k_mt" : mm ? "moe_gu_q4k_mm" : "moe_gu_q4k_m",
                             {xq->ptr, xs->ptr, (char *)gate->raw->ptr + gate->off, (char *)up->raw->ptr + up->off, act->ptr,
                              offsets, list},
                             {d, n_ff, ksel, NA}, g, mt_gu ? b512 : b256)))
            return rc;
    }
    // 4. quantize every assignment's activation (the CPU path quantizes `act` inside matvec_kq)
    {
        if ((rc = ojh_quant_q8k_launch(dev, act->ptr, OJH_X_F32, NA, n_ff, aq->ptr, as_->ptr))) return rc;
    }
    // 5. down, one launch over all experts.  Q5_K / Q6_K down tensors: once experts see a handful of tokens each, the
    //    int8 matrix tile of the dense path (one scale group per instruction) over each expert's assignments; the
    //    integer-dot form below keeps an expert's rows in registers and walks its assignments one by one
    const uint32_t gs_from = dev->moe_down_gs != 1 ? dev->moe_down_gs : 10u;
    if (down5 && gs_from && (uint64_t)NA >= (uint64_t)gs_from * E && dev->moe_mode != 2) {
        if ((rc = ensure(dev, "gemm_q8k"))) return rc;
        const std::string down_gs = std::string("moe_down_") + ojh_format(down->type)->tag + "_gs";
        uint32_t tiles = (T + 63) / 64;
        if (tiles > 65535) tiles = 65535;
        uint32_t g[3] = {(d + 127) / 128, tiles, E};
        if ((rc = ojh_launch(dev, down_gs.c_str(), {aq->ptr, as_->ptr, (char *)down->raw->ptr + down->off, dv->ptr, offsets, list},
                             {n_ff, d, NA}, g, b256)))
            return rc;
    } else {
        const bool dots = down5 || !mm;
        uint32_t g[3] = {mt_down ? ojh_moe_mt_groups(dev, d, E, 2) : dots && n_ff <= 1024 ? (d + 31) / 32 : (d + 15) / 16, E, 1};
        // (Q5_K rows have no matrix-core form: they stay on integer dots at every batch size)
        if ((rc = ojh_launch(dev, down5 ? down_m.c_str() : mt_down ? "moe_down_q4k_mt" : mm ? "moe_down_q4k_mm" : "moe_down_q4k_m",
                             {aq->ptr, as_->ptr, (char *)down->raw->ptr + down->off, dv->ptr, offsets, list},
                             {n_ff, d, NA}, g, mt_down ? b512 : b256)))
            return rc;
    }
    // 6. router-weighted sum over slots, in slot order
    {
        uint64_t n = (uint64_t)T * d;
        uint32_t g[3] = {(uint32_t)((n + 255) / 256), 1, 1};
        if ((rc = ojh_launch(dev, "moe_combine", {dv->ptr, wgt->ptr, y->ptr}, {T, ksel, d, (uint32_t)(accum != 0)}, g, b256)))
            return rc;
    }
    return OJH_OK;
}

// The decode form over streamed experts: every assignment's gate, up and down matrices sit at a
// byte offset of their arena (the reference's expert cache hands out slots,
// crates/ojas-cuda/src/expert_cache.rs; kernels crates/ojas-cuda/src/kernels/moe.rs:133-174).
extern "C" int ojh_moe_ffn_slots(ojh_device *dev, const ojh_buf *x, uint32_t T, uint32_t d, uint32_t n_ff, uint32_t ksel,
                                 const ojh_buf *arena_gate, const ojh_buf *off_gate, const ojh_buf *arena_up,
                                 const ojh_buf *off_up, const ojh_buf *arena_down, const ojh_buf *off_down,
                                 const ojh_buf *wgt, ojh_buf *y, int accum) {
    if (!dev || !arena_gate || !arena_up || !arena_down) return ojh_fail(OJH_ERR_ARG, "ojh_moe_ffn_slots: NULL argument");
    if (!T || !ksel || ksel > 64 || T > 65535u / ksel)
        return ojh_fail(OJH_ERR_ARG, "moe_ffn_slots: tokens=%u ksel=%u out of range (ksel <= 64, tokens * ksel <= 65535)", T, ksel);
    if (!d || !n_ff || d % 256 || n_ff % 256 || d > 8192 || n_ff > 2048 || (uint64_t)ksel * n_ff > 32768)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "moe_ffn_slots: d=%u (multiple of 256, <= 8192), n_ff=%u (<= 2048), ksel * n_ff <= 32768", d, n_ff);
    const uint32_t NA = T * ksel;
    const size_t gu_bytes = (size_t)n_ff * (d / 256) * 144, dn_bytes = (size_t)d * (n_ff / 256) * 144;
    int rc;
    if ((rc = span("moe_ffn_slots: x", x, (size_t)T * d * 4, 16))) return rc;
    if ((rc = span("moe_ffn_slots: gate arena", arena_gate, gu_bytes, 16))) return rc;
    if ((rc = span("moe_ffn_slots: up arena", arena_up, gu_bytes, 16))) return rc;
    if ((rc = span("moe_ffn_slots: down arena", arena_down, dn_bytes, 16))) return rc;
    if ((rc = span("moe_ffn_slots: gate offsets", off_gate, (size_t)NA * 8, 8))) return rc;
    if ((rc = span("moe_ffn_slots: up offsets", off_up, (size_t)NA * 8, 8))) return rc;
    if ((rc = span("moe_ffn_slots: down offsets", off_down, (size_t)NA * 8, 8))) return rc;
    if ((rc = span("moe_ffn_slots: wgt", wgt, (size_t)NA * 4, 4))) return rc;
    if ((rc = span("moe_ffn_slots: y", y, (size_t)T * d * 4, 4))) return rc;
    if ((rc = ensure(dev, "moe"))) return rc;
    // the last 256-byte step at which a whole expert still fits: offsets beyond it are clamped
    auto lim = [](const ojh_buf *a, size_t e) { return (uint32_t)std::min<size_t>((a->bytes - e) / 256, 0xFFFFFFFFu); };
    ojh_buf *act;
    if ((rc = ojh_scratch_get(dev, "moe_act", (size_t)NA * n_ff * 4, &act))) return rc;
    uint32_t b256[3] = {256, 1, 1}, g1[3] = {(n_ff + 7) / 8, NA, 1}, g2[3] = {(d + 7) / 8, T, 1};
    if ((rc = ojh_launch(dev, "moe_gu_q4k_slots", {x->ptr, arena_gate->ptr, arena_up->ptr, act->ptr, off_gate->ptr, off_up->ptr},
                         {d, n_ff, ksel, NA, lim(arena_gate, gu_bytes), lim(arena_up, gu_bytes)}, g1, b256)))
        return rc;
    return ojh_launch(dev, "moe_down_q4k_slots", {act->ptr, arena_down->ptr, off_down->ptr, wgt->ptr, y->ptr},
                      {n_ff, d, ksel, lim(arena_down, dn_bytes), (uint32_t)(accum != 0)}, g2, b256);
}

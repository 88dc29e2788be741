// Host side of the single-launch decode chain: validates the stages, works out which results travel from stage to
// stage inside the launch, fills the kernel's argument block (kernels/ojk_chain.h) and launches `decode_chain_q4k`
// with one workgroup per compute unit.  The op-level counterpart in the reference is a sequence of `CudaSsm::mm`
// calls (crates/ojas-cuda/src/qwen35.rs:644-702), one or more launches each; see the kernel for what the single
// launch changes.
#include <cstddef>
#include <cstring>

#include "kernels/ojk_chain.h"
#include "ojh_internal.h"

static_assert(OJH_CHAIN_MAX_STAGES == OJK_CHAIN_MAX_STAGES, "public and kernel-side stage limits differ");
static_assert(OJH_CHAIN_X_RMSNORM == OJK_CHAIN_X_RMSNORM && OJH_CHAIN_X_SILU_MUL == OJK_CHAIN_X_SILU_MUL &&
                  OJH_CHAIN_X_GELU_MUL == OJK_CHAIN_X_GELU_MUL,
              "public and kernel-side prologue codes differ");
static_assert(sizeof(ojk_chain_pair) == 8, "a handed-on result is one 8-byte access");

static bool overlaps(const void *a, size_t na, const void *b, size_t nb) {
    const uintptr_t x = (uintptr_t)a, y = (uintptr_t)b;
    return x < y + nb && y < x + na;
}
static bool within(const void *a, size_t na, const void *b, size_t nb) {   // [a, a + na) inside [b, b + nb)
    const uintptr_t x = (uintptr_t)a, y = (uintptr_t)b;
    return x >= y && x + na <= y + nb;
}

// Device state: the abort word (zeroed when allocated, cleared by the host after a failure) and the pinned status
// word the kernels write to.
static int chain_state(ojh_device *dev, uint32_t **abort_word) {
    ojh_buf *b;
    int rc = ojh_scratch_get_zeroed(dev, "chain_abort", 256, &b);
    if (rc) return rc;
    *abort_word = (uint32_t *)b->ptr;
    if (!dev->chain_status) {
        if (dev->capturing)
            return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: first call while recording: run it once eagerly first");
        void *p = nullptr;
        OJH_HIP(hipHostMalloc(&p, 64, hipHostMallocDefault));
        memset(p, 0, 64);
        dev->chain_status = (uint32_t *)p;
    }
    return OJH_OK;
}

int ojh_chain_check_status(ojh_device *dev) {
    if (!dev->chain_status) return OJH_OK;
    const uint32_t st = __atomic_load_n(dev->chain_status, __ATOMIC_ACQUIRE);
    if (!st) return OJH_OK;
    __atomic_store_n(dev->chain_status, 0u, __ATOMIC_RELEASE);
    // every kernel has exited (the stream was just synchronised): let the next launch wait again
    auto it = dev->scratch.find("chain_abort");
    if (it != dev->scratch.end() && it->second) {
        OJH_HIP(hipMemsetAsync(it->second->ptr, 0, 4, dev->stream));
        OJH_HIP(hipStreamSynchronize(dev->stream));
    }
    return ojh_fail(OJH_ERR_HIP, "ojh_decode_chain: a wait for the input of stage %u gave up after its bounded number of polls — "
                                 "the grid was not resident as a whole (or the limit is too small); outputs of chain calls since "
                                 "the last synchronisation are undefined", st - 1);
}

extern "C" int ojh_chain_trace(ojh_device *dev, ojh_buf *buf) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_chain_trace: NULL device");
    const size_t need = (size_t)OJK_CHAIN_MAX_STAGES * OJK_CHAIN_TRACE_EVENTS * 8;
    if (buf && buf->bytes < need)
        return ojh_fail(OJH_ERR_BOUNDS, "ojh_chain_trace: the buffer has %zu bytes, %zu are needed", buf->bytes, need);
    if (buf && (uintptr_t)buf->ptr % 8) return ojh_fail(OJH_ERR_ARG, "ojh_chain_trace: the buffer must be 8-byte aligned");
    dev->chain_trace = buf ? buf->ptr : nullptr;
    return OJH_OK;
}

extern "C" int ojh_chain_spin_limit(ojh_device *dev, uint32_t polls) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_chain_spin_limit: NULL device");
    dev->chain_spin = polls;
    return OJH_OK;
}

// rows per wave of a stage of `rows` rows: two once every compute unit gets several workgroups (the separate
// launches' rule, measured on Q4_K with K = 4096)
static uint32_t rows_per_wave(uint64_t rows, uint32_t cus) { return rows >= (uint64_t)cus * 32u ? 2u : 1u; }

extern "C" int ojh_decode_chain(ojh_device *dev, const ojh_chain_stage *stages, int n_stages) {
    if (!dev || !stages) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: NULL argument");
    if (n_stages < 1 || n_stages > OJK_CHAIN_MAX_STAGES)
        return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: %d stages, takes 1 to %d", n_stages, OJK_CHAIN_MAX_STAGES);
    const uint32_t cus = (uint32_t)dev->prop.multiProcessorCount;
    ojk_chain_args args;
    memset(&args, 0, sizeof args);
    uint64_t rows_of[OJK_CHAIN_MAX_STAGES] = {0};
    int rc;
    for (int s = 0; s < n_stages; s++) {
        const ojh_chain_stage &in = stages[s];
        ojk_chain_stage &out = args.st[s];
        if (in.count < 1 || in.count > 4)
            return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d has count=%d, takes 1 to 4 projections", s, in.count);
        if (in.prologue < OJH_CHAIN_X_PLAIN || in.prologue > OJH_CHAIN_X_RMSNORM)
            return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: unknown prologue %d", s, in.prologue);
        uint64_t total = 0;
        for (int i = 0; i < in.count; i++) {
            const ojh_block_format *fi;
            if ((rc = ojh_mm_checks("ojh_decode_chain", in.ws[i], in.ys[i], in.y_offs[i], nullptr, 1, in.accum, &fi))) return rc;
            if (in.ws[i]->type != OJH_Q4_K)
                return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_decode_chain: stage %d projection %d is %s; the chain multiplies Q4_K rows", s, i,
                                fi->tag);
            if (in.ws[i]->k != in.ws[0]->k)
                return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d projection %d has K=%u, the first has K=%u", s, i, in.ws[i]->k,
                                in.ws[0]->k);
            total += in.ws[i]->n;
        }
        const uint32_t K = in.ws[0]->k;
        if (K % 256 || K > OJK_CHAIN_MAX_K)
            return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_decode_chain: stage %d has K=%u; needs a multiple of 256 up to %u", s, K,
                            OJK_CHAIN_MAX_K);
        if (total > 0x3FFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d has too many rows", s);
        rows_of[s] = total;
        if (!in.x) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: x is NULL", s);
        if (in.x_off > in.x->bytes || (size_t)K * 4 > in.x->bytes - in.x_off)
            return ojh_fail(OJH_ERR_BOUNDS, "ojh_decode_chain: stage %d: x needs %zu bytes at offset %zu, has %zu", s, (size_t)K * 4,
                            in.x_off, in.x->bytes);
        out.x = (const char *)in.x->ptr + in.x_off;
        if ((uintptr_t)out.x % 16) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: x must be 16-byte aligned", s);
        out.x2 = out.x;
        if (in.prologue != OJH_CHAIN_X_PLAIN) {
            if (!in.x2) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: this prologue needs x2", s);
            if (in.x2_off > in.x2->bytes || (size_t)K * 4 > in.x2->bytes - in.x2_off)
                return ojh_fail(OJH_ERR_BOUNDS, "ojh_decode_chain: stage %d: x2 needs %zu bytes at offset %zu, has %zu", s,
                                (size_t)K * 4, in.x2_off, in.x2->bytes);
            out.x2 = (const char *)in.x2->ptr + in.x2_off;
            if ((uintptr_t)out.x2 % 16) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: x2 must be 16-byte aligned", s);
        }
        uint32_t run = 0;
        for (int i = 0; i < 4; i++) {
            const int j = i < in.count ? i : in.count - 1;
            out.w[i] = (const char *)in.ws[j]->raw->ptr + in.ws[j]->off;
            out.y[i] = (char *)in.ys[j]->ptr + in.y_offs[j];
            if (i < in.count) run += in.ws[i]->n;
            out.ends[i] = run;
        }
        // every workgroup reads x while others may already be storing y: they must not share bytes
        for (int i = 0; i < in.count; i++) {
            const size_t yb = (size_t)in.ws[i]->n * 4;
            if (overlaps(out.x, (size_t)K * 4, out.y[i], yb) ||
                (in.prologue != OJH_CHAIN_X_PLAIN && overlaps(out.x2, (size_t)K * 4, out.y[i], yb)))
                return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: output %d overlaps the stage's own input", s, i);
            for (int j2 = 0; j2 < i; j2++)
                if (overlaps(out.y[j2], (size_t)in.ws[j2]->n * 4, out.y[i], yb))
                    return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: outputs %d and %d overlap", s, j2, i);
        }
        out.K = K;
        out.prologue = (uint32_t)in.prologue;
        out.accum = in.accum ? 1u : 0u;
        memcpy(&out.eps_bits, &in.eps, 4);
    }

    // ---- what travels inside the launch.  An input that lies inside an output of an earlier stage is read from
    // that output's tagged copy (the latest such stage wins); one that only straddles such an output cannot be
    // followed and is refused.  The norm's weights are constants and are never handed on.
    struct need { int stage, tensor; };
    size_t xchg_pairs = 0;
    size_t xchg_off[OJK_CHAIN_MAX_STAGES][4];
    bool xchg_used[OJK_CHAIN_MAX_STAGES][4] = {};
    for (int s = 0; s < n_stages; s++)
        for (int i = 0; i < stages[s].count; i++) {
            xchg_off[s][i] = xchg_pairs;
            xchg_pairs += (stages[s].ws[i]->n + 31u) & ~31u;   // every tensor's pairs start on a 256-byte line
        }
    struct src { const void *p; int stage, tensor; size_t first; };
    src from[OJK_CHAIN_MAX_STAGES][2];
    for (int s = 0; s < n_stages; s++) {
        const size_t xb = (size_t)args.st[s].K * 4;
        const bool mul = stages[s].prologue == OJH_CHAIN_X_SILU_MUL || stages[s].prologue == OJH_CHAIN_X_GELU_MUL;
        for (int which = 0; which < 2; which++) {
            from[s][which] = {nullptr, -1, -1, 0};
            if (which && !mul) {
                // the norm's weights (or nothing): must not be something this launch writes
                if (stages[s].prologue == OJH_CHAIN_X_RMSNORM)
                    for (int e = 0; e < n_stages; e++)
                        for (int i = 0; i < stages[e].count; i++)
                            if (overlaps(args.st[s].x2, xb, args.st[e].y[i], (size_t)stages[e].ws[i]->n * 4))
                                return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: stage %d: the norm's weights overlap output %d of stage %d", s, i, e);
                continue;
            }
            const void *p = which ? args.st[s].x2 : args.st[s].x;
            for (int e = s - 1; e >= 0 && from[s][which].stage < 0; e--)
                for (int i = 0; i < stages[e].count; i++) {
                    const size_t yb = (size_t)stages[e].ws[i]->n * 4;
                    if (!overlaps(p, xb, args.st[e].y[i], yb)) continue;
                    if (!within(p, xb, args.st[e].y[i], yb))
                        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_decode_chain: stage %d reads bytes that straddle output %d of stage %d", s, i, e);
                    from[s][which] = {p, e, i, ((uintptr_t)p - (uintptr_t)args.st[e].y[i]) / 4};
                    xchg_used[e][i] = true;
                    break;
                }
            // a later stage may not overwrite what this one reads from the caller's buffers while slower
            // workgroups are still reading it: stages are at most one apart, and stage s + 1 starts only after
            // every workgroup has read its stage-s input, so only the same stage could (refused above)
        }
    }
    // An accumulating stage reads the old values of its outputs.  If an earlier stage of this launch wrote them, they
    // are read from that stage's pairs (whose tags say that they have arrived): the two must then be the same vector,
    // and the stage must depend on the earlier one through its inputs, or nothing orders the two.
    uint32_t dep[OJK_CHAIN_MAX_STAGES] = {0};      // bit e: stage s reads (directly or not) what stage e wrote
    for (int s = 0; s < n_stages; s++)
        for (int which = 0; which < 2; which++)
            if (from[s][which].stage >= 0) dep[s] |= (1u << from[s][which].stage) | dep[from[s][which].stage];
    struct { int stage, tensor; } addfrom[OJK_CHAIN_MAX_STAGES][4];
    for (int s = 0; s < n_stages; s++)
        for (int i = 0; i < 4; i++) addfrom[s][i] = {-1, -1};
    for (int s = 0; s < n_stages; s++) {
        if (!stages[s].accum) continue;
        for (int i = 0; i < stages[s].count; i++)
            for (int e = s - 1; e >= 0 && addfrom[s][i].stage < 0; e--)
                for (int j = 0; j < stages[e].count; j++) {
                    const size_t yb = (size_t)stages[s].ws[i]->n * 4, eb = (size_t)stages[e].ws[j]->n * 4;
                    if (!overlaps(args.st[s].y[i], yb, args.st[e].y[j], eb)) continue;
                    if (args.st[s].y[i] != args.st[e].y[j] || yb != eb)
                        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_decode_chain: stage %d accumulates onto a part of output %d of stage %d; "
                                                             "it must be that whole vector", s, j, e);
                    if (!(dep[s] & (1u << e)))
                        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_decode_chain: stage %d accumulates onto output %d of stage %d without "
                                                             "reading anything that depends on that stage", s, j, e);
                    addfrom[s][i] = {e, j};
                    xchg_used[e][j] = true;
                    break;
                }
    }
    if ((rc = ojh_ensure_family(dev, "chain"))) return rc;
    if (dev->capturing && dev->capture_hip_graph)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_decode_chain: every launch takes a fresh tag, which a captured hipGraph would "
                                             "freeze: record it with the library's own replay (unset OJAS_HIP_REPLAY)");
    uint32_t *abort_word = nullptr;
    if ((rc = chain_state(dev, &abort_word))) return rc;
    // scratch: the handed-on pairs, and per stage the int8 input and the copies of its {scale, tag} table
    size_t xq_bytes = 0;
    for (int s = 0; s < n_stages; s++) xq_bytes += ((size_t)args.st[s].K + 255) & ~(size_t)255;
    const size_t xs_pairs = (size_t)OJK_CHAIN_REPLICAS * 64;
    ojh_buf *xqb, *xsb;
    if ((rc = ojh_scratch_get(dev, "chain_xq", xq_bytes, &xqb))) return rc;
    if ((rc = ojh_scratch_get_zeroed(dev, "chain_xs", (size_t)n_stages * xs_pairs * sizeof(ojk_chain_pair), &xsb))) return rc;
    ojk_chain_pair *xchg = nullptr;
    if (xchg_pairs) {   // zero tags never match: a launch's tag is at least 1
        ojh_buf *xb;
        if ((rc = ojh_scratch_get_zeroed(dev, "chain_xchg", xchg_pairs * sizeof(ojk_chain_pair), &xb))) return rc;
        xchg = (ojk_chain_pair *)xb->ptr;
    }
    uint32_t wg = 0;
    size_t xq_off = 0;
    for (int s = 0; s < n_stages; s++) {
        ojk_chain_stage &st = args.st[s];
        for (int i = 0; i < 4; i++) {
            const int j = i < stages[s].count ? i : stages[s].count - 1;
            st.xchg[i] = xchg_used[s][j] ? xchg + xchg_off[s][j] : nullptr;
            st.addsrc[i] = addfrom[s][j].stage >= 0 ? xchg + xchg_off[addfrom[s][j].stage][addfrom[s][j].tensor] : nullptr;
        }
        for (int which = 0; which < 2; which++) {
            const src &f = from[s][which];
            if (f.stage < 0) continue;
            const void *p = xchg + xchg_off[f.stage][f.tensor] + f.first;
            if (which) st.x2 = p; else st.x = p;
            st.tagged |= 1u << which;
        }
        st.xq = (signed char *)xqb->ptr + xq_off;
        xq_off += ((size_t)st.K + 255) & ~(size_t)255;
        st.xs = (ojk_chain_pair *)xsb->ptr + (size_t)s * xs_pairs;
        st.rows_per_wave = rows_per_wave(rows_of[s], cus);
        st.wg_first = wg;
        st.n_quant = (st.K / 256 + OJK_CHAIN_QSEGS - 1) / OJK_CHAIN_QSEGS;
        const uint64_t row_wgs = (rows_of[s] + 4 * st.rows_per_wave - 1) / (4 * st.rows_per_wave);
        if ((uint64_t)wg + st.n_quant + row_wgs > 0x7FFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_decode_chain: too many workgroups");
        wg += st.n_quant + (uint32_t)row_wgs;
    }
    args.abort_word = abort_word;
    args.status = dev->chain_status;
    args.trace = (uint64_t *)dev->chain_trace;
    args.nstages = (uint32_t)n_stages;
    args.spin_cap = dev->chain_spin;
    args.tag = 0;   // filled in at every launch (also of a recorded one)
    const uint32_t grid[3] = {wg, 1, 1}, block[3] = {OJK_CHAIN_THREADS, 1, 1};
    return ojh_launch_blob(dev, "decode_chain_q4k", &args, sizeof args, grid, block, (int)offsetof(ojk_chain_args, tag));
}

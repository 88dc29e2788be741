// `ojh_mm_noalloc`: the quantized-activation matmul of `ojh_mm` for callers that cannot allocate
// device memory (code under HIP graph capture, tight serving loops, harnesses that forbid it).
//
// `ojh_mm` under OJH_ACT_Q8K stages the int8 form of the activations and their per-256 scales in a
// per-device scratch buffer that it allocates and grows on demand.  Here that staging lives in a
// file-scope device array of fixed size instead, so nothing in the call allocates or frees: the
// quantizer writes into the array, the matvec / MFMA entries read it back: the launches `ojh_mm`
// issues for up to 95 tokens (bit-identical results); beyond, `ojh_mm` may take a prefill tile that
// stages more in library scratch, which this entry never does.
//
// The array's name is a host-side stand-in, not a device address.  Its address on each GPU is
// asked of the runtime once, when a device handle is opened with that GPU current, and only that
// address is ever handed to a kernel.  Every GPU holds its own copy of the array until the
// process ends; all handles opened on one GPU share it, so calls that overlap on one GPU race.
// Nothing in it has to start at zero: the quantizer rewrites every byte a later launch reads.
#include "ojh_internal.h"

// int8 activations [m][K] (K a multiple of 256) followed by f32 scales [m][K/256].
static __device__ __align__(256) unsigned char scratch[OJH_NOALLOC_MAX_ACT + OJH_NOALLOC_MAX_ACT / 64];

static const int kMaxDevices = 64;
static void *g_scratch_ptr[kMaxDevices];   // per GPU ordinal: device address of that GPU's copy

// Called by ojh_open with the device current.
int ojh_noalloc_setup(ojh_device *dev) {
    if (dev->ordinal < 0 || dev->ordinal >= kMaxDevices) {
        dev->noalloc_scratch = nullptr;   // the entry point reports it
        return OJH_OK;
    }
    if (!g_scratch_ptr[dev->ordinal]) {
        void *p = nullptr;
        OJH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p || (uintptr_t)p % 256) return ojh_fail(OJH_ERR_HIP, "the static scratch array resolved to %p", p);
        g_scratch_ptr[dev->ordinal] = p;
    }
    dev->noalloc_scratch = g_scratch_ptr[dev->ordinal];
    return OJH_OK;
}

extern "C" size_t ojh_noalloc_scratch_bytes(void) { return sizeof scratch; }

extern "C" int ojh_mm_noalloc(ojh_device *dev, const ojh_buf *x, size_t x_off, int x_dtype, const ojh_lin *w,
                              ojh_buf *y, size_t y_off, const ojh_buf *bias, uint32_t m, int accum) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_mm_noalloc: NULL device");
    if (!dev->noalloc_scratch)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm_noalloc: no static scratch on device ordinal %d", dev->ordinal);
    const ojh_block_format *f;
    int rc = ojh_mm_checks("ojh_mm_noalloc", w, y, y_off, bias, m, accum, &f);
    if (rc) return rc;
    if (x_dtype != OJH_X_F32 && x_dtype != OJH_X_BF16)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm_noalloc: activations must be f32 or bf16");
    if (ojh_float_rows(w->type))
        return ojh_fail(OJH_ERR_UNSUPPORTED, "ojh_mm_noalloc: %s rows take f32 activations and need no staging: call ojh_mm",
                        f->tag);
    const uint32_t K = w->k;
    const size_t esz = x_dtype == OJH_X_BF16 ? 2 : 4, nsb = K / 256;
    if ((uint64_t)m * nsb * 256 > OJH_NOALLOC_MAX_ACT)
        return ojh_fail(OJH_ERR_BOUNDS, "ojh_mm_noalloc: %u tokens of K=%u are %llu activations, the static scratch holds %u",
                        m, K, (unsigned long long)m * nsb * 256, (unsigned)OJH_NOALLOC_MAX_ACT);
    if (!x) return ojh_fail(OJH_ERR_ARG, "ojh_mm_noalloc: NULL activations");
    if (x_off > x->bytes || (size_t)m * K * esz > x->bytes - x_off)
        return ojh_fail(OJH_ERR_BOUNDS, "ojh_mm_noalloc: x needs %zu bytes at offset %zu, buffer has %zu", (size_t)m * K * esz,
                        x_off, x->bytes);
    if (((uintptr_t)x->ptr + x_off) % 16) return ojh_fail(OJH_ERR_ARG, "ojh_mm_noalloc: x (+%zu) must be 16-byte aligned", x_off);
    // loading a code object allocates: both families must be resident before the call
    if (!dev->modules.count("gemv_q8k") || !dev->modules.count("gemm_q8k"))
        return ojh_fail(OJH_ERR_NOT_LOADED, "ojh_mm_noalloc: ensure_family(\"gemv_q8k\") and (\"gemm_q8k\") first");
    if (ojh_grid_type(w->type) && !dev->modules.count("iq_grid"))   // (before anything is queued into the static scratch)
        return ojh_fail(OJH_ERR_NOT_LOADED, "ojh_mm_noalloc: ensure_family(\"iq_grid\") first");
    void *xq = dev->noalloc_scratch, *xs = (char *)dev->noalloc_scratch + OJH_NOALLOC_MAX_ACT;
    if ((rc = ojh_quant_q8k_launch(dev, (const char *)x->ptr + x_off, x_dtype, m, K, xq, xs))) return rc;
    dev->no_scratch = true;    // kernels that need further library scratch (which would be allocated) are not taken
    rc = ojh_mm_q8k_launch(dev, xq, xs, w, f, (char *)y->ptr + y_off, bias, m, accum);
    dev->no_scratch = false;
    return rc;
}

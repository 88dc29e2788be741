// Host side of the kernel seam: device lifetime, buffers, family loading (hipModuleLoad of the
// gfx950 code objects built offline), dispatch by canonical name, event timing.
// Stands in for `CudaGpu: Device + KernelRuntime` (crates/ojas-cuda/src/device.rs:91-166,
// :341-537) — same obligations (names resolve in exactly one family, unknown kernel is an error
// that says "ensure_family first", read synchronises), none of its code.
#include <dlfcn.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "ojh_internal.h"

static thread_local std::string g_last_error;

int ojh_fail(int code, const char *fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return code;
}

extern "C" const char *ojh_last_error(void) { return g_last_error.c_str(); }
extern "C" int ojh_abi_version(void) { return OJH_ABI_VERSION; }

// Directory holding <family>.hsaco: $OJAS_HIP_HSACO_DIR, else "hsaco" beside this library.
static std::string hsaco_dir() {
    if (const char *e = getenv("OJAS_HIP_HSACO_DIR")) return e;
    Dl_info info;
    if (dladdr((const void *)&ojh_abi_version, &info) && info.dli_fname) {
        std::string p = info.dli_fname;
        size_t s = p.find_last_of('/');
        return (s == std::string::npos ? std::string(".") : p.substr(0, s)) + "/hsaco";
    }
    return "hsaco";
}

extern "C" int ojh_open(int ordinal, ojh_device **out) {
    if (!out) return ojh_fail(OJH_ERR_ARG, "ojh_open: out is NULL");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0)
        return ojh_fail(OJH_ERR_NO_DEVICE, "no HIP device visible (%s); this backend has no CPU fallback",
                        e == hipSuccess ? "count=0" : hipGetErrorString(e));
    if (ordinal < 0 || ordinal >= count)
        return ojh_fail(OJH_ERR_ARG, "device ordinal %d out of range (0..%d)", ordinal, count - 1);
    OJH_HIP(hipSetDevice(ordinal));
    ojh_device *d = new ojh_device();
    d->ordinal = ordinal;
    e = hipGetDeviceProperties(&d->prop, ordinal);
    if (e != hipSuccess) {
        delete d;
        return ojh_fail(OJH_ERR_HIP, "hipGetDeviceProperties: %s", hipGetErrorString(e));
    }
    if (strncmp(d->prop.gcnArchName, "gfx950", 6) != 0 && !getenv("OJAS_HIP_ANY_ARCH")) {
        std::string arch = d->prop.gcnArchName;
        delete d;
        return ojh_fail(OJH_ERR_NO_DEVICE, "device %d is %s; the code objects are built for gfx950 only",
                        ordinal, arch.c_str());
    }
    e = hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&d->ev0);
    if (e == hipSuccess) e = hipEventCreate(&d->ev1);
    if (e != hipSuccess) {
        delete d;
        return ojh_fail(OJH_ERR_HIP, "stream/event creation: %s", hipGetErrorString(e));
    }
    d->name = std::string("hip:") + d->prop.name + " (" + d->prop.gcnArchName + ")";
    if (const char *r = getenv("OJAS_HIP_GEMV_R")) d->gemv_rows_override = atoi(r);
    if (const char *r = getenv("OJAS_HIP_GEMM_MIN_M")) d->gemm_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_GEMM_SPLIT")) d->gemm_split_override = atoi(r);
    if (const char *r = getenv("OJAS_HIP_GEMM_EXACT")) d->gemm_exact = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_Q80_LDS")) d->q80_lds = atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q80_LDS_MIN_N")) d->q80_lds_min_n = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q80_LDS_BPC")) d->q80_lds_bpc = (uint32_t)std::max(0, atoi(r));
    if (const char *r = getenv("OJAS_HIP_Q6K_MF_MIN_M")) d->q6k_mf_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q4K_ML_MIN_M")) d->q4k_ml_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q6K_ML")) d->q6k_ml = atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q6K_ML_MIN_M")) d->q6k_ml_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_PX_BPC")) d->px_bpc = (uint32_t)std::max(0, atoi(r));
    if (const char *r = getenv("OJAS_HIP_PX")) d->px = atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q4K_XT_MIN_M")) d->q4k_xt_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_RMS_THREADS")) d->rms_threads = atoi(r) == 1024 ? 1024u : atoi(r) == 256 ? 256u : 0u;
    if (const char *r = getenv("OJAS_HIP_Q4K_XT_SPLIT")) d->q4k_xt_split = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q4K_XT64")) d->q4k_xt64 = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_Q4K_MF_MIN_M")) d->q4k_mf_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_KQ_GS_MIN_M")) d->kq_gs_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_GEMM_M128")) d->gemm_m128 = atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q80_TILE_MIN_M")) d->q80_tile_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q8ROW_MT_MIN_M")) d->q8row_mt_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q8ROW_T128_MIN_M")) d->q8row_t128_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_MOE_MM_TILE")) d->moe_mm_tile = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_IQ4_TILE")) d->iq4_tile = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_IQ4_TILE_CAP")) d->iq4_tile_cap = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_GEMM_FEW")) d->gemm_few = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_MOE_FEW")) d->moe_few = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_MOE_DOWN_GS")) d->moe_down_gs = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_Q8ROW_DEC")) d->q8row_dec = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_Q8ROW_SPLIT")) d->q8row_split = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_DEQ_BIG_M")) d->deq_big_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_DEQ_MIN_M")) d->deq_min_m = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_KQ_GS_SPLIT")) d->kq_gs_split = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_MOE")) d->moe_mode = atoi(r);
    if (const char *r = getenv("OJAS_HIP_MOE_DEC_TOKENS")) d->moe_dec_tokens = (uint32_t)atoi(r);
    if (const char *r = getenv("OJAS_HIP_MOE_FUSE")) d->moe_fuse = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_MOE_ROUTE_FUSE")) d->moe_route_fuse = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_GEMM_SR")) d->gemm_sr = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_GEMM_BDK")) d->gemm_bdk = atoi(r);
    if (const char *r = getenv("OJAS_HIP_FUSED_QUANT")) d->fused_quant = atoi(r) != 0;
    if (const char *r = getenv("OJAS_HIP_FQ_ROWS")) d->fq_rows = atoi(r) == 1 || atoi(r) == 2 ? atoi(r) : 0;
    if (const char *r = getenv("OJAS_HIP_FQ_THREADS")) d->fq_threads = atoi(r) == 512 ? 512u : atoi(r) == 256 ? 256u : 1024u;
    if (const char *r = getenv("OJAS_HIP_FQ_MULTI_BLOCKS")) d->fq_multi_blocks = atoi(r) > 0 ? (uint32_t)atoi(r) : 1u;
    if (const char *r = getenv("OJAS_HIP_FQ_MULTI")) d->fq_multi = atoi(r);
    if (const char *r = getenv("OJAS_HIP_CHAIN_SPIN")) d->chain_spin = (uint32_t)strtoul(r, nullptr, 10);
    if (const char *r = getenv("OJAS_HIP_FQ_BLOCKS")) d->fq_blocks_per_cu = atoi(r) > 0 ? (uint32_t)atoi(r) : 8u;
    int rc = ojh_noalloc_setup(d);
    if (rc) {
        ojh_close(d);
        return rc;
    }
    *out = d;
    return OJH_OK;
}

extern "C" int ojh_close(ojh_device *dev) {
    if (!dev) return OJH_OK;
    hipSetDevice(dev->ordinal);
    hipStreamSynchronize(dev->stream);
    for (auto &kv : dev->scratch) {
        if (kv.second) {
            if (kv.second->owned) hipFree(kv.second->ptr);
            delete kv.second;
        }
    }
    for (ojh_buf *b : dev->parked) {
        if (b->owned) hipFree(b->ptr);
        delete b;
    }
    if (dev->chain_status) hipHostFree(dev->chain_status);
    for (auto &kv : dev->modules) hipModuleUnload(kv.second);
    for (auto e : dev->marks)
        if (e) hipEventDestroy(e);
    if (dev->ev0) hipEventDestroy(dev->ev0);
    if (dev->ev1) hipEventDestroy(dev->ev1);
    if (dev->stream) hipStreamDestroy(dev->stream);
    delete dev;
    return OJH_OK;
}

extern "C" const char *ojh_name(const ojh_device *dev) { return dev ? dev->name.c_str() : ""; }

extern "C" int ojh_caps_get(const ojh_device *dev, ojh_caps *out) {
    if (!dev || !out) return ojh_fail(OJH_ERR_ARG, "ojh_caps_get: NULL argument");
    memset(out, 0, sizeof *out);
    out->tier = 2;  // matrix units
    out->f16_compute = 1;
    out->simd_width = (uint32_t)dev->prop.warpSize;
    out->unified_memory = 0;
    out->max_buffer = dev->prop.totalGlobalMem;
    out->compute_units = (uint32_t)dev->prop.multiProcessorCount;
    out->clock_mhz = (uint32_t)(dev->prop.clockRate / 1000);
    out->total_memory = dev->prop.totalGlobalMem;
    snprintf(out->arch, sizeof out->arch, "%s", dev->prop.gcnArchName);
    out->features = "mfma_bf16,mfma_f16,mfma_i8,dot4_i8,wave64,offline_code_objects,hip_graphs";
    return OJH_OK;
}

// ---- buffers -----------------------------------------------------------------------------------
extern "C" int ojh_alloc(ojh_device *dev, size_t bytes, ojh_buf **out) {
    if (!dev || !out) return ojh_fail(OJH_ERR_ARG, "ojh_alloc: NULL argument");
    *out = nullptr;
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_alloc while recording a graph");
    OJH_HIP(hipSetDevice(dev->ordinal));
    void *p = nullptr;
    OJH_HIP(hipMalloc(&p, bytes ? bytes : 1));
    ojh_buf *b = new ojh_buf();
    b->ptr = p;
    b->bytes = bytes;
    b->owned = true;
    *out = b;
    return OJH_OK;
}

extern "C" int ojh_wrap(ojh_device *dev, void *device_ptr, size_t bytes, ojh_buf **out) {
    if (!dev || !out || !device_ptr) return ojh_fail(OJH_ERR_ARG, "ojh_wrap: NULL argument");
    ojh_buf *b = new ojh_buf();
    b->ptr = device_ptr;
    b->bytes = bytes;
    b->owned = false;
    *out = b;
    return OJH_OK;
}

extern "C" int ojh_free(ojh_device *dev, ojh_buf *buf) {
    if (!buf) return OJH_OK;
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_free: NULL device");
    if (buf->owned && dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_free while recording a graph");
    if (buf->owned) {
        // work queued on the stream may still read the buffer
        OJH_HIP(hipStreamSynchronize(dev->stream));
        OJH_HIP(hipFree(buf->ptr));
    }
    delete buf;
    return OJH_OK;
}

extern "C" size_t ojh_buf_bytes(const ojh_buf *buf) { return buf ? buf->bytes : 0; }
extern "C" void *ojh_buf_ptr(const ojh_buf *buf) { return buf ? buf->ptr : nullptr; }

static int range_ok(const char *what, const ojh_buf *b, size_t off, size_t bytes) {
    if (!b) return ojh_fail(OJH_ERR_ARG, "%s: NULL buffer", what);
    if (off > b->bytes || bytes > b->bytes - off)
        return ojh_fail(OJH_ERR_BOUNDS, "%s: [%zu, +%zu) exceeds the buffer's %zu bytes", what, off, bytes,
                        b->bytes);
    return OJH_OK;
}

extern "C" int ojh_upload(ojh_device *dev, ojh_buf *dst, size_t off, const void *host, size_t bytes) {
    if (!dev || (!host && bytes)) return ojh_fail(OJH_ERR_ARG, "ojh_upload: NULL argument");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_upload while recording a graph");
    int rc = range_ok("ojh_upload", dst, off, bytes);
    if (rc) return rc;
    if (!bytes) return OJH_OK;
    // Ordered after earlier work on the stream; returns when the host buffer has been consumed.
    OJH_HIP(hipMemcpyAsync((char *)dst->ptr + off, host, bytes, hipMemcpyHostToDevice, dev->stream));
    OJH_HIP(hipStreamSynchronize(dev->stream));
    return OJH_OK;
}

extern "C" int ojh_download(ojh_device *dev, const ojh_buf *src, size_t off, void *host, size_t bytes) {
    if (!dev || (!host && bytes)) return ojh_fail(OJH_ERR_ARG, "ojh_download: NULL argument");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_download while recording a graph");
    int rc = range_ok("ojh_download", src, off, bytes);
    if (rc) return rc;
    if (!bytes) return OJH_OK;
    OJH_HIP(hipMemcpyAsync(host, (const char *)src->ptr + off, bytes, hipMemcpyDeviceToHost, dev->stream));
    OJH_HIP(hipStreamSynchronize(dev->stream));
    return ojh_chain_check_status(dev);
}

extern "C" int ojh_memset0(ojh_device *dev, ojh_buf *dst, size_t off, size_t bytes) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_memset0: NULL device");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_memset0 while recording a graph: dispatch fill_zero_u32");
    int rc = range_ok("ojh_memset0", dst, off, bytes);
    if (rc) return rc;
    if (!bytes) return OJH_OK;
    OJH_HIP(hipMemsetAsync((char *)dst->ptr + off, 0, bytes, dev->stream));
    return OJH_OK;
}

// `fresh` (optional) tells whether the slot was (re)allocated by this call: its contents are then undefined.
static int scratch_get(ojh_device *dev, const char *name, size_t bytes, ojh_buf **out, bool *fresh) {
    ojh_buf *&slot = dev->scratch[name];
    if (fresh) *fresh = false;
    if (!slot || slot->bytes < bytes) {
        if (dev->capturing)
            return ojh_fail(OJH_ERR_ARG, "scratch '%s' would have to grow while recording a graph: run the call once "
                                          "eagerly first", name);
        if (slot && dev->live_graphs > 0) {   // a recorded chain may still replay into it
            dev->parked.push_back(slot);
            slot = nullptr;
        } else if (slot) {
            int rc = ojh_free(dev, slot);
            slot = nullptr;
            if (rc) return rc;
        }
        size_t cap = bytes < 4096 ? 4096 : bytes + bytes / 4;
        int rc = ojh_alloc(dev, cap, &slot);
        if (rc) return rc;
        if (fresh) *fresh = true;
    }
    *out = slot;
    return OJH_OK;
}

int ojh_scratch_get(ojh_device *dev, const char *name, size_t bytes, ojh_buf **out) {
    return scratch_get(dev, name, bytes, out, nullptr);
}

// Cleared whenever the slot is (re)allocated — decided by the allocation itself, not by comparing addresses: the
// allocator may hand a grown slot the address the freed one had.
int ojh_scratch_get_zeroed(ojh_device *dev, const char *name, size_t bytes, ojh_buf **out) {
    bool fresh = false;
    int rc = scratch_get(dev, name, bytes, out, &fresh);
    if (rc) return rc;
    if (fresh) OJH_HIP(hipMemsetAsync((*out)->ptr, 0, (*out)->bytes, dev->stream));   // (never while capturing: growth is refused there)
    return OJH_OK;
}

// ---- families ----------------------------------------------------------------------------------
extern "C" int ojh_ensure_family(ojh_device *dev, const char *family) {
    if (!dev || !family) return ojh_fail(OJH_ERR_ARG, "ojh_ensure_family: NULL argument");
    if (dev->modules.count(family)) return OJH_OK;
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_ensure_family(%s) while recording a graph", family);
    bool known = false;
    for (const auto &s : ojh_manifest_table())
        if (!strcmp(s.family, family)) known = true;
    if (!known) return ojh_fail(OJH_ERR_UNSUPPORTED, "unknown kernel family '%s'", family);
    OJH_HIP(hipSetDevice(dev->ordinal));
    std::string path = hsaco_dir() + "/" + family + ".hsaco";
    hipModule_t mod = nullptr;
    hipError_t e = hipModuleLoad(&mod, path.c_str());
    if (e != hipSuccess)
        return ojh_fail(OJH_ERR_HIP, "hipModuleLoad(%s): %s — build the code objects first", path.c_str(),
                        hipGetErrorString(e));
    // every manifest entry of the family must resolve: a name that drifted is a build error
    std::map<std::string, hipFunction_t> found;
    for (const auto &s : ojh_manifest_table()) {
        if (strcmp(s.family, family)) continue;
        hipFunction_t fn = nullptr;
        e = hipModuleGetFunction(&fn, mod, s.name);
        if (e != hipSuccess) {
            hipModuleUnload(mod);
            return ojh_fail(OJH_ERR_HIP, "family '%s' does not define kernel '%s': %s", family, s.name,
                            hipGetErrorString(e));
        }
        found[s.name] = fn;
    }
    dev->modules[family] = mod;
    for (auto &kv : found) dev->functions[kv.first] = kv.second;
    return OJH_OK;
}

extern "C" int ojh_has_kernel(const ojh_device *dev, const char *name) {
    return dev && name && dev->functions.count(name) ? 1 : 0;
}

extern "C" int ojh_launch_shape(const ojh_device *dev, const char *name, uint32_t K, uint32_t N, uint32_t M,
                                uint32_t grid[3], uint32_t block[3]) {
    const ojh_kernel_spec *s = ojh_find_kernel(name);
    if (!s) return ojh_fail(OJH_ERR_UNSUPPORTED, "unknown kernel '%s'", name ? name : "(null)");
    if (!grid || !block) return ojh_fail(OJH_ERR_ARG, "ojh_launch_shape: NULL output");
    return s->shape(s, dev, K, N, M, grid, block);
}

int ojh_launch(ojh_device *dev, const char *name, const std::vector<void *> &ptrs,
               const std::vector<uint32_t> &consts, const uint32_t grid[3], const uint32_t block[3]) {
    auto it = dev->functions.find(name);
    if (it == dev->functions.end())
        return ojh_fail(OJH_ERR_NOT_LOADED, "kernel '%s' not loaded — ensure_family first", name);
    if (!grid[0] || !grid[1] || !grid[2] || !block[0] || !block[1] || !block[2])
        return ojh_fail(OJH_ERR_ARG, "%s: empty grid or block", name);
    if (ptrs.size() + consts.size() > 16) return ojh_fail(OJH_ERR_ARG, "%s: too many arguments", name);
    if (dev->capturing && !dev->capture_hip_graph) {
        ojh_command cmd;
        cmd.fn = it->second;
        cmd.ptrs = ptrs;
        cmd.consts = consts;
        for (int i = 0; i < 3; i++) { cmd.grid[i] = grid[i]; cmd.block[i] = block[i]; }
        dev->recorded.push_back(cmd);
        return OJH_OK;
    }
    std::vector<void *> p = ptrs;
    std::vector<uint32_t> c = consts;
    void *args[16];
    int n = 0;
    for (auto &x : p) args[n++] = &x;
    for (auto &x : c) args[n++] = &x;
    OJH_HIP(hipModuleLaunchKernel(it->second, grid[0], grid[1], grid[2], block[0], block[1], block[2], 0,
                                  dev->stream, args, nullptr));
    return OJH_OK;
}

static hipError_t launch_command(ojh_device *dev, ojh_command &c) {
    if (!c.blob.empty()) {
        if (c.tag_offset >= 0) {   // a tag no earlier launch of this device had (0 is never one)
            if (++dev->chain_tag == 0) ++dev->chain_tag;
            memcpy(c.blob.data() + c.tag_offset, &dev->chain_tag, 4);
        }
        size_t bytes = c.blob.size();
        void *extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, c.blob.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &bytes, HIP_LAUNCH_PARAM_END};
        return hipModuleLaunchKernel(c.fn, c.grid[0], c.grid[1], c.grid[2], c.block[0], c.block[1], c.block[2], 0, dev->stream,
                                     nullptr, extra);
    }
    void *args[16];
    int n = 0;
    for (auto &p : c.ptrs) args[n++] = &p;
    for (auto &v : c.consts) args[n++] = &v;
    return hipModuleLaunchKernel(c.fn, c.grid[0], c.grid[1], c.grid[2], c.block[0], c.block[1], c.block[2], 0, dev->stream, args,
                                 nullptr);
}

int ojh_launch_blob(ojh_device *dev, const char *name, const void *args, size_t bytes, const uint32_t grid[3],
                    const uint32_t block[3], int tag_offset) {
    auto it = dev->functions.find(name);
    if (it == dev->functions.end())
        return ojh_fail(OJH_ERR_NOT_LOADED, "kernel '%s' not loaded — ensure_family first", name);
    if (!grid[0] || !grid[1] || !grid[2] || !block[0] || !block[1] || !block[2])
        return ojh_fail(OJH_ERR_ARG, "%s: empty grid or block", name);
    ojh_command cmd;
    cmd.fn = it->second;
    cmd.blob.assign((const uint8_t *)args, (const uint8_t *)args + bytes);
    cmd.tag_offset = tag_offset;
    for (int i = 0; i < 3; i++) { cmd.grid[i] = grid[i]; cmd.block[i] = block[i]; }
    if (dev->capturing && !dev->capture_hip_graph) {
        dev->recorded.push_back(std::move(cmd));
        return OJH_OK;
    }
    OJH_HIP(launch_command(dev, cmd));
    return OJH_OK;
}

extern "C" int ojh_dispatch(ojh_device *dev, const char *name, int n_bufs, ojh_buf *const *bufs,
                            const uint64_t *offsets, int n_consts, const uint32_t *consts,
                            const uint32_t grid[3], const uint32_t block[3]) {
    if (!dev || !name || !grid || !block) return ojh_fail(OJH_ERR_ARG, "ojh_dispatch: NULL argument");
    const ojh_kernel_spec *s = ojh_find_kernel(name);
    if (!s) return ojh_fail(OJH_ERR_NOT_LOADED, "kernel '%s' not loaded — ensure_family first", name);
    if (!dev->functions.count(name))
        return ojh_fail(OJH_ERR_NOT_LOADED, "kernel '%s' not loaded — ensure_family(\"%s\") first", name,
                        s->family);
    if (n_bufs != s->n_bufs || n_consts != s->n_consts)
        return ojh_fail(OJH_ERR_ARG, "%s takes %d buffers then %d constants, got %d and %d", name, s->n_bufs,
                        s->n_consts, n_bufs, n_consts);
    if ((n_bufs && !bufs) || (n_consts && !consts)) return ojh_fail(OJH_ERR_ARG, "%s: NULL argument array", name);
    size_t need[16] = {0}, align[16];
    for (auto &a : align) a = 16;
    int rc = s->check(s, consts, grid, block, need, align);
    if (rc) return rc;
    std::vector<void *> ptrs;
    for (int i = 0; i < n_bufs; i++) {
        size_t off = offsets ? (size_t)offsets[i] : 0;
        if (!bufs[i] && align[i] == 0) {     // a buffer the kernel takes as optional (a bias that may be absent)
            ptrs.push_back(nullptr);
            continue;
        }
        if (!bufs[i]) return ojh_fail(OJH_ERR_ARG, "%s: buffer %d is NULL", name, i);
        if (align[i] == 0) align[i] = 4;
        if (off > bufs[i]->bytes || need[i] > bufs[i]->bytes - off)
            return ojh_fail(OJH_ERR_BOUNDS, "%s: buffer %d needs %zu bytes at offset %zu, has %zu", name, i,
                            need[i], off, bufs[i]->bytes);
        uintptr_t addr = (uintptr_t)bufs[i]->ptr + off;
        if (addr % align[i])
            return ojh_fail(OJH_ERR_ARG, "%s: buffer %d (+%zu) must be %zu-byte aligned", name, i, off, align[i]);
        ptrs.push_back((void *)addr);
    }
    std::vector<uint32_t> cv(consts, consts + n_consts);
    if (s->expert_bufs) {   // how many experts the tensors hold: the kernel's bound on the routed indices
        size_t experts = 0xFFFFFFFFu;
        for (int i = s->bound_first; i < s->bound_first + s->expert_bufs; i++) {
            size_t off = offsets ? (size_t)offsets[i] : 0;
            experts = std::min(experts, (bufs[i]->bytes - off) / need[i]);
        }
        cv.push_back((uint32_t)experts);
    }
    for (int i = 1; i <= s->arena_bufs; i++) {   // the kernels clamp their u32 offsets to this
        size_t off = offsets ? (size_t)offsets[i] : 0;
        cv.push_back((uint32_t)std::min<size_t>(bufs[i]->bytes - off - need[i], 0xFFFFFFFEu));
    }
    return ojh_launch(dev, name, ptrs, cv, grid, block);
}

extern "C" int ojh_submit(ojh_device *dev) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_submit: NULL device");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_submit while recording a graph");
    OJH_HIP(hipStreamSynchronize(dev->stream));
    return ojh_chain_check_status(dev);
}

extern "C" int ojh_timer_start(ojh_device *dev) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_timer_start: NULL device");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_timer_start while recording a graph");
    OJH_HIP(hipEventRecord(dev->ev0, dev->stream));
    return OJH_OK;
}

extern "C" int ojh_timer_stop(ojh_device *dev, float *elapsed_ms) {
    if (!dev || !elapsed_ms) return ojh_fail(OJH_ERR_ARG, "ojh_timer_stop: NULL argument");
    OJH_HIP(hipEventRecord(dev->ev1, dev->stream));
    OJH_HIP(hipEventSynchronize(dev->ev1));
    OJH_HIP(hipEventElapsedTime(elapsed_ms, dev->ev0, dev->ev1));
    return OJH_OK;
}

extern "C" int ojh_mark(ojh_device *dev, int slot) {
    if (!dev || slot < 0 || slot >= OJH_MAX_MARKS) return ojh_fail(OJH_ERR_ARG, "ojh_mark: slot %d out of range", slot);
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_mark while recording a graph");
    if ((size_t)slot >= dev->marks.size()) dev->marks.resize((size_t)slot + 1, nullptr);
    if (!dev->marks[slot]) OJH_HIP(hipEventCreate(&dev->marks[slot]));
    OJH_HIP(hipEventRecord(dev->marks[slot], dev->stream));
    return OJH_OK;
}

extern "C" int ojh_mark_elapsed(ojh_device *dev, int a, int b, float *elapsed_ms) {
    if (!dev || !elapsed_ms) return ojh_fail(OJH_ERR_ARG, "ojh_mark_elapsed: NULL argument");
    if (a < 0 || b < 0 || (size_t)a >= dev->marks.size() || (size_t)b >= dev->marks.size() || !dev->marks[a] ||
        !dev->marks[b])
        return ojh_fail(OJH_ERR_ARG, "ojh_mark_elapsed: slot %d or %d was never recorded", a, b);
    OJH_HIP(hipEventSynchronize(dev->marks[b]));
    OJH_HIP(hipEventElapsedTime(elapsed_ms, dev->marks[a], dev->marks[b]));
    return OJH_OK;
}

// ---- record and replay -------------------------------------------------------------------------
// Two replay engines behind one interface.  The default keeps the recorded launches as a command
// list and re-issues them from one tight native loop: on this ROCm a HIP-graph kernel node costs
// about 4.5 us of device timeline against about 1.6 us for an in-order launch, so for chains of
// few-microsecond matvecs the list is the faster replay.  OJAS_HIP_REPLAY=graph selects stream
// capture into a hipGraph instead.
extern "C" int ojh_capture_begin(ojh_device *dev) {
    if (!dev) return ojh_fail(OJH_ERR_ARG, "ojh_capture_begin: NULL device");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_capture_begin: already recording");
    const char *mode = getenv("OJAS_HIP_REPLAY");
    dev->capture_hip_graph = mode && !strcmp(mode, "graph");
    if (dev->capture_hip_graph) OJH_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeThreadLocal));
    dev->recorded.clear();
    dev->capturing = true;
    return OJH_OK;
}

extern "C" int ojh_capture_end(ojh_device *dev, ojh_graph **out) {
    if (!dev || !out) return ojh_fail(OJH_ERR_ARG, "ojh_capture_end: NULL argument");
    *out = nullptr;
    if (!dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_capture_end: not recording");
    dev->capturing = false;
    ojh_graph *gr = new ojh_graph();
    if (dev->capture_hip_graph) {
        hipGraph_t g = nullptr;
        hipError_t e = hipStreamEndCapture(dev->stream, &g);
        if (e == hipSuccess) e = hipGraphInstantiate(&gr->exec, g, nullptr, nullptr, 0);
        if (e != hipSuccess) {
            // the capture has ended either way (an invalidated one too): the stream runs eagerly again
            if (g) hipGraphDestroy(g);
            delete gr;
            (void)hipGetLastError();
            return ojh_fail(OJH_ERR_HIP, "graph capture/instantiate: %s", hipGetErrorString(e));
        }
        gr->graph = g;
    } else {
        gr->list.swap(dev->recorded);
    }
    dev->live_graphs++;
    *out = gr;
    return OJH_OK;
}

extern "C" int ojh_graph_launch(ojh_device *dev, ojh_graph *graph) {
    if (!dev || !graph) return ojh_fail(OJH_ERR_ARG, "ojh_graph_launch: NULL argument");
    if (dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_graph_launch while recording a graph");
    if (graph->exec) {
        OJH_HIP(hipGraphLaunch(graph->exec, dev->stream));
        return OJH_OK;
    }
    for (auto &c : graph->list) OJH_HIP(launch_command(dev, c));
    return OJH_OK;
}

extern "C" int ojh_graph_free(ojh_device *dev, ojh_graph *graph) {
    if (!graph) return OJH_OK;
    if (dev) hipStreamSynchronize(dev->stream);
    if (graph->exec) hipGraphExecDestroy(graph->exec);
    if (graph->graph) hipGraphDestroy(graph->graph);
    delete graph;
    if (dev && dev->live_graphs > 0 && --dev->live_graphs == 0) {   // nothing can replay into the outgrown buffers any more
        for (ojh_buf *b : dev->parked) {
            if (b->owned) hipFree(b->ptr);
            delete b;
        }
        dev->parked.clear();
    }
    return OJH_OK;
}

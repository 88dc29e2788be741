// GGUF container reader and the loader that puts tensors on the device as `Lin` handles.
//
// What it follows in the reference: header / metadata / tensor-index parsing and its limits
// (crates/ojas-formats/src/gguf.rs:51-52, 100-206), `tensor_meta` and `read_tensor_raw`
// (:440-452, :551-556), the on-disk size table `stored_bytes` (:563-591), and `Lin::load`'s
// stacking and keep-in-place rules (crates/ojas-cuda/src/qwen35.rs:174-201): the tensors of a
// fused group must share K and the GGUF type, rows stack along N, and Q4_K / Q6_K / Q8_0 stay in
// the file's block bytes when K is a whole number of blocks.  Split (multi-file) models are not
// merged here: a file announcing split.count > 1 is refused.
#include <cstdio>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "ojh_internal.h"

namespace {

constexpr uint64_t kMaxHeaderBytes = 256ull << 20;   // gguf.rs:51
constexpr uint64_t kMaxHeaderItems = 1048576;        // gguf.rs:52

struct Meta {
    int kind = 0;   // 1 unsigned, 2 signed, 3 float, 4 bool, 5 string, 6 array (consumed)
    uint64_t u = 0;
    int64_t i = 0;
    double f = 0;
    std::string s;
};

struct TensorInfo {
    std::string name;
    std::vector<uint64_t> dims;
    uint32_t type = 0;
    uint64_t rel_offset = 0;
};

}  // namespace

struct ojh_gguf {
    FILE *fp = nullptr;
    std::string path;
    uint64_t file_len = 0, data_offset = 0;
    uint32_t version = 0;
    std::map<std::string, Meta> meta;
    std::vector<TensorInfo> tensors;
    std::map<std::string, size_t> by_name;
};

namespace {

struct Reader {
    FILE *fp;
    uint64_t pos, end;
    bool take(void *dst, uint64_t n) {
        if (n > end - pos) return false;
        if (n && fread(dst, 1, n, fp) != n) return false;
        pos += n;
        return true;
    }
    template <class T> bool get(T *v) { return take(v, sizeof(T)); }
    bool str(std::string *s) {
        uint64_t n;
        if (!get(&n) || n > end - pos) return false;
        s->resize(n);
        return take(n ? &(*s)[0] : nullptr, n);
    }
};

// bytes `elems` weights of GGUF type `ty` occupy on disk; 0 for a type this reader does not know
uint64_t stored_bytes(uint32_t ty, uint64_t elems) {
    switch (ty) {
    case 0: return elems * 4;            // F32
    case 1: case 30: return elems * 2;   // F16, BF16
    case 2: case 20: return elems / 32 * 18;   // Q4_0, IQ4_NL
    case 3: return elems / 32 * 20;      // Q4_1
    case 6: return elems / 32 * 22;      // Q5_0
    case 7: return elems / 32 * 24;      // Q5_1
    case 8: return elems / 32 * 34;      // Q8_0
    case 10: return elems / 256 * 84;    // Q2_K
    case 11: case 21: return elems / 256 * 110;  // Q3_K, IQ3_S
    case 12: return elems / 256 * 144;   // Q4_K
    case 13: return elems / 256 * 176;   // Q5_K
    case 14: return elems / 256 * 210;   // Q6_K
    case 16: return elems / 256 * 66;    // IQ2_XXS
    case 17: return elems / 256 * 74;    // IQ2_XS
    case 18: return elems / 256 * 98;    // IQ3_XXS
    case 19: return elems / 256 * 50;    // IQ1_S
    case 22: return elems / 256 * 82;    // IQ2_S
    case 23: return elems / 256 * 136;   // IQ4_XS
    case 29: return elems / 256 * 56;    // IQ1_M
    case 42: return elems / 128 * 34;    // Q2_0
    default: return 0;
    }
}

bool read_scalar(Reader &r, uint32_t t, Meta *m) {
    switch (t) {
    case 0: { uint8_t v; if (!r.get(&v)) return false; m->kind = 1; m->u = v; return true; }
    case 1: { int8_t v; if (!r.get(&v)) return false; m->kind = 2; m->i = v; return true; }
    case 2: { uint16_t v; if (!r.get(&v)) return false; m->kind = 1; m->u = v; return true; }
    case 3: { int16_t v; if (!r.get(&v)) return false; m->kind = 2; m->i = v; return true; }
    case 4: { uint32_t v; if (!r.get(&v)) return false; m->kind = 1; m->u = v; return true; }
    case 5: { int32_t v; if (!r.get(&v)) return false; m->kind = 2; m->i = v; return true; }
    case 6: { float v; if (!r.get(&v)) return false; m->kind = 3; m->f = v; return true; }
    case 7: { uint8_t v; if (!r.get(&v)) return false; m->kind = 4; m->u = v != 0; return true; }
    case 8: m->kind = 5; return r.str(&m->s);
    case 10: { uint64_t v; if (!r.get(&v)) return false; m->kind = 1; m->u = v; return true; }
    case 11: { int64_t v; if (!r.get(&v)) return false; m->kind = 2; m->i = v; return true; }
    case 12: { double v; if (!r.get(&v)) return false; m->kind = 3; m->f = v; return true; }
    default: return false;
    }
}

int parse(ojh_gguf *g) {
    Reader r{g->fp, 0, g->file_len < kMaxHeaderBytes ? g->file_len : kMaxHeaderBytes};
    char magic[4];
    if (!r.take(magic, 4) || memcmp(magic, "GGUF", 4)) return ojh_fail(OJH_ERR_ARG, "%s: not a GGUF file", g->path.c_str());
    uint64_t n_tensors, n_kv;
    if (!r.get(&g->version) || (g->version != 2 && g->version != 3))
        return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: unsupported GGUF version %u", g->path.c_str(), g->version);
    if (!r.get(&n_tensors) || !r.get(&n_kv) || n_tensors > kMaxHeaderItems || n_kv > kMaxHeaderItems)
        return ojh_fail(OJH_ERR_ARG, "%s: GGUF header item count exceeds limit", g->path.c_str());
    for (uint64_t k = 0; k < n_kv; k++) {
        std::string key;
        uint32_t t;
        if (!r.str(&key) || !r.get(&t)) return ojh_fail(OJH_ERR_ARG, "%s: truncated GGUF metadata", g->path.c_str());
        Meta m;
        if (t == 9) {   // array: element type + count; consumed, not kept
            uint32_t et;
            uint64_t n;
            if (!r.get(&et) || !r.get(&n) || et > 12 || et == 9)
                return ojh_fail(OJH_ERR_ARG, "%s: invalid or nested GGUF array type in '%s'", g->path.c_str(), key.c_str());
            if (n > kMaxHeaderItems || n > r.end - r.pos)
                return ojh_fail(OJH_ERR_ARG, "%s: GGUF array '%s' exceeds metadata bounds", g->path.c_str(), key.c_str());
            for (uint64_t i = 0; i < n; i++) {
                Meta e;
                if (!read_scalar(r, et, &e)) return ojh_fail(OJH_ERR_ARG, "%s: truncated GGUF array '%s'", g->path.c_str(), key.c_str());
            }
            m.kind = 6;
            m.u = n;
        } else if (!read_scalar(r, t, &m)) {
            return ojh_fail(OJH_ERR_ARG, "%s: bad GGUF metadata value for '%s' (type %u)", g->path.c_str(), key.c_str(), t);
        }
        g->meta[key] = m;
    }
    for (uint64_t i = 0; i < n_tensors; i++) {
        TensorInfo ti;
        uint32_t nd;
        if (!r.str(&ti.name) || !r.get(&nd)) return ojh_fail(OJH_ERR_ARG, "%s: truncated GGUF tensor index", g->path.c_str());
        if (nd < 1 || nd > 4) return ojh_fail(OJH_ERR_ARG, "%s: invalid GGUF tensor rank %u", g->path.c_str(), nd);
        uint64_t elems = 1;
        bool ok = true;
        for (uint32_t d = 0; d < nd; d++) {
            uint64_t v;
            if (!r.get(&v)) return ojh_fail(OJH_ERR_ARG, "%s: truncated GGUF tensor index", g->path.c_str());
            ti.dims.push_back(v);
            if (v == 0 || elems > (UINT64_MAX / 8) / v) ok = false; else elems *= v;
        }
        if (!ok) return ojh_fail(OJH_ERR_ARG, "%s: invalid or overflowing dimensions of tensor '%s'", g->path.c_str(), ti.name.c_str());
        if (!r.get(&ti.type) || !r.get(&ti.rel_offset)) return ojh_fail(OJH_ERR_ARG, "%s: truncated GGUF tensor index", g->path.c_str());
        if (g->by_name.count(ti.name)) return ojh_fail(OJH_ERR_ARG, "%s: duplicate GGUF tensor %s", g->path.c_str(), ti.name.c_str());
        g->by_name[ti.name] = g->tensors.size();
        g->tensors.push_back(ti);
    }
    uint64_t align = 32;
    auto it = g->meta.find("general.alignment");
    if (it != g->meta.end() && it->second.kind == 1) align = it->second.u;
    if (!align || (align & (align - 1))) return ojh_fail(OJH_ERR_ARG, "%s: invalid GGUF alignment %llu", g->path.c_str(), (unsigned long long)align);
    g->data_offset = (r.pos + align - 1) & ~(align - 1);
    auto sc = g->meta.find("split.count");
    if (sc != g->meta.end() && ((sc->second.kind == 1 && sc->second.u > 1) || (sc->second.kind == 2 && sc->second.i > 1)))
        return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: split GGUF models (split.count > 1) are not merged by this loader", g->path.c_str());
    for (const auto &t : g->tensors) {
        uint64_t elems = 1;
        for (uint64_t d : t.dims) elems *= d;
        uint64_t bytes = stored_bytes(t.type, elems), start = g->data_offset + t.rel_offset;
        if (start < g->data_offset || start >= g->file_len)
            return ojh_fail(OJH_ERR_ARG, "%s: GGUF tensor %s starts outside file", g->path.c_str(), t.name.c_str());
        if (bytes && bytes > g->file_len - start)
            return ojh_fail(OJH_ERR_ARG, "%s: GGUF tensor %s extends past the end of the file", g->path.c_str(), t.name.c_str());
    }
    return OJH_OK;
}

const TensorInfo *find(const ojh_gguf *g, const char *name) {
    if (!g || !name) return nullptr;
    auto it = g->by_name.find(name);
    return it == g->by_name.end() ? nullptr : &g->tensors[it->second];
}

}  // namespace

extern "C" int ojh_gguf_open(const char *path, ojh_gguf **out) {
    if (!path || !out) return ojh_fail(OJH_ERR_ARG, "ojh_gguf_open: NULL argument");
    *out = nullptr;
    FILE *fp = fopen(path, "rb");
    if (!fp) return ojh_fail(OJH_ERR_ARG, "ojh_gguf_open: cannot open %s", path);
    ojh_gguf *g = new ojh_gguf();
    g->fp = fp;
    g->path = path;
    fseeko(fp, 0, SEEK_END);
    g->file_len = (uint64_t)ftello(fp);
    fseeko(fp, 0, SEEK_SET);
    int rc = parse(g);
    if (rc) {
        fclose(fp);
        delete g;
        return rc;
    }
    *out = g;
    return OJH_OK;
}

extern "C" int ojh_gguf_close(ojh_gguf *g) {
    if (!g) return OJH_OK;
    if (g->fp) fclose(g->fp);
    delete g;
    return OJH_OK;
}

extern "C" int ojh_gguf_tensor_count(const ojh_gguf *g) { return g ? (int)g->tensors.size() : 0; }

extern "C" const char *ojh_gguf_tensor_name(const ojh_gguf *g, int i) {
    return (g && i >= 0 && (size_t)i < g->tensors.size()) ? g->tensors[i].name.c_str() : nullptr;
}

extern "C" int ojh_gguf_tensor_meta(const ojh_gguf *g, const char *name, uint32_t *ggml_type, uint32_t *n_dims,
                                    uint64_t dims[4], uint64_t *file_offset, uint64_t *bytes) {
    const TensorInfo *t = find(g, name);
    if (!t) return ojh_fail(OJH_ERR_ARG, "tensor %s not found", name ? name : "(null)");
    uint64_t elems = 1;
    for (uint64_t d : t->dims) elems *= d;
    if (ggml_type) *ggml_type = t->type;
    if (n_dims) *n_dims = (uint32_t)t->dims.size();
    if (dims) for (size_t i = 0; i < 4; i++) dims[i] = i < t->dims.size() ? t->dims[i] : 1;
    if (file_offset) *file_offset = g->data_offset + t->rel_offset;
    if (bytes) *bytes = stored_bytes(t->type, elems);   // 0: a type without a fixed size this reader knows
    return OJH_OK;
}

extern "C" int ojh_gguf_meta_u64(const ojh_gguf *g, const char *key, uint64_t *out) {
    if (!g || !key || !out) return ojh_fail(OJH_ERR_ARG, "ojh_gguf_meta_u64: NULL argument");
    auto it = g->meta.find(key);
    if (it == g->meta.end()) return ojh_fail(OJH_ERR_ARG, "GGUF metadata key %s not found", key);
    const Meta &m = it->second;
    if (m.kind == 1 || m.kind == 4) *out = m.u;
    else if (m.kind == 2 && m.i >= 0) *out = (uint64_t)m.i;
    else return ojh_fail(OJH_ERR_ARG, "GGUF metadata key %s is not a nonnegative integer", key);
    return OJH_OK;
}

extern "C" int ojh_gguf_meta_str(const ojh_gguf *g, const char *key, char *out, size_t cap) {
    if (!g || !key || !out || !cap) return ojh_fail(OJH_ERR_ARG, "ojh_gguf_meta_str: NULL argument");
    auto it = g->meta.find(key);
    if (it == g->meta.end() || it->second.kind != 5) return ojh_fail(OJH_ERR_ARG, "GGUF metadata key %s is not a string", key);
    if (it->second.s.size() + 1 > cap) return ojh_fail(OJH_ERR_BOUNDS, "GGUF metadata string %s needs %zu bytes", key, it->second.s.size() + 1);
    memcpy(out, it->second.s.c_str(), it->second.s.size() + 1);
    return OJH_OK;
}

static int read_at(ojh_gguf *g, uint64_t off, void *dst, uint64_t n) {
    if (fseeko(g->fp, (off_t)off, SEEK_SET) || fread(dst, 1, n, g->fp) != n)
        return ojh_fail(OJH_ERR_ARG, "%s: short read of %llu bytes at %llu", g->path.c_str(), (unsigned long long)n,
                        (unsigned long long)off);
    return OJH_OK;
}

extern "C" int ojh_gguf_read_raw(ojh_gguf *g, const char *name, void *dst, uint64_t cap) {
    const TensorInfo *t = find(g, name);
    if (!t || !dst) return ojh_fail(OJH_ERR_ARG, "tensor %s not found", name ? name : "(null)");
    uint64_t elems = 1;
    for (uint64_t d : t->dims) elems *= d;
    uint64_t bytes = stored_bytes(t->type, elems);
    if (!bytes) return ojh_fail(OJH_ERR_UNSUPPORTED, "read_tensor_raw: unsupported GGUF type %u", t->type);
    if (bytes > cap) return ojh_fail(OJH_ERR_BOUNDS, "tensor %s needs %llu bytes, buffer has %llu", name, (unsigned long long)bytes,
                                     (unsigned long long)cap);
    return read_at(g, g->data_offset + t->rel_offset, dst, bytes);
}

// Lin::load: stack the named tensors along N, keep the file's block bytes.
extern "C" int ojh_lin_load(ojh_device *dev, ojh_gguf *g, const char *const *names, int count, ojh_lin **out) {
    if (!dev || !g || !names || !out || count < 1) return ojh_fail(OJH_ERR_ARG, "ojh_lin_load: NULL argument");
    *out = nullptr;
    uint64_t k0 = 0, n = 0, total = 0;
    uint32_t ty0 = 0;
    std::vector<const TensorInfo *> ts;
    for (int i = 0; i < count; i++) {
        const TensorInfo *t = find(g, names[i]);
        if (!t) return ojh_fail(OJH_ERR_ARG, "missing tensor %s", names[i] ? names[i] : "(null)");
        if (t->dims.size() > 2) return ojh_fail(OJH_ERR_UNSUPPORTED, "%s: a Lin takes 1-D or 2-D tensors, rank is %zu", t->name.c_str(), t->dims.size());
        uint64_t k = t->dims[0], rows = t->dims.size() > 1 ? t->dims[1] : 1;
        if (i && k != k0) return ojh_fail(OJH_ERR_ARG, "%s: K %llu differs from the fused group's", t->name.c_str(), (unsigned long long)k);
        if (i && t->type != ty0) return ojh_fail(OJH_ERR_ARG, "%s: type differs from the fused group's", t->name.c_str());
        k0 = k;
        ty0 = t->type;
        n += rows;
        total += stored_bytes(t->type, k * rows);
        ts.push_back(t);
    }
    const ojh_block_format *f = ojh_format(ty0);
    if (!f || k0 % f->weights)
        return ojh_fail(OJH_ERR_UNSUPPORTED, "GGUF type %u with K=%llu is not kept in place by this backend (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K .. Q6_K, IQ4_NL, IQ4_XS, the grid-codebook IQ types, with whole blocks)",
                        ty0, (unsigned long long)k0);
    if (n > 0xFFFFFFFFull || k0 > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_lin_load: tensor too large");
    ojh_buf *buf = nullptr;
    int rc = ojh_alloc(dev, total, &buf);
    if (rc) return rc;
    // file -> pinned staging -> device, in pieces
    const size_t chunk = 32u << 20;
    void *stage = nullptr;
    if (hipHostMalloc(&stage, chunk, hipHostMallocDefault) != hipSuccess) {
        ojh_free(dev, buf);
        return ojh_fail(OJH_ERR_HIP, "ojh_lin_load: cannot allocate the staging buffer");
    }
    uint64_t dst = 0;
    for (const TensorInfo *t : ts) {
        uint64_t bytes = stored_bytes(t->type, t->dims[0] * (t->dims.size() > 1 ? t->dims[1] : 1));
        uint64_t src = g->data_offset + t->rel_offset;
        for (uint64_t done = 0; done < bytes && !rc; done += chunk) {
            uint64_t piece = bytes - done < chunk ? bytes - done : chunk;
            if ((rc = read_at(g, src + done, stage, piece))) break;
            rc = ojh_upload(dev, buf, dst + done, stage, piece);
        }
        if (rc) break;
        dst += bytes;
    }
    (void)hipHostFree(stage);
    if (rc) {
        ojh_free(dev, buf);
        return rc;
    }
    ojh_lin *l = nullptr;
    if ((rc = ojh_lin_wrap(dev, ty0, (uint32_t)n, (uint32_t)k0, buf, 0, &l))) {
        ojh_free(dev, buf);
        return rc;
    }
    l->owns_raw = true;
    *out = l;
    return OJH_OK;
}

// Resident expert cache: a bounded device arena of fixed-size expert slots with least-recently-used
// eviction, for MoE layers whose experts do not all fit (or need not all sit) in device memory.  The
// behaviour of crates/ojas-cuda/src/expert_cache.rs:34-152 — `gather` makes every requested expert
// resident and returns one byte offset per request, which the `_slots` expert kernels take in place of an
// expert index — with the transfer shaped for this machine:
//   * misses go through two page-locked staging buffers in turn, each guarded by an event, so the caller's
//     `load` of the next expert (a pread from the model file) overlaps the previous expert's copy to the
//     device;
//   * the copies are queued on the device's compute stream: a kernel queued after `gather` sees them, and a
//     slot is overwritten only after the kernels queued before, which may still read it, have run.
// A cache created without a device keeps the books only (no arena, `load` never called): hit rates of a
// routing trace under a given budget, without touching a GPU.
#include <algorithm>
#include <unordered_map>

#include "ojh_internal.h"

struct ojh_expert_cache {
    ojh_device *dev = nullptr;   // NULL: bookkeeping only
    ojh_buf *arena = nullptr;
    void *staging[2] = {nullptr, nullptr};
    hipEvent_t staged[2] = {nullptr, nullptr};
    bool in_flight[2] = {false, false};
    int next_stage = 0;
    size_t expert_bytes = 0;
    uint32_t slots = 0;
    std::unordered_map<uint32_t, uint32_t> resident;   // expert id -> slot
    struct Slot { bool used = false; uint32_t id = 0; uint64_t tick = 0; };
    std::vector<Slot> slot_of;
    uint64_t tick = 0;
    ojh_gather_stats stats{};
};

extern "C" int ojh_expert_cache_create(ojh_device *dev, size_t budget_bytes, size_t expert_bytes,
                                       ojh_expert_cache **out) {
    if (!out) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_create: NULL output");
    *out = nullptr;
    if (!expert_bytes) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_create: expert_bytes must be non-zero");
    // the arena holds as many whole experts as the budget allows, and at least one; slots start on
    // 256-byte boundaries of the arena whenever an expert is a multiple of 256 bytes, as block tensors are
    size_t slots = std::max<size_t>(budget_bytes / expert_bytes, 1);
    if (slots > 0xFFFFFFFFull) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_create: %zu slots", slots);
    ojh_expert_cache *c = new ojh_expert_cache();
    c->dev = dev;
    c->expert_bytes = expert_bytes;
    c->slots = (uint32_t)slots;
    c->slot_of.resize(slots);
    c->resident.reserve(slots);
    if (dev) {
        int rc = ojh_alloc(dev, slots * expert_bytes, &c->arena);
        if (rc) { delete c; return rc; }
        for (int i = 0; i < 2; i++) {
            hipError_t e = hipHostMalloc(&c->staging[i], expert_bytes, hipHostMallocDefault);
            if (e == hipSuccess) e = hipEventCreateWithFlags(&c->staged[i], hipEventDisableTiming);
            if (e != hipSuccess) {
                ojh_expert_cache_destroy(c);
                return ojh_fail(OJH_ERR_HIP, "ojh_expert_cache_create: staging of %zu bytes: %s", expert_bytes,
                                hipGetErrorString(e));
            }
        }
    }
    *out = c;
    return OJH_OK;
}

extern "C" int ojh_expert_cache_destroy(ojh_expert_cache *c) {
    if (!c) return OJH_OK;
    for (int i = 0; i < 2; i++) {
        if (c->in_flight[i]) (void)hipEventSynchronize(c->staged[i]);
        if (c->staged[i]) (void)hipEventDestroy(c->staged[i]);
        if (c->staging[i]) (void)hipHostFree(c->staging[i]);
    }
    if (c->arena) ojh_free(c->dev, c->arena);
    delete c;
    return OJH_OK;
}

extern "C" uint32_t ojh_expert_cache_slots(const ojh_expert_cache *c) { return c ? c->slots : 0; }
extern "C" size_t ojh_expert_cache_resident_bytes(const ojh_expert_cache *c) {
    return c ? (size_t)c->slots * c->expert_bytes : 0;
}
extern "C" ojh_buf *ojh_expert_cache_arena(ojh_expert_cache *c) { return c ? c->arena : nullptr; }

extern "C" int ojh_expert_cache_stats(const ojh_expert_cache *c, ojh_gather_stats *out) {
    if (!c || !out) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_stats: NULL argument");
    *out = c->stats;
    return OJH_OK;
}

extern "C" int ojh_expert_cache_gather(ojh_expert_cache *c, const uint32_t *ids, size_t n, ojh_expert_load_fn load,
                                       void *user, uint64_t *offsets) {
    if (!c || (n && (!ids || !offsets))) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_gather: NULL argument");
    if (c->dev && c->dev->capturing) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_gather while recording a chain");
    if (c->dev && !load) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_gather: a cache with an arena needs a load callback");
    // more distinct experts than slots would evict an expert the same gather still needs: refuse
    std::vector<uint32_t> distinct(ids, ids + n);
    std::sort(distinct.begin(), distinct.end());
    distinct.erase(std::unique(distinct.begin(), distinct.end()), distinct.end());
    if (distinct.size() > c->slots)
        return ojh_fail(OJH_ERR_BOUNDS, "gather wants %zu distinct experts but the arena holds %u; raise the budget",
                        distinct.size(), c->slots);
    if (c->dev) OJH_HIP(hipSetDevice(c->dev->ordinal));
    for (size_t i = 0; i < n; i++) {
        const uint32_t id = ids[i];
        c->tick++;
        auto hit = c->resident.find(id);
        if (hit != c->resident.end()) {
            c->slot_of[hit->second].tick = c->tick;
            c->stats.hits++;
            offsets[i] = (uint64_t)hit->second * c->expert_bytes;
            continue;
        }
        // miss: the first free slot, else the least recently used one.  Every id of this call already seen
        // carries a newer tick than anything from earlier calls, and there are at most `slots` distinct
        // ids, so the victim is never one this call has handed out.
        uint32_t slot = c->slots;
        for (uint32_t s = 0; s < c->slots; s++)
            if (!c->slot_of[s].used) { slot = s; break; }
        if (slot == c->slots) {
            slot = 0;
            for (uint32_t s = 1; s < c->slots; s++)
                if (c->slot_of[s].tick < c->slot_of[slot].tick) slot = s;
            c->resident.erase(c->slot_of[slot].id);
            c->slot_of[slot].used = false;   // nothing lives here until the copy below is queued
            c->stats.evictions++;
        }
        if (c->dev) {
            const int st = c->next_stage;
            if (c->in_flight[st]) {
                OJH_HIP(hipEventSynchronize(c->staged[st]));
                c->in_flight[st] = false;
            }
            int rc = load(user, id, c->staging[st], c->expert_bytes);
            if (rc) return ojh_fail(OJH_ERR_ARG, "ojh_expert_cache_gather: load of expert %u returned %d", id, rc);
            OJH_HIP(hipMemcpyAsync((char *)c->arena->ptr + (size_t)slot * c->expert_bytes, c->staging[st], c->expert_bytes,
                                   hipMemcpyHostToDevice, c->dev->stream));
            OJH_HIP(hipEventRecord(c->staged[st], c->dev->stream));
            c->in_flight[st] = true;
            c->next_stage = st ^ 1;
        }
        c->resident[id] = slot;
        c->slot_of[slot].used = true;
        c->slot_of[slot].id = id;
        c->slot_of[slot].tick = c->tick;
        c->stats.misses++;
        c->stats.bytes_streamed += c->expert_bytes;
        offsets[i] = (uint64_t)slot * c->expert_bytes;
    }
    return OJH_OK;
}

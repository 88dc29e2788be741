"""Resident expert cache (`ExpertCache`, crates/ojas-cuda/src/expert_cache.rs:34-152): slot bookkeeping without
a GPU, and on the GPU the streamed expert FFN through the cache against the resident, index-addressed one."""
import numpy as np
import pytest

Q8_0 = 8


class _Lru:
    """The policy restated independently: first free slot, else the slot used longest ago."""

    def __init__(self, slots):
        self.slot_of, self.used, self.tick = {}, [None] * slots, 0
        self.hits = self.misses = self.evictions = 0

    def gather(self, ids):
        out = []
        for e in ids:
            self.tick += 1
            if e in self.slot_of:
                s = self.slot_of[e]
                self.hits += 1
            else:
                free = [i for i, u in enumerate(self.used) if u is None]
                if free:
                    s = free[0]
                else:
                    s = min(range(len(self.used)), key=lambda i: self.used[i][1])
                    del self.slot_of[self.used[s][0]]
                    self.evictions += 1
                self.slot_of[e] = s
                self.misses += 1
            self.used[s] = (e, self.tick)
            out.append(s)
        return out


def test_bookkeeping_without_a_device(pkg):
    eb = 1000
    c = pkg.ExpertCache(None, budget_bytes=5 * eb + 999, expert_bytes=eb)
    assert c.slots == 5 and c.resident_bytes == 5 * eb and c.arena is None
    model = _Lru(5)
    g = np.random.default_rng(7)
    for step in range(400):
        ids = g.choice(12, size=int(g.integers(1, 6)), replace=bool(step % 3 == 0)).astype(np.uint32)
        offs = c.gather(ids)
        assert offs.dtype == np.uint64 and list(offs) == [s * eb for s in model.gather(list(ids))], step
    st = c.stats
    assert (st["hits"], st["misses"], st["evictions"]) == (model.hits, model.misses, model.evictions)
    assert st["bytes_streamed"] == model.misses * eb and st["evictions"] > 0 and 0.0 < c.hit_rate < 1.0
    assert c.hit_rate == model.hits / (model.hits + model.misses)
    # a request repeated inside one call is one miss and then hits, in the order asked
    c2 = pkg.ExpertCache(None, 3 * eb, eb)
    assert list(c2.gather([4, 4, 9, 4])) == [0, 0, eb, 0] and c2.stats["misses"] == 2 and c2.stats["hits"] == 2
    # the least recently used expert goes first: touch 4 again, then two new ones evict 9 and then 7
    c2.gather([7])
    c2.gather([4])
    assert list(c2.gather([1])) == [eb] and list(c2.gather([2])) == [2 * eb] and c2.stats["evictions"] == 2
    assert list(c2.gather([4])) == [0] and c2.stats["misses"] == 5


def test_refusals_without_a_device(pkg):
    c = pkg.ExpertCache(None, 10, 1000)            # a budget below one expert still holds one
    assert c.slots == 1
    with pytest.raises(pkg.OjasHipError, match="2 distinct experts but the arena holds 1"):
        c.gather([3, 5])
    assert list(c.gather([3, 3, 3])) == [0, 0, 0]   # repeats of one expert fit
    assert c.stats["misses"] == 1 and c.stats["hits"] == 2
    with pytest.raises(pkg.OjasHipError, match="expert_bytes must be non-zero"):
        pkg.ExpertCache(None, 10, 0)
    assert list(c.gather([])) == []


@pytest.mark.gpu
def test_streamed_q80_experts_through_the_cache(gpu, pkg):
    """Experts kept as gate | up | down per slot, as the reference's streaming example lays them out
    (crates/ojas-cuda/examples/stream_moe.rs:60-160): tokens routed through gather + `moe_*_q80_slots` give the
    bits of the resident `moe_gu_q80` / `moe_down_q80` on the same experts, under eviction pressure; `load` runs
    once per miss; its failure and a wrong size surface as errors and leave the cache usable."""
    E, ksel, k, n = 12, 3, 256, 96
    gate = pkg.synth.q80_weights(E * n, k, "cache", "gate").reshape(E, -1)
    up = pkg.synth.q80_weights(E * n, k, "cache", "up").reshape(E, -1)
    down = pkg.synth.q80_weights(E * k, n, "cache", "down").reshape(E, -1)
    gu_bytes, down_bytes = gate.shape[1], down.shape[1]
    eb = 2 * gu_bytes + down_bytes
    experts = np.concatenate([gate, up, down], axis=1)
    cache = pkg.ExpertCache(gpu, budget_bytes=5 * eb, expert_bytes=eb)
    assert cache.slots == 5 and cache.arena.nbytes == 5 * eb
    loads = []

    def load(e):
        loads.append(e)
        return experts[e]

    gpu.ensure_family("moe")
    gd, ud, dd = gpu.upload_bytes(gate), gpu.upload_bytes(up), gpu.upload_bytes(down)
    g = pkg.synth.rng("cache", "route")
    model = _Lru(5)
    for step in range(24):
        idx = g.permutation(E)[:ksel].astype(np.uint32)
        wgt = g.random(ksel).astype(np.float32)
        x = pkg.synth.normal_f32(k, "cache", "x", step)
        xd, idxd, wgtd = gpu.upload(x), gpu.upload_bytes(idx), gpu.upload(wgt)
        act1, y1 = gpu.alloc(ksel * n), gpu.upload(np.zeros(k, np.float32))
        gpu.dispatch(gpu.begin(), "moe_gu_q80", [(xd, 0), (gd, 0), (ud, 0), (act1, 0), (idxd, 0)], [k, n], [-(-n // 8), ksel, 1], [256, 1, 1])
        gpu.dispatch(gpu.begin(), "moe_down_q80", [(act1, 0), (dd, 0), (y1, 0), (idxd, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 16), 1, 1], [256, 1, 1])
        before = len(loads)
        offs = cache.gather(idx, load)
        assert list(offs) == [s_ * eb for s_ in model.gather([int(v) for v in idx])]
        assert len(loads) - before == len(set(loads[before:])) <= ksel
        tbl = lambda extra: gpu.upload_bytes((offs + extra).astype(np.uint32))
        og, ou, od = tbl(0), tbl(gu_bytes), tbl(2 * gu_bytes)
        act2, y2 = gpu.alloc(ksel * n), gpu.upload(np.zeros(k, np.float32))
        A = cache.arena
        gpu.dispatch(gpu.begin(), "moe_gu_q80_slots", [(xd, 0), (A, 0), (A, 0), (act2, 0), (og, 0), (ou, 0)], [k, n], [-(-n // 8), ksel, 1], [256, 1, 1])
        gpu.dispatch(gpu.begin(), "moe_down_q80_slots", [(act2, 0), (A, 0), (y2, 0), (od, 0), (wgtd, 0)], [n, k, ksel], [-(-k // 8), 1, 1], [256, 1, 1])
        assert np.array_equal(gpu.read(y1, k), gpu.read(y2, k)), step
    st = cache.stats
    assert st["misses"] == len(loads) and st["hits"] + st["misses"] == 24 * ksel and st["evictions"] == st["misses"] - 5
    assert st["bytes_streamed"] == st["misses"] * eb and st["hits"] > 0
    assert (st["hits"], st["misses"], st["evictions"]) == (model.hits, model.misses, model.evictions)
    # what the arena holds is what was loaded, slot by slot
    held = gpu.read(cache.arena, 5 * eb, np.uint8).reshape(5, eb)
    for e, s_ in model.slot_of.items():
        assert np.array_equal(held[s_], experts[e]), (e, s_)
    # failures of the callback surface as errors and leave the cache usable
    missing = next(e for e in range(E) if e not in model.slot_of)

    def bad(e):
        raise OSError("disk gone")

    with pytest.raises(OSError, match="disk gone"):
        cache.gather([missing], bad)
    with pytest.raises(ValueError, match="the slot holds"):
        cache.gather([missing], lambda e: experts[e][:-1])
    off = cache.gather([missing], load)
    assert np.array_equal(gpu.read(cache.arena, eb, np.uint8, off=int(off[0])), experts[missing])
    cache.close()

"""Expert-slot cache on the GPU: LRU semantics against a direct model of the reference rule
(src/expert_cache.cuh:2252-2326, :2467-2493), device slot table contents, bytes in the slots, and a
layer pass through the slot table that is bit-identical to the all-resident pass."""
import ctypes as C
import json

import numpy as np
import pytest

from warpdecode_amd import capi, synth

pytestmark = pytest.mark.gpu
SEED = 20261014


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.init()
    return gpu_util


class ModelCache:
    """The reference rule, written the slow way: first empty slot, else smallest last_use."""

    def __init__(self, n_slots, n_layers=1, partition=False):
        self.slots = [None] * n_slots          # (key, last_use)
        self.clock = 0
        self.n_layers, self.partition = n_layers, partition and n_layers <= n_slots
        self.hits = self.misses = self.evictions = 0

    def bounds(self, layer):
        n = len(self.slots)
        if not self.partition:
            return 0, n
        per, rem = divmod(n, self.n_layers)
        b = layer * per + min(layer, rem)
        return b, b + per + (1 if layer < rem else 0)

    def acquire(self, layer, expert):
        key = (layer, expert)
        self.clock += 1
        for i, s in enumerate(self.slots):
            if s is not None and s[0] == key:
                self.slots[i] = (key, self.clock)
                self.hits += 1
                return i, True
        self.misses += 1
        b, e = self.bounds(layer)
        empty = [i for i in range(b, e) if self.slots[i] is None]
        if empty:
            i = empty[0]
        else:
            i = min(range(b, e), key=lambda q: self.slots[q][1])
            self.evictions += 1
        self.slots[i] = (key, self.clock)
        return i, False


def _host_layers(n_layers, E, gb, ub, db, seed):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n_layers):
        out.append([rng.integers(0, 256, E * gb, dtype=np.uint8), rng.integers(0, 256, E * ub, dtype=np.uint8),
                    rng.integers(0, 256, E * db, dtype=np.uint8)])
    return out


@pytest.mark.parametrize("partition", [0, 1])
def test_lru_semantics_and_contents(g, partition):
    n_layers, E, k = 3, 24, 4
    gb, ub, db = 256, 128, 64
    n_slots = 17
    host = _host_layers(n_layers, E, gb, ub, db, SEED)
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), n_slots * (gb + ub + db) + 5, gb, ub, db, n_layers, E, partition)
    for l in range(n_layers):
        capi.call("wd_expert_cache_register_layer", cache, l, *[h.ctypes.data_as(C.c_void_p) for h in host[l]])
    model = ModelCache(n_slots, n_layers, bool(partition))
    rng = np.random.default_rng(SEED + 1)
    lib = capi.load()
    pool = lib.wd_expert_cache_pool(cache)
    for step in range(60):
        layer = int(rng.integers(0, n_layers))
        ids = rng.choice(E, size=k, replace=False, p=(lambda p: p / p.sum())(1.0 / np.arange(1, E + 1) ** 1.1)).astype(np.int32)
        hits = np.zeros(k, np.uint8)
        capi.call("wd_expert_cache_acquire", cache, layer, ids.ctypes.data_as(C.c_void_p), k,
                  hits.ctypes.data_as(C.c_void_p), g.stream())
        want = [model.acquire(layer, int(e)) for e in ids]
        assert [bool(h) for h in hits] == [w[1] for w in want]
        g.sync()
        table = g.view(lib.wd_expert_cache_slot_table(cache, layer), E, np.int32)
        for e, (slot, _) in zip(ids, want):
            assert table[e] == slot
            got = g.view(pool + slot * (gb + ub + db), gb + ub + db, np.uint8)
            assert np.array_equal(got[:gb], host[layer][0][e * gb:(e + 1) * gb])
            assert np.array_equal(got[gb:gb + ub], host[layer][1][e * ub:(e + 1) * ub])
            assert np.array_equal(got[gb + ub:], host[layer][2][e * db:(e + 1) * db])
        # every table entry agrees with the model, evicted experts read -1
        for l in range(n_layers):
            t = g.view(lib.wd_expert_cache_slot_table(cache, l), E, np.int32)
            resident = {s[0][1]: i for i, s in enumerate(model.slots) if s is not None and s[0][0] == l}
            for e in range(E):
                assert t[e] == resident.get(e, -1)
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    assert (st.hits, st.misses, st.evictions) == (model.hits, model.misses, model.evictions)
    assert st.accesses == 60 * k and st.bytes_copied == model.misses * (gb + ub + db)
    assert st.slots == n_slots and st.resident == sum(s is not None for s in model.slots)
    capi.call("wd_expert_cache_destroy", cache)


@pytest.mark.parametrize("copy_kernel", [1, 0])
def test_host_copy_packed_per_expert(g, copy_kernel):
    """A host copy that holds each expert's gate, up and down bytes back to back (one record per expert, the three
    strides all one record) is filled as one piece; the slots must read as they do from three separate tensors."""
    import torch
    n_layers, E, k = 2, 12, 3
    gb, ub, db = 512, 256, 1024
    rec = gb + ub + db
    n_slots = 7
    host = _host_layers(n_layers, E, gb, ub, db, SEED + 21)
    packed = []
    for l in range(n_layers):
        p = np.concatenate([host[l][0].reshape(E, gb), host[l][1].reshape(E, ub), host[l][2].reshape(E, db)], axis=1)
        packed.append(torch.from_numpy(np.ascontiguousarray(p).reshape(-1)).pin_memory())
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), n_slots * rec, gb, ub, db, n_layers, E, 0)
    capi.call("wd_expert_cache_set_copy_kernel", cache, copy_kernel)
    for l in range(n_layers):
        base = packed[l].data_ptr()
        capi.call("wd_expert_cache_register_layer_strided", cache, l, C.c_void_p(base), C.c_void_p(base + gb),
                  C.c_void_p(base + gb + ub), rec, rec, rec)
    model = ModelCache(n_slots, n_layers, False)
    rng = np.random.default_rng(SEED + 22)
    lib = capi.load()
    pool = lib.wd_expert_cache_pool(cache)
    for step in range(30):
        layer = int(rng.integers(0, n_layers))
        ids = rng.choice(E, size=k, replace=False).astype(np.int32)
        capi.call("wd_expert_cache_acquire", cache, layer, ids.ctypes.data_as(C.c_void_p), k, None, g.stream())
        want = [model.acquire(layer, int(e)) for e in ids]
        g.sync()
        table = g.view(lib.wd_expert_cache_slot_table(cache, layer), E, np.int32)
        for e, (slot, _) in zip(ids, want):
            assert table[e] == slot
            got = g.view(pool + slot * rec, rec, np.uint8)
            assert np.array_equal(got[:gb], host[layer][0][e * gb:(e + 1) * gb])
            assert np.array_equal(got[gb:gb + ub], host[layer][1][e * ub:(e + 1) * ub])
            assert np.array_equal(got[gb + ub:], host[layer][2][e * db:(e + 1) * db])
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    assert (st.hits, st.misses) == (model.hits, model.misses) and st.bytes_copied == model.misses * rec
    need = lib.wd_expert_cache_dump_json(cache, None, 0)
    buf = C.create_string_buffer(need + 1)
    lib.wd_expert_cache_dump_json(cache, buf, need + 1)
    d = json.loads(buf.value.decode())
    by = ("fills_by_copy_kernel", "fills_by_memcpy")
    assert d[by[1 - copy_kernel]] == model.misses and d[by[copy_kernel]] == 0
    capi.call("wd_expert_cache_destroy", cache)


def test_cache_errors(g):
    cache = C.c_void_p()
    lib = capi.load()
    assert lib.wd_expert_cache_create(C.byref(cache), 100, 256, 128, 64, 1, 8, 0) == -1      # smaller than one slot
    assert lib.wd_expert_cache_create(C.byref(cache), 0, 256, 128, 64, 1, 8, 0) == -1
    capi.call("wd_expert_cache_create", C.byref(cache), 3 * 448, 256, 128, 64, 1, 8, 0)
    ids = np.arange(4, dtype=np.int32)
    assert lib.wd_expert_cache_acquire(cache, 0, ids.ctypes.data_as(C.c_void_p), 4, None, None) == -1   # unregistered
    h = [np.zeros(8 * b, np.uint8) for b in (256, 128, 64)]
    capi.call("wd_expert_cache_register_layer", cache, 0, *[x.ctypes.data_as(C.c_void_p) for x in h])
    assert lib.wd_expert_cache_acquire(cache, 0, ids.ctypes.data_as(C.c_void_p), 4, None, None) == -1   # 3 slots < k
    bad = np.array([0, 9], np.int32)
    assert lib.wd_expert_cache_acquire(cache, 0, bad.ctypes.data_as(C.c_void_p), 2, None, None) == -1   # id range
    capi.call("wd_expert_cache_destroy", cache)


def test_state_after_a_failing_acquire(g, tmp_path):
    """A call that fails part-way (the file behind the experts has lost its tail, so the read of one expert comes up
    short) must leave the host's index, the device's slot table and the pool agreeing with each other: the experts
    acquired before the failure are resident with their bytes in place, the failing one and those after it are not.
    An id out of range is refused before anything changes.  Every failure here is a host-side error return."""
    import mmap
    import os
    E, gb, ub, db = 8, 4096, 4096, 2048
    slot = gb + ub + db
    rng = np.random.default_rng(SEED + 17)
    data = rng.integers(0, 256, E * slot, dtype=np.uint8)
    path = tmp_path / "experts.bin"
    data.tofile(path)
    fd = os.open(path, os.O_RDWR)
    mm = mmap.mmap(fd, E * slot)
    base = np.frombuffer(mm, dtype=np.uint8).ctypes.data
    lib = capi.load()
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), 5 * slot, gb, ub, db, 1, E, 0)
    capi.call("wd_expert_cache_register_layer", cache, 0, C.c_void_p(base), C.c_void_p(base + E * gb), C.c_void_p(base + E * (gb + ub)))
    capi.call("wd_expert_cache_attach_file", cache, C.c_void_p(base), E * slot, fd, 2)
    os.ftruncate(fd, E * slot - db // 2)        # the last expert's down slice is no longer whole

    def acquire(ids):
        a = np.asarray(ids, np.int32)
        hit = np.zeros(len(a), np.uint8)
        rc = lib.wd_expert_cache_acquire(cache, 0, a.ctypes.data_as(C.c_void_p), len(a), hit.ctypes.data_as(C.c_void_p), g.stream())
        g.sync()
        return rc, hit

    def expert_bytes(e):
        return np.concatenate([data[e * gb:(e + 1) * gb], data[E * gb + e * ub:E * gb + (e + 1) * ub],
                               data[E * (gb + ub) + e * db:E * (gb + ub) + (e + 1) * db]])

    def check_state(resident):
        table = g.view(lib.wd_expert_cache_slot_table(cache, 0), E, np.int32)
        pool = g.view(lib.wd_expert_cache_pool(cache), 5 * slot, np.uint8)
        for e in range(E):
            s_host = lib.wd_expert_cache_slot_of(cache, 0, e)
            assert s_host == table[e], (e, s_host, table[e])
            assert (s_host >= 0) == (e in resident), (e, s_host)
            if s_host >= 0:
                assert np.array_equal(pool[s_host * slot:(s_host + 1) * slot], expert_bytes(e)), e
        st = capi.CacheStats()
        capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
        assert st.resident == len(resident)

    rc, _ = acquire([0, 9, 1])                    # an id out of range: nothing changes
    assert rc == -1
    check_state(set())
    rc, hit = acquire([0, 1, 7, 2])               # 0 and 1 are filled, 7 cannot be read, 2 is never reached
    assert rc < 0 and "pread" in lib.wd_last_error().decode()
    check_state({0, 1})
    rc, hit = acquire([1, 0, 2])
    assert rc == 0 and hit.tolist() == [1, 1, 0]
    check_state({0, 1, 2})
    rc, hit = acquire([3, 4, 5])                  # recycles slots: the one given back by the failed fill among them
    assert rc == 0 and hit.tolist() == [0, 0, 0]
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    assert st.evictions == 1
    check_state({0, 2, 3, 4, 5} if lib.wd_expert_cache_slot_of(cache, 0, 1) < 0 else {1, 2, 3, 4, 5})
    capi.call("wd_expert_cache_destroy", cache)
    del base
    os.close(fd)


def test_layer_through_slot_table(g, oracle):
    """A C2-shaped layer (fewer experts) whose routed tensors live only in the slot pool."""
    L = synth.make_c2(n_experts=64)
    H, F, E, k = 2048, 512, 64, 10
    gb = F * synth.row_bytes(synth.IQ3_S, H)
    db = H * synth.row_bytes(synth.Q8_0, F)
    import torch
    pinned = [torch.from_numpy(np.ascontiguousarray(L[n]).reshape(-1)).pin_memory() for n in ("gate", "up", "down")]
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), 24 * (2 * gb + db), gb, gb, db, 1, E, 0)
    capi.call("wd_expert_cache_register_layer", cache, 0, *[C.c_void_p(t.data_ptr()) for t in pinned])
    lib = capi.load()
    dl = g.DeviceLayer(L)
    d = dl.desc
    d.gate = d.up = d.down = None
    d.slot_of_expert = lib.wd_expert_cache_slot_table(cache, 0)
    d.slot_pool = lib.wd_expert_cache_pool(cache)
    d.slot_bytes, d.slot_gate_bytes, d.slot_up_bytes = 2 * gb + db, gb, gb
    sc = g.Scratch(H, F, E, k)
    rng = np.random.default_rng(SEED + 5)
    for step in range(6):
        x = synth.rms_normed(synth.rng_for(SEED, 61, step), H)
        ids = rng.choice(E, size=k, replace=False).astype(np.int32)
        wts = rng.uniform(0.05, 0.15, k).astype(np.float32)
        capi.call("wd_expert_cache_acquire", cache, 0, ids.ctypes.data_as(C.c_void_p), k, None, g.stream())
        capi.call("wd_memcpy_h2d", C.c_void_p(sc.raw("ids")), ids.ctypes.data_as(C.c_void_p), 4 * k, g.stream())
        capi.call("wd_memcpy_h2d", C.c_void_p(sc.raw("weights")), wts.ctypes.data_as(C.c_void_p), 4 * k, g.stream())
        dx, out = g.dev(x), g.empty(H, np.float32)
        for flags in (capi.MOE_PRESELECTED, capi.MOE_PRESELECTED | capi.MOE_STAGED):
            capi.call("wd_moe_layer_f32", C.byref(d), g.ptr(dx), g.ptr(out), sc.h, flags, g.stream())
            g.sync()
            want, _ = oracle.moe_layer(L, x, ids=ids, weights=wts)
            assert g.same_bits(g.host(out), want), (step, flags)
    st = capi.CacheStats()
    capi.call("wd_expert_cache_get_stats", cache, C.byref(st))
    assert st.misses > 24 and st.evictions > 0 and st.hits > 0
    # The router's own selection over a pool that holds 24 of the 64 experts: the kernels meet negative entries of the
    # slot table.  They read slot 0 instead (memory that exists), report it through the status word, and the fused
    # combine hands NaN to the caller.
    table = g.view(lib.wd_expert_cache_slot_table(cache, 0), E, np.int32)
    x = synth.rms_normed(synth.rng_for(SEED, 61, 99), H)
    _, dump = oracle.moe_layer(L, x)
    assert any(table[e] < 0 for e in dump["ids"]), "the selection should include an expert without a slot"
    dx, out = g.dev(x), g.empty(H, np.float32)
    for flags in (0, capi.MOE_SPLIT_AB, capi.MOE_STAGED):
        capi.call("wd_moe_layer_f32", C.byref(d), g.ptr(dx), g.ptr(out), sc.h, flags, g.stream())
        g.sync()
        assert lib.wd_moe_scratch_status(sc.h) == 2, flags
        if flags != capi.MOE_STAGED:
            assert np.isnan(g.host(out)).all(), flags
        capi.call("wd_moe_scratch_set_wait_limit", sc.h, 0)
        assert lib.wd_moe_scratch_status(sc.h) == 0
    sc.close()
    capi.call("wd_expert_cache_destroy", cache)


def test_monitor_and_shadow_caches(g):
    """Counters and counterfactual caches against a direct model: an LRU shadow with the pool's own capacity must
    hit exactly as often as the pool, a larger one at least as often, and the JSON dump must carry the counters."""
    E, NL, k = 16, 2, 4
    gb, ub, db = 256, 256, 512
    slots = 6
    host = _host_layers(NL, E, gb, ub, db, SEED + 9)
    cache = C.c_void_p()
    capi.call("wd_expert_cache_create", C.byref(cache), slots * (gb + ub + db), gb, ub, db, NL, E, 0)
    capi.call("wd_expert_cache_add_shadow", cache, 0, slots)
    capi.call("wd_expert_cache_add_shadow", cache, 0, 3 * slots)
    capi.call("wd_expert_cache_add_shadow", cache, 1, slots)
    capi.call("wd_expert_cache_set_timing", cache, 1)
    import torch
    pinned = [[torch.from_numpy(a).pin_memory() for a in layer] for layer in host]
    for l in range(NL):
        capi.call("wd_expert_cache_register_layer", cache, l, *[C.c_void_p(t.data_ptr()) for t in pinned[l]])
    rng = np.random.default_rng(SEED + 10)
    model = ModelCache(slots, NL, False)
    big = ModelCache(3 * slots, NL, False)
    accesses = 0
    for step in range(40):
        for l in range(NL):
            ids = rng.choice(E, size=k, replace=False, p=np.arange(E, 0, -1) / np.arange(E, 0, -1).sum()).astype(np.int32)
            capi.call("wd_expert_cache_acquire", cache, l, ids.ctypes.data_as(C.c_void_p), k, None, g.stream())
            for e in ids:
                model.acquire(l, int(e)); big.acquire(l, int(e))
            accesses += k
    g.sync()
    lib = capi.load()
    need = lib.wd_expert_cache_dump_json(cache, None, 0)
    buf = C.create_string_buffer(need + 1)
    lib.wd_expert_cache_dump_json(cache, buf, need + 1)
    d = json.loads(buf.value.decode())
    assert d["accesses"] == accesses and d["hits"] == model.hits and d["misses"] == model.misses
    assert d["evictions"] == model.evictions and d["bytes_copied"] == model.misses * (gb + ub + db)
    assert sum(d["layer_access"]) == accesses and sum(d["layer_misses"]) == model.misses
    assert d["shadows"][0] == dict(policy="lru", slots=slots, hits=model.hits, hit_rate=round(model.hits / accesses, 4))
    assert d["shadows"][1]["hits"] == big.hits >= model.hits
    assert d["shadows"][2]["policy"] == "lfu" and 0 < d["shadows"][2]["hits"] <= accesses
    assert d["distinct_pairs"] <= NL * E and 0.0 < d["prev_token_reuse"] < 1.0
    # the timings: one timed interval per acquire call that missed (every slot's events had passed before the dump), the
    # copy stream's waits and fills of a few 1 KB experts take microseconds each; 40 passes over 2 layers, all gaps between
    # two calls are between different layers here
    missed_calls = d["io_dma_calls"]
    assert d["io_timing"] is True and 0 < missed_calls <= 40 * NL and d["io_dma_stall_calls"] == missed_calls
    assert d["io_timing_skipped"] + missed_calls >= 1
    assert 0.0 < d["io_dma_max_ms"] < 50.0 and d["io_dma_ms"] <= missed_calls * d["io_dma_max_ms"] + 0.1
    assert 0.0 <= d["io_dma_stall_max_ms"] < 50.0
    assert d["tokens"] == 40 and d["intra_gap_ms"] == 0.0 and d["layer_gap_ms"] > 0.0
    assert abs(d["layer_gap_per_token"] - d["layer_gap_ms"] / 40) < 0.011 and d["acquire_per_token"] > 0.0
    capi.call("wd_expert_cache_destroy", cache)

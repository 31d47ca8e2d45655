"""GPU parity tests of the streaming insert path (ash_map_insert_bulk): forced
on for every batch that it accepts, it must leave the same map as the oracle and
as the per-key kernel -- same key set, masks, sizes, heap protocol, and each
stored key carrying the value rows of ONE of its source rows."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_is_bijection_into, sort_rows
from test_gpu_hash import _assert_same_map, _oracle_map

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture()
def bulk_ash(gpu_ash, monkeypatch):
    monkeypatch.setattr(gpu_ash.common, "BULK_INSERT", "always")
    return gpu_ash


def _random_keys(rng, n, dim, span):
    return torch.from_numpy(rng.integers(-span, span, size=(n, dim)).astype(np.int32))


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_bulk_keys_with_duplicates_match_oracle(bulk_ash, oracle, dim):
    capacity = 150_000
    rng = np.random.default_rng(900 + dim)
    span = {1: 60_000, 2: 170, 3: 25, 4: 10}[dim]
    keys = _random_keys(rng, 300_000, dim, span)
    engine = bulk_ash.ASHEngine(dim, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    engine.backend.insert_keys(keys.to(DEV))
    omap.insert_keys(keys)
    probe = _random_keys(rng, 50_000, dim, span + 2)
    _assert_same_map(engine, omap, probe.to(DEV))
    # indices of a fresh map are exactly 0 .. size-1 (heap[counter++])
    _, idx = engine.items()
    assert torch.equal(torch.sort(idx).values.cpu(), torch.arange(engine.size()))
    assert engine.backend.status()["dropped"] == 0


def test_bulk_into_a_populated_table_with_erases(bulk_ash, oracle):
    """Second and third bulk batches meet live entries, tombstones and recycled
    heap entries."""
    dim, capacity = 3, 400_000
    rng = np.random.default_rng(910)
    engine = bulk_ash.ASHEngine(dim, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    first = _random_keys(rng, 250_000, dim, 40)
    engine.backend.insert_keys(first.to(DEV))
    omap.insert_keys(first)
    gone = first[rng.permutation(len(first))[:90_000]]
    engine.erase(gone.to(DEV))
    omap.erase(gone)
    second = torch.cat([_random_keys(rng, 200_000, dim, 45), gone[:20_000]])
    engine.backend.insert_keys(second.to(DEV))
    omap.insert_keys(second)
    probe = _random_keys(rng, 100_000, dim, 47)
    _assert_same_map(engine, omap, probe.to(DEV))
    # a small per-key batch and another bulk batch on top
    third = _random_keys(rng, 3_000, dim, 46)
    engine.backend.insert_keys(third.to(DEV))
    omap.insert_keys(third)
    fourth = _random_keys(rng, 150_000, dim, 46)
    engine.backend.insert_keys(fourth.to(DEV))
    omap.insert_keys(fourth)
    _assert_same_map(engine, omap, probe.to(DEV))


@pytest.mark.parametrize("capacity", [1_000, 200_000])
def test_bulk_values_come_from_one_source_row(bulk_ash, capacity):
    dim = 3
    rng = np.random.default_rng(920)
    n = 180_000
    span = 4 if capacity == 1_000 else 30
    keys = _random_keys(rng, n, dim, span).to(DEV)
    row = torch.arange(n, device=DEV, dtype=torch.float32)
    values = {
        "color": torch.stack([row, row + 0.5, 2 * row], dim=1),
        "depth": row.view(-1, 1).clone(),
    }
    hm = bulk_ash.HashMap(dim, {"color": 3, "depth": 1}, capacity, DEV)
    hm.insert(keys, values)
    uniq = torch.unique(keys, dim=0)
    assert hm.size() == len(uniq)
    idx, masks = hm.engine.find(uniq)
    assert bool(masks.all())
    assert_is_bijection_into(idx, capacity)
    color, depth = hm.color[idx], hm.depth[idx]
    src = depth[:, 0].long()
    assert bool((src >= 0).all()) and bool((src < n).all())
    # both rows come from the same source row, and that row holds this key
    assert torch.equal(color, values["color"][src])
    assert torch.equal(keys[src], uniq)


def test_bulk_piles_of_duplicates_and_unpackable_keys(bulk_ash, oracle):
    """Every key far beyond its partition's capacity (spill lists) plus keys
    that do not fit the packed code (second region)."""
    dim, capacity = 3, 50_000
    rng = np.random.default_rng(930)
    few = _random_keys(rng, 40, dim, 1000)
    piles = few[rng.integers(0, 40, size=120_000)]
    spread = _random_keys(rng, 60_000, dim, 18)
    big = torch.from_numpy(
        rng.integers(-(2**31), 2**31 - 1, size=(4_000, dim)).astype(np.int32))
    keys = torch.cat([piles, spread, big, big[:500]])
    keys = keys[torch.from_numpy(rng.permutation(len(keys)))]
    engine = bulk_ash.ASHEngine(dim, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    stores = {"v": torch.zeros(capacity, dim, dtype=torch.int32, device=DEV)}
    engine.insert(keys.to(DEV), {"v": keys.to(DEV)}, stores)
    omap.insert_keys(keys)
    probe = torch.cat([keys[:50_000], keys[:20_000] + 1])
    _assert_same_map(engine, omap, probe.to(DEV))
    idx, mask = engine.find(keys.to(DEV))
    assert bool(mask.all()) and torch.equal(stores["v"][idx].cpu(), keys)


def test_bulk_overflow_drops_and_stays_usable(bulk_ash):
    capacity = 30_000
    engine = bulk_ash.ASHEngine(3, capacity, DEV)
    g = torch.Generator().manual_seed(940)
    keys = torch.arange(45_000, dtype=torch.int32).view(-1, 1).tile((1, 3))
    keys = keys[torch.randperm(len(keys), generator=g)].to(DEV)
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        engine.insert_keys(keys)
    assert engine.size() == capacity
    idx, mask = engine.find(keys)
    assert int(mask.sum()) == capacity
    assert_is_bijection_into(idx[mask], capacity)
    assert engine.backend.status()["dropped"] == 15_000
    engine.erase(keys[mask][:9_000])
    engine.insert_keys(keys[~mask][:9_000])
    assert engine.size() == capacity
    assert bool(engine.find(keys[~mask][:9_000])[1].all())


def test_bulk_equals_per_key_kernel(gpu_ash, monkeypatch):
    """The two insert paths on the same input: same key set, same size, and
    finds agree key by key (indices are free)."""
    dim, capacity = 3, 1_500_000
    rng = np.random.default_rng(950)
    keys = _random_keys(rng, 1_200_000, dim, 70).to(DEV)
    probe = _random_keys(rng, 300_000, dim, 72).to(DEV)
    maps = {}
    for policy in ("always", "never"):
        monkeypatch.setattr(gpu_ash.common, "BULK_INSERT", policy)
        engine = gpu_ash.ASHEngine(dim, capacity, DEV)
        engine.backend.insert_keys(keys)
        maps[policy] = engine
    a, b = maps["always"], maps["never"]
    assert a.size() == b.size() == len(torch.unique(keys, dim=0))
    assert torch.equal(sort_rows(a.items()[0])[0], sort_rows(b.items()[0])[0])
    (ia, ma), (ib, mb) = a.find(probe), b.find(probe)
    assert torch.equal(ma, mb)
    assert_is_bijection_into(a.items()[1], capacity)


@pytest.mark.parametrize("policy", ["always", "never"])
def test_clear_leaves_the_fill_to_the_next_call(gpu_ash, monkeypatch, policy):
    """clear() resets counters and heap at once and leaves the fill of the
    bucket array to the next call on the table; a streaming insert rewrites
    every bucket instead.  Whatever comes first after a clear -- find, items,
    erase, size, a per-key or a streaming insert (also one that reaches only a
    few partitions) -- sees an empty table, and nothing of the old keys comes
    back later."""
    monkeypatch.setattr(gpu_ash.common, "BULK_INSERT", policy)
    rng = np.random.default_rng(61)
    old = torch.unique(_random_keys(rng, 60_000, 3, 300), dim=0).to(DEV)
    new = torch.unique(_random_keys(rng, 50_000, 3, 300), dim=0).to(DEV)
    few = new[:3000].contiguous()

    def fresh():
        hm = gpu_ash.HashMap(3, 2, 2_000_000, DEV)
        hm.insert(old, torch.ones(len(old), 2, device=DEV))
        assert hm.size() == len(old)
        hm.clear()
        return hm

    hm = fresh()
    assert hm.size() == 0
    masks, _ = hm.find(old)
    assert not bool(masks.any())
    hm = fresh()
    keys, idx = hm.items()
    assert len(keys) == 0 and len(idx) == 0
    hm = fresh()
    hm.erase(old[:100])
    assert hm.size() == 0
    for batch in (new, few):
        hm = fresh()
        values = torch.arange(len(batch), device=DEV, dtype=torch.float32).view(-1, 1).repeat(1, 2)
        hm.insert(batch, values)
        assert hm.size() == len(batch)
        masks, idx, got = hm.find(batch, return_values=True)
        assert bool(masks.all()) and torch.equal(got, values)
        assert_is_bijection_into(idx.cpu(), 2_000_000)
        keys, _ = hm.items()
        assert torch.equal(sort_rows(keys)[0], sort_rows(batch)[0])
    # a streaming insert that leaves many partitions of a large table without a
    # record: those are written as empty ones, or old keys would reappear
    big = gpu_ash.HashMap(3, 2, 20_000_000, DEV)
    spread = torch.unique(_random_keys(rng, 400_000, 3, 2000), dim=0).to(DEV)
    big.insert(spread, torch.ones(len(spread), 2, device=DEV))
    big.clear()
    sparse_batch = torch.unique(_random_keys(rng, 20_000, 3, 2000), dim=0).to(DEV)
    if policy == "always":
        # (the streaming path applies to this batch)
        rows, nbytes = (ctypes.c_int64 * 1)(8), ctypes.c_int64(0)
        backend = big.engine.backend
        assert backend._lib.ash_map_insert_scratch_bytes(
            backend._handle, len(sparse_batch), 1, rows, 1, ctypes.byref(nbytes)) == 0
        assert nbytes.value > len(sparse_batch) * 20
    big.insert(sparse_batch, torch.zeros(len(sparse_batch), 2, device=DEV))
    keys, _ = big.items()
    assert torch.equal(sort_rows(keys)[0], sort_rows(sparse_batch)[0])
    masks, _ = big.find(spread)
    assert int(masks.sum()) <= len(sparse_batch)   # only keys that are in both sets
    del big
    # twice in a row, and a clear right after a clear
    hm = fresh()
    hm.clear()
    hm.insert(few, torch.zeros(len(few), 2, device=DEV))
    hm.clear()
    hm.insert(new, torch.zeros(len(new), 2, device=DEV))
    keys, _ = hm.items()
    assert torch.equal(sort_rows(keys)[0], sort_rows(new)[0])


def test_pending_fill_is_refused_under_capture(gpu_ash):
    """A look-up recorded into a HIP graph right after a clear would record the
    pending fill with it and empty the table at every replay: the call fails
    instead, and works once the fill has run outside the capture."""
    engine = gpu_ash.ASHEngine(3, 5000, DEV)
    keys = torch.randint(-50, 50, (3000, 3), dtype=torch.int32, device=DEV)
    engine.insert_keys(keys)
    engine.clear()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with pytest.raises(RuntimeError, match="cleared"):
            with torch.cuda.graph(graph, stream=side):
                engine.find(keys)
    torch.cuda.synchronize()
    _, masks = engine.find(keys)
    assert not bool(masks.any())


def _assert_indices_and_free_list_partition(hm, size, capacity):
    both = torch.cat([hm.engine.items()[1], hm.engine._heap[size:].long()])
    assert torch.equal(torch.sort(both)[0].cpu(), torch.arange(capacity))


def _check_value_map(hm, keys, values, capacity, untouched):
    """Every distinct key of `keys` is stored once; its rows come from ONE
    source row that holds this key; the indices in use and the free list
    heap[size ..] together are every index once (ash/src/hashmap_gpu.cuh:226-231:
    a new key takes heap[counter++], inserts never write to the heap); rows of
    free indices still hold `untouched`."""
    uniq = torch.unique(keys, dim=0)
    n = keys.shape[0]
    size = hm.size()
    idx, masks = hm.engine.find(uniq)
    assert bool(masks.all())
    assert_is_bijection_into(idx, capacity)
    heap = hm.engine._heap
    _assert_indices_and_free_list_partition(hm, size, capacity)
    color, depth = hm.color[idx], hm.depth[idx]
    src = depth[:, 0].long()
    assert bool((src >= 0).all()) and bool((src < n).all())
    assert torch.equal(color, values["color"][src]) and torch.equal(keys[src], uniq)
    free = heap[size:].long()
    assert bool((hm.color[free] == untouched).all()) and bool((hm.depth[free] == untouched).all())
    return uniq


@pytest.mark.parametrize("duplicates", [0.0, 0.001, 0.5])
def test_bulk_values_keep_the_heap_protocol(bulk_ash, oracle, duplicates):
    """The streaming insert with value rows promises row i the heap position
    counter + i and repairs the promise where keys lose: no duplicates (the
    promise holds), a few (a handful of moves), half of the batch (most winners
    of the upper half move).  Checked each time: key set against the oracle,
    one source row per key, indices = heap[0 .. size), free rows untouched."""
    dim, capacity = 3, 300_000
    rng = np.random.default_rng(960 + int(duplicates * 1000))
    n = 200_000
    distinct = torch.unique(_random_keys(rng, 3 * n, dim, 60), dim=0)
    distinct = distinct[torch.from_numpy(rng.permutation(len(distinct)))][:n]
    n_dup = int(n * duplicates)
    keys = distinct.clone()
    if n_dup:
        keys[rng.permutation(n)[:n_dup]] = distinct[rng.integers(0, n, size=n_dup)]
    keys = keys.to(DEV)
    row = torch.arange(n, device=DEV, dtype=torch.float32)
    values = {"color": torch.stack([row, row + 0.5, 2 * row], dim=1), "depth": row.view(-1, 1).clone()}
    hm = bulk_ash.HashMap(dim, {"color": 3, "depth": 1}, capacity, DEV)
    hm.color.fill_(-7.0)
    hm.depth.fill_(-7.0)
    hm.insert(keys, values)
    uniq = _check_value_map(hm, keys, values, capacity, -7.0)
    assert hm.size() == len(uniq)
    # a fresh heap: the indices are 0 .. size-1
    assert torch.equal(torch.sort(hm.engine.items()[1])[0].cpu(), torch.arange(len(uniq)))
    omap = _oracle_map(oracle, dim, capacity)
    omap.insert_keys(keys.cpu())
    _assert_same_map(hm.engine, omap, _random_keys(rng, 50_000, dim, 62).to(DEV))


def test_bulk_values_into_a_populated_map_with_a_shuffled_heap(bulk_ash, oracle):
    """Second batch with value rows into a map that holds keys (half of the
    batch is already stored), after erases have put indices back on the heap in
    another order (the heap is read instead of assumed to be 0, 1, 2, ...), and
    a third batch that asks for more than the heap still has."""
    dim, capacity = 3, 260_000
    rng = np.random.default_rng(970)
    pool = torch.unique(_random_keys(rng, 900_000, dim, 70), dim=0)
    pool = pool[torch.from_numpy(rng.permutation(len(pool)))].to(DEV)
    first, second_new, third_new = pool[:120_000], pool[120_000:200_000], pool[200_000:420_000]

    def rows_for(keys, offset):
        row = torch.arange(len(keys), device=DEV, dtype=torch.float32) + offset
        return {"color": torch.stack([row, row + 0.5, 2 * row], dim=1), "depth": row.view(-1, 1).clone()}

    hm = bulk_ash.HashMap(dim, {"color": 3, "depth": 1}, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    hm.insert(first, rows_for(first, 0))
    omap.insert_keys(first.cpu())
    gone = first[torch.from_numpy(rng.permutation(len(first))[:50_000]).to(DEV)]
    hm.erase(gone)
    omap.erase(gone.cpu())
    assert hm.size() == 70_000
    hm.color[hm.engine._heap[70_000:].long()] = -7.0
    hm.depth[hm.engine._heap[70_000:].long()] = -7.0
    second = torch.cat([second_new, first[:80_000]])
    second = second[torch.from_numpy(rng.permutation(len(second))).to(DEV)]
    before = {k: v.clone() for k, v in hm.values.items()}
    old_idx, old_mask = hm.engine.find(second)
    hm.insert(second, rows_for(second, 1_000_000))
    omap.insert_keys(second.cpu())
    _assert_same_map(hm.engine, omap, pool[:450_000:3].contiguous())
    size = hm.size()
    heap = hm.engine._heap
    _assert_indices_and_free_list_partition(hm, size, capacity)
    # keys that were stored keep their index and their rows
    new_idx, new_mask = hm.engine.find(second)
    assert bool(new_mask.all()) and torch.equal(new_idx[old_mask], old_idx[old_mask])
    kept = old_idx[old_mask]
    assert torch.equal(hm.color[kept], before["color"][kept])
    # new keys carry the rows of their source row
    fresh = ~old_mask
    src = (hm.depth[new_idx[fresh], 0] - 1_000_000).long()
    assert torch.equal(second[src], second[fresh])
    free = heap[size:].long()
    assert bool((hm.color[free] == -7.0).all()) and bool((hm.depth[free] == -7.0).all())
    # third batch: more new keys than the heap has left
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        hm.insert(third_new, rows_for(third_new, 2_000_000))
    assert hm.size() == capacity
    idx3, mask3 = hm.engine.find(third_new)
    assert int(mask3.sum()) == capacity - size
    src3 = (hm.depth[idx3[mask3], 0] - 2_000_000).long()
    assert torch.equal(third_new[src3], third_new[mask3])
    assert_is_bijection_into(hm.engine.items()[1], capacity)


def test_streaming_insert_refuses_a_pending_fill_under_capture(gpu_ash):
    """ash_map_insert_bulk after a clear decides on the host that the build
    pass rewrites every bucket; recorded into a graph that decision would be
    replayed against whatever the table holds then, so the call fails while
    the stream is being captured and works outside."""
    lib = gpu_ash.common.load_library()
    engine = gpu_ash.ASHEngine(3, 50_000, DEV)
    backend = engine.backend
    keys = torch.unique(torch.randint(-40, 40, (30_000, 3), dtype=torch.int32), dim=0).to(DEV)
    engine.insert_keys(keys)
    engine.clear()
    nbytes, worth = ctypes.c_int64(0), ctypes.c_int(0)
    assert lib.ash_map_bulk_workspace_bytes(backend._handle, len(keys), 0, None,
                                            ctypes.byref(nbytes), ctypes.byref(worth)) == 0
    assert nbytes.value > 0
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.ash_map_insert_bulk(backend._handle, keys.data_ptr(), len(keys), 0, None, None,
                                         None, ws.data_ptr(), ws.numel(), side.cuda_stream)
    assert rc != 0 and "cleared" in lib.ash_last_error().decode()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream(DEV).cuda_stream
    rc = lib.ash_map_insert_bulk(backend._handle, keys.data_ptr(), len(keys), 0, None, None, None,
                                 ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, lib.ash_last_error().decode()
    assert backend.status()["size"] == len(keys)
    assert bool(engine.find(keys)[1].all())


def test_streaming_insert_returns_before_its_counters_are_read(bulk_ash, oracle):
    """A streaming insert whose first pass hands no key to the per-key kernel
    returns without waiting for the table's counters; they are looked at when
    somebody asks (size, items, the next insert) and dropped when an erase or a
    clear makes them stale.  A batch with an unpackable key takes the waiting
    path (the key has to be re-issued into the second region before anything
    else looks at the map).  Two maps at once: each has its own landing place."""
    dim, capacity = 3, 120_000
    rng = np.random.default_rng(990)
    a, b = bulk_ash.ASHEngine(dim, capacity, DEV), bulk_ash.ASHEngine(dim, capacity, DEV)
    oa, ob = _oracle_map(oracle, dim, capacity), _oracle_map(oracle, dim, capacity)
    ka, kb = _random_keys(rng, 90_000, dim, 30), _random_keys(rng, 70_000, dim, 28)
    a.insert_keys(ka.to(DEV))
    b.insert_keys(kb.to(DEV))
    assert a.backend.counters_queued and b.backend.counters_queued
    # look-ups do not need the counters
    _, mask = a.find(ka[:1000].to(DEV))
    assert bool(mask.all()) and a.backend.counters_queued
    oa.insert_keys(ka)
    ob.insert_keys(kb)
    assert b.size() == ob.size() and not b.backend.counters_queued
    assert a.size() == oa.size() and not a.backend.counters_queued
    # an erase makes queued counters stale
    a.insert_keys(_random_keys(rng, 10_000, dim, 31).to(DEV))
    assert a.backend.counters_queued
    gone = ka[:5_000]
    a.erase(gone.to(DEV))
    assert not a.backend.counters_queued
    oa2 = _oracle_map(oracle, dim, capacity)
    k_now, _ = a.items()
    oa2.insert_keys(k_now.cpu())
    assert a.size() == oa2.size()
    _, mask = a.find(gone.to(DEV))
    left = set(map(tuple, k_now.cpu().tolist()))
    assert mask.cpu().tolist() == [tuple(k) in left for k in gone.tolist()]
    # a batch with a key that does not pack waits and re-issues
    odd = torch.tensor([[2**30, 5, -(2**30)]], dtype=torch.int32)
    batch = torch.cat([_random_keys(rng, 8_000, dim, 29), odd])
    b.insert_keys(batch.to(DEV))
    assert not b.backend.counters_queued
    ob.insert_keys(batch)
    _assert_same_map(b, ob, torch.cat([batch, kb[:2000]]).to(DEV))
    # with the second region attached an unpackable key still takes the waiting path
    b.insert_keys(torch.cat([_random_keys(rng, 6_000, dim, 27), odd + 1]).to(DEV))
    assert not b.backend.counters_queued
    b.insert_keys(_random_keys(rng, 6_000, dim, 27).to(DEV))
    assert b.backend.counters_queued and b.size() <= capacity

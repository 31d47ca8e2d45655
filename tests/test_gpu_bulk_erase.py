"""GPU parity tests of the streaming erase path (ash_map_erase_bulk): forced on
for every batch that it accepts, it must leave the same map as the oracle and
as the per-key kernel -- same key set, masks and size, every freed index back
on the heap once, and the key log cleared so that items() lists what is left."""
import numpy as np
import pytest
import torch

from helpers import sort_rows
from test_gpu_hash import _assert_same_map, _oracle_map

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture()
def streaming(gpu_ash, monkeypatch):
    monkeypatch.setattr(gpu_ash.common, "BULK_ERASE", "always")
    return gpu_ash


def _random_keys(rng, n, dim, span):
    return torch.from_numpy(rng.integers(-span, span, size=(n, dim)).astype(np.int32))


def _assert_heap_partition(engine):
    """Indices in use and the free list heap[size ..] are every index once
    (ash/src/hashmap_gpu.cuh:316-351: an erased key's index goes back to
    heap[--counter])."""
    size = engine.size()
    both = torch.cat([engine.items()[1], engine._heap[size:].long()])
    assert torch.equal(torch.sort(both)[0].cpu(), torch.arange(engine.capacity))


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_streaming_erase_matches_oracle(streaming, oracle, dim):
    """Stored keys, keys that are not stored, the same key several times in
    one batch; then the freed indices are taken again by an insert."""
    capacity = 200_000
    rng = np.random.default_rng(1200 + dim)
    span = {1: 90_000, 2: 210, 3: 30, 4: 11}[dim]
    engine = streaming.ASHEngine(dim, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    first = _random_keys(rng, 260_000, dim, span)
    engine.insert_keys(first.to(DEV))
    omap.insert_keys(first)
    stored = torch.unique(first, dim=0)
    gone = torch.cat([
        stored[rng.permutation(len(stored))[: len(stored) // 2]],
        _random_keys(rng, 30_000, dim, span + 3),          # mostly not stored
        stored[rng.integers(0, len(stored), size=20_000)],  # repeats
    ])
    gone = gone[torch.from_numpy(rng.permutation(len(gone)))]
    engine.erase(gone.to(DEV))
    assert engine.backend.last_erase_path == "streaming"
    omap.erase(gone)
    probe = torch.cat([first[:60_000], gone[:40_000]])
    _assert_same_map(engine, omap, probe.to(DEV))
    _assert_heap_partition(engine)
    second = _random_keys(rng, 120_000, dim, span + 1)
    engine.insert_keys(second.to(DEV))
    omap.insert_keys(second)
    _assert_same_map(engine, omap, probe.to(DEV))
    _assert_heap_partition(engine)
    # everything that is left
    left, _ = engine.items()
    engine.erase(left)
    assert engine.size() == 0 and engine.backend.status()["dropped"] == 0
    _, mask = engine.find(probe.to(DEV))
    assert not bool(mask.any())
    _assert_heap_partition(engine)


def test_streaming_erase_equals_per_key_kernel(gpu_ash, monkeypatch):
    """The same operations through both paths: same keys left, same size, and in
    both the freed indices are the free list.  The number of tombstones is
    about the same (a slot becomes a tombstone when its bucket has no empty slot
    at that moment, which depends on which erase of a full bucket comes
    first)."""
    dim, capacity = 3, 300_000
    rng = np.random.default_rng(1210)
    keys = torch.unique(_random_keys(rng, 500_000, dim, 45), dim=0)
    keys = keys[torch.from_numpy(rng.permutation(len(keys)))][:280_000].to(DEV)
    gone = keys[torch.from_numpy(rng.permutation(len(keys)))[:150_000].to(DEV)]
    results = []
    for mode in ("never", "always"):
        monkeypatch.setattr(gpu_ash.common, "BULK_ERASE", mode)
        engine = gpu_ash.ASHEngine(dim, capacity, DEV)
        engine.insert_keys(keys)
        engine.erase(gone)
        assert engine.backend.last_erase_path == ("per-key" if mode == "never" else "streaming")
        left, idx = engine.items()
        _assert_heap_partition(engine)
        results.append((sort_rows(left)[0], engine.size(), engine.backend.status()["tombstones"]))
    assert torch.equal(results[0][0], results[1][0])
    assert results[0][1] == results[1][1]
    assert abs(results[0][2] - results[1][2]) <= 0.25 * max(results[0][2], results[1][2]) + 50


def test_streaming_erase_piles_unpackable_keys_and_values(streaming, oracle):
    """One key repeated far beyond what a range of the split holds (those
    records go to the per-key kernel), keys that do not fit the packed code
    (second region), and a map with value rows: rows of the keys that stay are
    untouched, rows freed are given to the keys inserted afterwards."""
    dim, capacity = 3, 60_000
    rng = np.random.default_rng(1220)
    spread = torch.unique(_random_keys(rng, 60_000, dim, 20), dim=0)[:40_000]
    big = torch.unique(torch.from_numpy(
        rng.integers(-(2**31), 2**31 - 1, size=(3_000, dim)).astype(np.int32)), dim=0)
    keys = torch.cat([spread, big])
    hm = streaming.HashMap(dim, {"v": dim}, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    hm.insert(keys.to(DEV), {"v": keys.to(DEV).float()})
    omap.insert_keys(keys)
    pile = spread[:5][rng.integers(0, 5, size=150_000)]
    gone = torch.cat([pile, spread[100:15_000], big[:1_500], big[:200]])
    gone = gone[torch.from_numpy(rng.permutation(len(gone)))]
    hm.erase(gone.to(DEV))
    assert hm.engine.backend.last_erase_path == "streaming"
    omap.erase(gone)
    _assert_same_map(hm.engine, omap, keys.to(DEV))
    _assert_heap_partition(hm.engine)
    masks, idx, rows = hm.find(keys.to(DEV), return_values=True)
    assert torch.equal(rows["v"][masks].cpu(), keys[masks.cpu()].float())
    fresh = _random_keys(rng, 15_000, dim, 20) + 100
    hm.insert(fresh.to(DEV), {"v": fresh.to(DEV).float()})
    omap.insert_keys(fresh)
    _assert_same_map(hm.engine, omap, torch.cat([keys, fresh]).to(DEV))
    everything = torch.cat([keys, fresh]).to(DEV)
    masks, idx, rows = hm.find(everything, return_values=True)
    assert torch.equal(rows["v"][masks], everything[masks].float())
    _assert_heap_partition(hm.engine)


def test_path_is_chosen_by_batch_size(gpu_ash):
    """As shipped: a batch of the order of the table streams, a small one goes
    key by key; a table too small for the streaming path never streams."""
    dim = 3
    rng = np.random.default_rng(1230)
    engine = gpu_ash.ASHEngine(dim, 4_000_000, DEV)
    keys = torch.unique(_random_keys(rng, 3_000_000, dim, 200), dim=0).to(DEV)
    engine.insert_keys(keys)
    engine.erase(keys[:10_000])
    assert engine.backend.last_erase_path == "per-key"
    engine.erase(keys[10_000:])
    assert engine.backend.last_erase_path == "streaming"
    assert engine.size() == 0
    small = gpu_ash.ASHEngine(dim, 50_000, DEV)
    small.insert_keys(keys[:40_000])
    small.erase(keys[:40_000])
    assert small.backend.last_erase_path == "per-key" and small.size() == 0

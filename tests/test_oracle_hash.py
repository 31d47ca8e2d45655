"""Pins the hash-map half of the CPU oracle without the reference binary:
against a sequential dictionary model with the reference's heap protocol, and
against the invariants the reference's own unit tests assert
(unittests/test_engine.py, test_hashset.py)."""
import numpy as np
import pytest
import torch

from helpers import DictMap, assert_is_bijection_into, sort_rows


def _heap(capacity):
    return torch.arange(capacity, dtype=torch.int32)


def _tiled_keys(dim, num, seed):
    g = torch.Generator().manual_seed(seed)
    keys = torch.arange(num, dtype=torch.int32).view(-1, 1).tile((1, dim))
    return keys[torch.randperm(num, generator=g)]


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_random_ops_match_dict_model(oracle, dim):
    """Insert / find / erase batches with duplicates and misses; single-thread
    oracle is sequential, so even the allocated indices must equal the model's."""
    oracle.set_num_threads(1)
    try:
        capacity = 500
        rng = np.random.default_rng(100 + dim)
        heap = _heap(capacity)
        m = oracle.HashMap(dim, capacity, heap)
        model = DictMap(dim, capacity)
        for step in range(30):
            n = int(rng.integers(1, 200))
            keys = rng.integers(-6, 6, size=(n, dim)).astype(np.int32)
            op = step % 3
            if op == 0:
                m.insert_keys(torch.from_numpy(keys))
                model.insert(keys)
            elif op == 1:
                m.erase(torch.from_numpy(keys[: n // 3]))
                model.erase(keys[: n // 3])
            probe = rng.integers(-7, 7, size=(300, dim)).astype(np.int32)
            idx, mask = m.find(torch.from_numpy(probe))
            ref_idx, ref_mask = model.find(probe)
            assert np.array_equal(mask.numpy(), ref_mask)
            assert np.array_equal(idx.numpy(), ref_idx)
            assert m.size() == model.size()
            assert heap.tolist() == model.heap
        keys_out, idx_out = m.items()
        got = {tuple(k): int(i) for k, i in zip(keys_out.tolist(), idx_out.tolist())}
        assert got == model.table
    finally:
        oracle.set_num_threads(0)


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_reference_engine_invariants(oracle, dim):
    """unittests/test_engine.py:21-83: exactly-capacity inserts succeed and use
    exactly the indices [0, num); erase empties; 3x duplicates insert once;
    items() equals the inserted set."""
    capacity = num = 20000
    keys = _tiled_keys(dim, num, seed=dim)
    m = oracle.HashMap(dim, capacity, _heap(capacity))
    m.insert_keys(keys)
    assert m.size() == num
    idx, mask = m.find(keys)
    assert int(mask.sum()) == num
    assert torch.equal(torch.unique(idx), torch.arange(num))

    active_keys, active_idx = m.items()
    assert torch.equal(sort_rows(active_keys)[0], sort_rows(keys)[0])
    assert_is_bijection_into(active_idx, capacity)

    m.erase(keys)
    assert m.size() == 0
    assert not m.find(keys)[1].any()

    dup = keys.tile((3, 1))[torch.randperm(3 * num, generator=torch.Generator().manual_seed(7))]
    m.insert_keys(dup)
    assert m.size() == num
    idx, mask = m.find(dup)
    assert int(mask.sum()) == 3 * num
    assert torch.equal(torch.unique(idx), torch.arange(num))


def test_find_miss_returns_index_zero(oracle):
    """ash/src/hashmap_gpu.cuh:177: indices of misses are 0, not -1."""
    m = oracle.HashMap(3, 16, _heap(16))
    m.insert_keys(torch.tensor([[1, 2, 3]], dtype=torch.int32))
    idx, mask = m.find(torch.tensor([[1, 2, 3], [9, 9, 9]], dtype=torch.int32))
    assert mask.tolist() == [True, False]
    assert idx[1].item() == 0


def test_values_follow_their_keys(oracle):
    """unittests/test_engine.py:121-159: mixed int64 / float32 value rows land at
    the key's index."""
    capacity, num, dim = 4096, 3000, 3
    keys = _tiled_keys(dim, num, seed=3)
    store = {
        "0": torch.zeros(capacity, dim, dtype=torch.int64),
        "1": torch.zeros(capacity, dim, dtype=torch.float32),
    }
    values = {"0": keys.long() * 2, "1": keys.float() * 4}
    m = oracle.HashMap(dim, capacity, _heap(capacity))
    m.insert(keys, values, store)
    idx, mask = m.find(keys)
    assert mask.all()
    assert torch.equal(store["0"][idx], keys.long() * 2)
    assert torch.equal(store["1"][idx], keys.float() * 4)


def test_overflow_is_refused_and_counted(oracle):
    capacity = 100
    keys = _tiled_keys(2, 150, seed=5)
    heap = _heap(capacity)
    m = oracle.HashMap(2, capacity, heap)
    m.insert_keys(keys)
    st = m.status()
    assert st["size"] == capacity and st["dropped"] == 50
    idx, mask = m.find(keys)
    assert int(mask.sum()) == capacity
    assert_is_bijection_into(idx[mask], capacity)


def test_parallel_overflow_keeps_the_map_consistent(oracle):
    capacity, dim = 30000, 3
    g = torch.Generator().manual_seed(22)
    keys = torch.randint(-40, 40, (120000, dim), generator=g, dtype=torch.int32)
    oracle.set_num_threads(4)
    try:
        m = oracle.HashMap(dim, capacity, _heap(capacity))
        m.insert_keys(keys)
    finally:
        oracle.set_num_threads(0)
    assert m.size() == capacity
    k, i = m.items()
    assert len(torch.unique(k, dim=0)) == capacity
    assert torch.equal(torch.sort(i)[0], torch.arange(capacity))
    idx, mask = m.find(keys)
    assert int(mask.sum()) >= capacity


def test_load_round_trip(oracle):
    """unittests/test_engine.py:85-106 at the backend level, including the
    empty map."""
    capacity, dim = 1000, 3
    for num in (0, 700):
        heap = _heap(capacity)
        a = oracle.HashMap(dim, capacity, heap)
        keys = _tiled_keys(dim, num, seed=11) if num else torch.zeros((0, dim), dtype=torch.int32)
        if num:
            a.insert_keys(keys)
            a.erase(keys[:50])
        k, i = a.items()
        # as load_state_dict does: a fresh map, then the saved heap copied into
        # its buffer, then the pairs handed to load_states
        heap_b = _heap(capacity)
        b = oracle.HashMap(dim, capacity, heap_b)
        heap_b.copy_(heap)
        b.load_states({"active_keys": k, "active_indices": i, "heap": heap_b})
        assert b.size() == a.size()
        k2, i2 = b.items()
        assert all(torch.equal(x, y) for x, y in zip(sort_rows(k, i), sort_rows(k2, i2)))
        # the loaded map keeps allocating from where the saved one stopped
        fresh = torch.tensor([[5000, 5000, 5000]], dtype=torch.int32)
        a.insert_keys(fresh)
        b.insert_keys(fresh)
        assert a.find(fresh)[0].item() == b.find(fresh)[0].item()


def test_parallel_matches_sequential_as_sets(oracle):
    """With OpenMP threads the order of allocation is free, everything else is
    not: same key set, same masks, indices a bijection onto [0, n)."""
    capacity, dim = 200000, 3
    g = torch.Generator().manual_seed(21)
    keys = torch.randint(-40, 40, (120000, dim), generator=g, dtype=torch.int32)
    oracle.set_num_threads(4)
    try:
        par = oracle.HashMap(dim, capacity, _heap(capacity))
        par.insert_keys(keys)
    finally:
        oracle.set_num_threads(1)
    seq = oracle.HashMap(dim, capacity, _heap(capacity))
    seq.insert_keys(keys)
    oracle.set_num_threads(0)
    assert par.size() == seq.size() == len(torch.unique(keys, dim=0))
    kp, ip = par.items()
    ks, _ = seq.items()
    assert torch.equal(sort_rows(kp)[0], sort_rows(ks)[0])
    assert torch.equal(torch.sort(ip)[0], torch.arange(par.size()))

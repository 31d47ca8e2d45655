"""GPU parity tests of the hash map: the HIP table against the CPU oracle on
identical seeded inputs (masks and key sets bit-exact, indices compared through
the values they address, since parallel allocation order is free), and the
reference's own unit-test assertions (unittests/test_engine.py,
test_hashset.py, test_hashmap.py, test_embedding.py) on the device."""
import os

import numpy as np
import pytest
import torch

import workloads
from helpers import assert_is_bijection_into, sort_rows

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _tiled_keys(dim, num, seed=0):
    g = torch.Generator().manual_seed(seed)
    keys = torch.arange(num, dtype=torch.int32).view(-1, 1).tile((1, dim))
    return keys[torch.randperm(num, generator=g)].to(DEV)


def _oracle_map(oracle, dim, capacity):
    return oracle.HashMap(dim, capacity, torch.arange(capacity, dtype=torch.int32))


def _assert_same_map(engine, omap, probe):
    """Same size, same key set, same masks for `probe`, indices a bijection."""
    assert engine.size() == omap.size()
    k_gpu, i_gpu = engine.items()
    k_cpu, _ = omap.items()
    assert torch.equal(sort_rows(k_gpu)[0], sort_rows(k_cpu)[0])
    assert_is_bijection_into(i_gpu, engine.capacity)
    idx, mask = engine.find(probe)
    _, mask_cpu = omap.find(probe.cpu())
    assert torch.equal(mask.cpu(), mask_cpu)
    assert bool((idx[~mask] == 0).all())
    # find() and items() agree on the mapping
    lookup, found = engine.find(k_gpu)
    assert bool(found.all()) and torch.equal(lookup, i_gpu)


# ------------------------------------------------ reference unit tests, engine
@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_engine_insert_find_erase_duplicates(gpu_ash, dim):
    capacity = num = 100000
    engine = gpu_ash.ASHEngine(dim, capacity, DEV)
    keys = _tiled_keys(dim, num, seed=dim)
    engine.insert_keys(keys)
    assert engine.size() == num
    idx, mask = engine.find(keys)
    assert int(mask.sum()) == num
    assert torch.equal(torch.unique(idx), torch.arange(num, device=DEV))

    active_keys, _ = engine.items()
    assert torch.equal(sort_rows(active_keys)[0], sort_rows(keys)[0])

    engine.erase(keys)
    assert engine.size() == 0
    assert not bool(engine.find(keys)[1].any())

    dup = keys.tile((3, 1))[torch.randperm(3 * num, device=DEV)]
    engine.insert_keys(dup)
    assert engine.size() == num
    idx, mask = engine.find(dup)
    assert int(mask.sum()) == 3 * num
    assert torch.equal(torch.unique(idx), torch.arange(num, device=DEV))


@pytest.mark.parametrize("dim", [1, 2, 3, 4])
@pytest.mark.parametrize("num", [0, 100000])
def test_engine_state_dict_round_trip(gpu_ash, dim, num, tmp_path):
    capacity = 100000
    engine = gpu_ash.ASHEngine(dim, capacity, DEV)
    keys = _tiled_keys(dim, num, seed=10 + dim)
    if num:
        engine.insert_keys(keys)
        engine.erase(keys[:1000])
        kept = keys[1000:]
    else:
        kept = keys
    path = os.path.join(tmp_path, "state.pt")
    torch.save(engine.state_dict(), path)
    before_keys, before_idx = engine.items()
    del engine
    state = torch.load(path, map_location=DEV)
    assert set(state) == {"_heap", "_keys", "_indices", "_size"}
    assert state["_heap"].dtype == torch.int32 and state["_keys"].shape == (capacity, dim)
    assert state["_indices"].dtype == torch.int64 and state["_size"].dtype == torch.int32
    engine = gpu_ash.ASHEngine(dim, capacity, DEV)
    engine.load_state_dict(state)
    after_keys, after_idx = engine.items()
    assert len(after_keys) == len(kept)
    assert all(
        torch.equal(a, b)
        for a, b in zip(sort_rows(before_keys, before_idx), sort_rows(after_keys, after_idx))
    )
    if num:
        # the restored heap continues where the saved one stopped
        engine.insert_keys(keys[:10])
        idx, mask = engine.find(keys[:10])
        assert bool(mask.all())
        assert_is_bijection_into(engine.items()[1], capacity)


def test_gather_rows_equals_torch_indexing(gpu_ash):
    """ash_gather_rows behind HashMap.find / items (return_values=True) against
    the reference's formulation, values[name][indices] (ash/hashmap.py:87-95):
    one to five tensors (more than one launch), row widths 1..5 and 20 words,
    float and int rows, sorted and random indices, and the tables torch keeps
    (rows of 2 bytes)."""
    backend = gpu_ash.core.backend
    g = torch.Generator().manual_seed(5)
    rows = 50_000
    tables = {
        "a": torch.rand(rows, 3, generator=g),
        "b": torch.rand(rows, 1, generator=g),
        "c": torch.randint(-9, 9, (rows, 5), generator=g, dtype=torch.int32),
        "d": torch.rand(rows, 4, generator=g, dtype=torch.float64),
        "e": torch.rand(rows, 20, generator=g),
        "f": torch.rand(rows, 1, generator=g).to(torch.float16),
    }
    tables = {k: v.to(DEV) for k, v in tables.items()}
    for n in (0, 1, 70_001):
        for order in ("random", "sorted"):
            idx = torch.randint(0, rows, (n,), generator=g)
            idx = (torch.sort(idx)[0] if order == "sorted" else idx).to(DEV)
            for names in (("a",), ("a", "b"), tuple("abcdef")):
                got = backend.gather_rows({k: tables[k] for k in names}, idx)
                assert tuple(got) == names
                for k in names:
                    assert got[k].dtype == tables[k].dtype
                    assert torch.equal(got[k], tables[k][idx]), (k, n, order)
    # through the map: values of found keys and of items()
    hm = gpu_ash.HashMap(3, {"color": 3, "depth": 1}, 40_000, DEV)
    keys = torch.unique(torch.randint(-30, 30, (30_000, 3), generator=g, dtype=torch.int32), dim=0).to(DEV)
    values = {"color": torch.rand(len(keys), 3, device=DEV), "depth": torch.rand(len(keys), 1, device=DEV)}
    hm.insert(keys, values)
    masks, idx, found = hm.find(keys, return_values=True)
    assert bool(masks.all())
    assert torch.equal(found["color"], values["color"]) and torch.equal(found["depth"], values["depth"])
    k2, i2, v2 = hm.items(return_indices=True, return_values=True)
    assert torch.equal(v2["color"], hm.color[i2]) and torch.equal(v2["depth"], hm.depth[i2])
    order = sort_rows(k2, i2)
    assert torch.equal(order[0], sort_rows(keys)[0])


def test_listing_in_index_order_while_nothing_was_erased(gpu_ash):
    """While nothing has been erased or loaded since the clear (and no key
    lives in the second region) entry i of items() is index i and the value
    rows of the listing are the first rows of the value tensors, copied; after
    an erase, with a key that does not pack, or after a load the listing goes
    by the key log and the rows are gathered.  Either way:
    values[name][indices] (ash/hashmap.py:138-146)."""
    g = torch.Generator().manual_seed(77)
    hm = gpu_ash.HashMap(3, {"color": 3, "depth": 1}, 60_000, DEV)
    backend = hm.engine.backend
    keys = torch.unique(torch.randint(-40, 40, (50_000, 3), generator=g, dtype=torch.int32), dim=0)
    keys = keys[torch.randperm(len(keys), generator=g)].to(DEV)
    first, second = keys[:20_000], keys[20_000:45_000]

    def check(expect_dense, stored):
        k, i, v = hm.items(return_indices=True, return_values=True)
        assert backend.last_items_in_index_order == expect_dense
        if expect_dense:
            assert torch.equal(i, torch.arange(len(i), device=DEV))
        assert torch.equal(v["color"], hm.color[i]) and torch.equal(v["depth"], hm.depth[i])
        assert v["color"].data_ptr() != hm.color.data_ptr()   # a copy, not a view
        assert torch.equal(sort_rows(k)[0], sort_rows(stored)[0])
        masks, idx = hm.find(k)
        assert bool(masks.all()) and torch.equal(idx, i)
        # a second listing may come in another order; every row belongs to its key
        k2, v2 = hm.items(return_indices=False, return_values=True)
        assert torch.equal(v2["color"], k2.float()) and torch.equal(v2["depth"], k2[:, :1].float() * 0.5)

    def rows(k):
        return {"color": k.float(), "depth": k[:, :1].float() * 0.5}

    hm.insert(first, rows(first))
    check(True, first)
    hm.insert(torch.cat([second, first[:500]]), rows(torch.cat([second, first[:500]])))
    check(True, torch.cat([first, second]))
    hm.erase(first[:3_000])
    check(False, torch.cat([first[3_000:], second]))
    hm.clear()
    hm.insert(second, rows(second))
    check(True, second)
    odd = torch.tensor([[2**30, -(2**30), 5]], dtype=torch.int32, device=DEV)
    hm.insert(odd, rows(odd))
    check(False, torch.cat([second, odd]))
    state = hm.state_dict()
    other = gpu_ash.HashMap(3, {"color": 3, "depth": 1}, 60_000, DEV)
    other.load_state_dict(state)
    k, i, v = other.items(return_indices=True, return_values=True)
    assert not other.engine.backend.last_items_in_index_order
    assert torch.equal(v["color"], other.color[i])


def test_state_with_duplicate_keys_is_refused(gpu_ash):
    """A saved state whose active keys repeat a key (the reference prints
    "should never reach here", ash/src/hashmap_gpu.cuh:420-422, and goes on
    with a heap counter that exceeds the stored entries) is refused and leaves
    the map empty and usable."""
    capacity = 5000
    engine = gpu_ash.ASHEngine(3, capacity, DEV)
    keys = _tiled_keys(3, 3000, seed=77)
    engine.insert_keys(keys)
    state = {k: v.clone() for k, v in engine.state_dict().items()}
    state["_keys"][10] = state["_keys"][20]
    other = gpu_ash.ASHEngine(3, capacity, DEV)
    with pytest.raises(RuntimeError, match="duplicate keys"):
        other.load_state_dict(state)
    assert other.size() == 0 and other.items()[0].shape[0] == 0
    other.insert_keys(keys[:100])
    idx, mask = other.find(keys[:200])
    assert int(mask.sum()) == 100 and other.size() == 100
    assert torch.equal(torch.sort(idx[:100])[0].cpu(), torch.arange(100))


@pytest.mark.parametrize(
    "dim,num,old,new", [(1, 50000, 100000, 50000), (1, 100000, 100000, 200000),
                        (3, 50000, 100000, 50000), (3, 100000, 100000, 200000)]
)
def test_engine_resize_and_multivalue(gpu_ash, dim, num, old, new):
    """unittests/test_engine.py:108-159,200-250."""
    engine = gpu_ash.ASHEngine(dim, old, DEV)
    stores = {
        "0": torch.zeros(old, dim, dtype=torch.int64, device=DEV),
        "1": torch.zeros(old, dim, dtype=torch.float32, device=DEV),
    }
    keys = _tiled_keys(dim, num, seed=20 + dim)
    values = {"0": keys.long() * 2, "1": keys.float() * 4}
    engine.insert(keys, values, stores)
    idx, mask = engine.find(keys)
    assert int(mask.sum()) == num
    assert torch.equal(stores["0"][idx], keys.long() * 2)
    assert torch.equal(stores["1"][idx], keys.float() * 4)

    grown = {
        "0": torch.zeros(new, dim, dtype=torch.int64, device=DEV),
        "1": torch.zeros(new, dim, dtype=torch.float32, device=DEV),
    }
    engine.resize(new, stores, grown)
    assert engine.size() == num and engine.capacity == new
    idx, mask = engine.find(keys)
    assert int(mask.sum()) == num
    assert torch.equal(grown["0"][idx], keys.long() * 2)
    assert torch.equal(grown["1"][idx], keys.float() * 4)
    assert torch.equal(sort_rows(engine.keys())[0], sort_rows(keys)[0])


# ------------------------------------------- reference unit tests, set and map
@pytest.mark.parametrize("dim", [1, 2, 3])
@pytest.mark.parametrize("num", [100, 1000, 10000, 100000])
def test_hashset(gpu_ash, dim, num):
    """unittests/test_hashset.py:19-63."""
    hs = gpu_ash.HashSet(dim, 100000, DEV)
    keys = _tiled_keys(dim, num, seed=num + dim)
    hs.insert(keys)
    assert int(hs.find(keys).sum()) == num
    assert torch.equal(sort_rows(hs.keys())[0], sort_rows(keys)[0])
    hs.erase(keys[: num // 2])
    assert int(hs.find(keys).sum()) == num - num // 2
    assert hs.size() == num - num // 2
    hs.erase(keys)
    assert hs.size() == 0
    hs.insert(keys)
    hs.resize(num * 10)
    assert int(hs.find(keys).sum()) == num


@pytest.mark.parametrize(
    "dim,value_dims", [(1, 1), (2, [1, 2, 3]), (3, {"a": 4, "b": 10, "c": 1})]
)
def test_hashmap_values_items_resize_state(gpu_ash, dim, value_dims, tmp_path):
    """unittests/test_hashmap.py:22-204."""
    capacity = num = 100000
    hm = gpu_ash.HashMap(dim, value_dims, capacity, DEV)
    keys = _tiled_keys(dim, num, seed=30 + dim)
    named = {
        name: torch.rand(num, width, device=DEV)
        for name, width in zip(hm.values.keys(), [v.shape[1] for v in hm.values.values()])
    }
    hm.insert(keys, hm.reinterpret_value_dict(named))
    masks, indices, found = hm.find(keys, return_indices=True, return_values=True)
    assert int(masks.sum()) == num
    found = found if isinstance(found, dict) else (
        {"default": found} if isinstance(found, torch.Tensor)
        else {f"default_{i}": v for i, v in enumerate(found)}
    )
    for name in named:
        assert torch.equal(found[name], named[name])  # value of key i is row i
        assert torch.equal(found[name], hm.values[name][indices])

    def check_items(m):
        active_keys, active_idx, active_vals = m.items(return_indices=True, return_values=True)
        assert len(active_keys) == num
        assert torch.equal(sort_rows(active_keys)[0], sort_rows(keys)[0])
        vals = active_vals if isinstance(active_vals, dict) else (
            {"default": active_vals} if isinstance(active_vals, torch.Tensor)
            else {f"default_{i}": v for i, v in enumerate(active_vals)}
        )
        # pair every enumerated key with the row it was inserted with
        order = sort_rows(keys, torch.arange(num))[1]
        for name in named:
            assert torch.equal(vals[name], m.values[name][active_idx])
            got = sort_rows(active_keys, vals[name])[1]
            assert torch.equal(got, named[name].cpu()[order])

    check_items(hm)
    hm.resize(capacity * 2)
    check_items(hm)

    path = os.path.join(tmp_path, "map.pt")
    torch.save(hm.state_dict(), path)
    del hm
    hm = gpu_ash.HashMap(dim, value_dims, capacity * 2, DEV)
    hm.load_state_dict(torch.load(path, map_location=DEV), strict=False)
    check_items(hm)
    hm.clear()
    assert hm.size() == 0 and all(float(v.abs().sum()) == 0 for v in hm.values.values())


@pytest.mark.parametrize("key_dim,feat_dim", [(1, 16), (2, 16), (3, 16), (3, 128)])
def test_embedding_forward_and_training(gpu_ash, key_dim, feat_dim, tmp_path):
    """unittests/test_embedding.py:29-94 (training shortened: the loss only has
    to fall well below its start, the 4000-step regression of the reference is
    a property of Adam, not of the map)."""
    capacity = 1000
    emb = gpu_ash.HashEmbedding(key_dim, capacity, feat_dim, DEV)
    keys = _tiled_keys(key_dim, capacity * 2, seed=40 + key_dim)
    valid = keys[:capacity]
    emb.spatial_init_(valid)
    out = emb(keys)
    assert out.shape == (capacity * 2, feat_dim)
    assert torch.equal(out[capacity:], torch.zeros_like(out[capacity:]))

    target = lambda k: (k[:, 0:1] / capacity).float()
    opt = torch.optim.Adam(emb.parameters(), lr=1e-2)
    first = None
    for step in range(300):
        opt.zero_grad()
        sel = keys[torch.randint(0, capacity * 2, (capacity,), device=DEV)]
        mask = emb.engine.find(sel)[1]
        loss = (((emb(sel) - target(sel)) ** 2).mean(dim=1) * mask).mean()
        loss.backward()
        opt.step()
        first = loss.item() if first is None else first
    assert loss.item() < 0.2 * first
    path = os.path.join(tmp_path, "emb.pt")
    torch.save(emb.state_dict(), path)
    ref = emb(valid).detach()
    emb2 = gpu_ash.HashEmbedding(key_dim, capacity, feat_dim, DEV)
    emb2.load_state_dict(torch.load(path, map_location=DEV))
    assert torch.equal(emb2(valid), ref)


# --------------------------------------------------------- HIP against oracle
@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_random_ops_match_oracle(gpu_ash, oracle, dim):
    capacity = 3000
    rng = np.random.default_rng(500 + dim)
    engine = gpu_ash.ASHEngine(dim, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    # the key universe stays below the capacity: which keys an overfull map
    # refuses is free, so overflow is tested on its own
    span = {1: 1400, 2: 26, 3: 7, 4: 3}[dim]
    for step in range(24):
        n = int(rng.integers(1, 1500))
        keys = torch.from_numpy(rng.integers(-span, span, size=(n, dim)).astype(np.int32))
        if step % 3 != 1:
            engine.backend.insert_keys(keys.to(DEV))
            omap.insert_keys(keys)
        else:
            engine.erase(keys[: n // 2].to(DEV))
            omap.erase(keys[: n // 2])
        probe = torch.from_numpy(rng.integers(-span - 1, span + 1, size=(2000, dim)).astype(np.int32))
        _assert_same_map(engine, omap, probe.to(DEV))


@pytest.mark.parametrize("dim", [2, 3, 4])
def test_unpackable_keys_take_the_second_region(gpu_ash, oracle, dim):
    """Keys whose components do not fit the 64-bit code (dim 3 beyond +-2^20,
    dim 4 beyond +-2^15, the two dim-2 sentinel codes) must behave like any
    other key."""
    capacity = 5000
    g = torch.Generator().manual_seed(60 + dim)
    small = torch.randint(-50, 50, (3000, dim), generator=g, dtype=torch.int32)
    big = torch.randint(-(2**31), 2**31 - 1, (1500, dim), generator=g, dtype=torch.int64).int()
    edge = {
        2: torch.tensor([[2**31 - 1, 2**31 - 1], [2**31 - 2, 2**31 - 1], [-(2**31), -(2**31)]]),
        3: torch.tensor([[2**20, 0, 0], [-(2**20) - 1, 5, 5], [2**20 - 1, -(2**20), 7]]),
        4: torch.tensor([[32767] * 4, [32766, 32767, 32767, 32767], [32768, 0, 0, 0], [-32769, 1, 2, 3]]),
    }[dim].int()
    keys = torch.cat([small, big, edge, edge, big[:200]])
    keys = keys[torch.randperm(len(keys), generator=g)]
    engine = gpu_ash.ASHEngine(dim, capacity, DEV)
    omap = _oracle_map(oracle, dim, capacity)
    stores = {"v": torch.zeros(capacity, dim, dtype=torch.int32, device=DEV)}
    engine.insert(keys.to(DEV), {"v": keys.to(DEV)}, stores)
    omap.insert_keys(keys)
    probe = torch.cat([keys, keys + 1])
    _assert_same_map(engine, omap, probe.to(DEV))
    idx, mask = engine.find(keys.to(DEV))
    assert bool(mask.all()) and torch.equal(stores["v"][idx].cpu(), keys)
    engine.erase(torch.cat([big[:700], edge, small[:100]]).to(DEV))
    omap.erase(torch.cat([big[:700], edge, small[:100]]))
    _assert_same_map(engine, omap, probe.to(DEV))
    # state dict round trip with both regions populated
    state = {k: v.clone() for k, v in engine.state_dict().items()}
    other = gpu_ash.ASHEngine(dim, capacity, DEV)
    other.load_state_dict(state)
    _assert_same_map(other, omap, probe.to(DEV))


def test_overflow_drops_and_warns(gpu_ash):
    capacity = 1000
    engine = gpu_ash.ASHEngine(3, capacity, DEV)
    keys = _tiled_keys(3, 1500, seed=70)
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        engine.insert_keys(keys)
    assert engine.size() == capacity
    idx, mask = engine.find(keys)
    assert int(mask.sum()) == capacity
    assert_is_bijection_into(idx[mask], capacity)
    assert engine.backend.status()["dropped"] == 500
    # the map stays usable: free some room and insert refused keys again
    engine.erase(keys[mask][:300])
    engine.insert_keys(keys[~mask][:300])
    assert engine.size() == capacity
    assert bool(engine.find(keys[~mask][:300])[1].all())


@pytest.mark.parametrize("capacity", [3078, 6150, 122_886])
def test_maps_just_beyond_whole_probe_ranges_fill_to_capacity(gpu_ash, monkeypatch, capacity):
    """Capacities whose bucket count is one bucket (or a few) beyond a multiple
    of the probe range: every distinct key up to the capacity is stored, as in
    the reference, whose map holds `capacity` keys.  Per-key and streaming
    insert, several key sets."""
    for seed, policy in ((0, "never"), (1, "never"), (2, "always"), (3, "always")):
        g = torch.Generator().manual_seed(900 + seed)
        keys = torch.unique(torch.randint(-2000, 2000, (capacity * 2, 3), generator=g,
                                          dtype=torch.int32), dim=0)
        keys = keys[torch.randperm(len(keys), generator=g)][:capacity].to(DEV)
        assert len(keys) == capacity
        engine = gpu_ash.ASHEngine(3, capacity, DEV)
        monkeypatch.setattr(gpu_ash.common, "BULK_INSERT", policy)
        engine.insert_keys(keys)
        status = engine.backend.status()
        assert status["dropped"] == 0 and status["size"] == capacity, (capacity, seed, status)
        idx, mask = engine.find(keys)
        assert bool(mask.all())
        assert_is_bijection_into(idx, capacity)


def test_erase_insert_cycles_at_full_load(gpu_ash, oracle):
    """Buckets that have been full keep tombstones; lookups of keys pushed to a
    following bucket must keep working through many cycles."""
    capacity = 6000
    engine = gpu_ash.ASHEngine(3, capacity, DEV)
    omap = _oracle_map(oracle, 3, capacity)
    g = torch.Generator().manual_seed(80)
    pool = torch.randint(-30, 30, (60000, 3), generator=g, dtype=torch.int32)
    pool = torch.unique(pool, dim=0)
    pool = pool[torch.randperm(len(pool), generator=g)]
    live = pool[:capacity]
    engine.insert_keys(live.to(DEV))
    omap.insert_keys(live)
    cursor = capacity
    for cycle in range(12):
        out = live[torch.randperm(capacity, generator=g)[: capacity // 3]]
        engine.erase(out.to(DEV))
        omap.erase(out)
        new = pool[cursor : cursor + capacity // 3]
        cursor += capacity // 3
        engine.backend.insert_keys(new.to(DEV))
        omap.insert_keys(new)
        live, _ = omap.items()
        _assert_same_map(engine, omap, pool[: cursor + 500].to(DEV))
    assert engine.size() == capacity


def test_empty_and_mistyped_inputs(gpu_ash):
    """ash/core.py:137-145,178-183,197-199: empty batches warn and do nothing,
    non-int32 keys warn and are converted, wrong shapes assert."""
    engine = gpu_ash.ASHEngine(3, 100, DEV)
    empty = torch.zeros((0, 3), dtype=torch.int32, device=DEV)
    with pytest.warns(UserWarning, match="empty keys"):
        idx, mask = engine.find(empty)
    assert idx.shape == (0,) and idx.dtype == torch.int64 and mask.dtype == torch.bool
    with pytest.warns(UserWarning, match="empty keys"):
        engine.insert_keys(empty)
    with pytest.warns(UserWarning, match="empty keys"):
        engine.erase(empty)
    assert engine.size() == 0
    k, i = engine.items()
    assert k.shape == (0, 3) and i.shape == (0,)
    with pytest.warns(UserWarning, match="not int32"):
        engine.insert_keys(torch.tensor([[1, 2, 3]], device=DEV))
    assert bool(engine.find(torch.tensor([[1, 2, 3]], dtype=torch.int32, device=DEV))[1].all())
    with pytest.raises(AssertionError):
        engine.find(torch.zeros((4, 2), dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError, match="Not implemented"):
        gpu_ash.ASHEngine(3, 10, torch.device("cpu"))
    moved = engine.to(DEV)
    assert moved.size() == 0 and moved.capacity == 100


def test_wide_and_odd_value_rows(gpu_ash):
    """Rows wider than the fused path, rows that are not a multiple of 4 bytes,
    and more than four value tensors all take the scatter path."""
    capacity, num = 4096, 3000
    keys = _tiled_keys(3, num, seed=90)
    g = torch.Generator(device=DEV).manual_seed(91)
    values = {
        "wide": torch.rand(num, 8, 40, generator=g, device=DEV),
        "bytes3": torch.randint(0, 255, (num, 3), generator=g, device=DEV, dtype=torch.uint8),
        "half5": torch.rand(num, 5, generator=g, device=DEV).half(),
        "a": torch.rand(num, 1, generator=g, device=DEV),
        "b": torch.rand(num, 2, generator=g, device=DEV).double(),
        "c": torch.randint(0, 9, (num, 4), generator=g, device=DEV),
    }
    stores = {k: torch.zeros((capacity,) + v.shape[1:], dtype=v.dtype, device=DEV) for k, v in values.items()}
    engine = gpu_ash.ASHEngine(3, capacity, DEV)
    engine.insert(keys, values, stores)
    idx, mask = engine.find(keys)
    assert bool(mask.all())
    for name, v in values.items():
        assert torch.equal(stores[name][idx], v), name


# ------------------------------------------------------- benchmark configs
def test_config1_uniform_keys_full_size(gpu_ash, oracle):
    """Configuration 1 at its full size: 1 M keys with 50 % duplicates into a
    set of capacity 2 M, then 1 M queries; masks bit-exact against the oracle."""
    w = workloads.hashset_uniform_keys(device=DEV)
    hs = gpu_ash.HashSet(3, 2_000_000, DEV)
    hs.insert(w["insert_keys"])
    omap = _oracle_map(oracle, 3, 2_000_000)
    omap.insert_keys(w["insert_keys"].cpu())
    assert hs.size() == omap.size()
    masks = hs.find(w["query_keys"])
    _, masks_cpu = omap.find(w["query_keys"].cpu())
    assert torch.equal(masks.cpu(), masks_cpu)
    idx, _ = hs.engine.find(w["query_keys"])
    assert bool((idx[~masks] == 0).all())
    assert torch.equal(sort_rows(hs.keys())[0], sort_rows(omap.items()[0])[0])
    assert torch.equal(torch.sort(hs.engine.items()[1])[0], torch.arange(hs.size(), device=DEV))


def _run_config2(gpu_ash, num_keys, capacity):
    w = workloads.hashmap_sphere_voxels(num_keys=num_keys, device=DEV)
    hm = gpu_ash.HashMap(3, {"color": 3, "depth": 1}, capacity, DEV)
    hm.insert(w["keys"], {"color": w["color"], "depth": w["depth"]})
    return w, hm


def test_config2_reduced_against_oracle(gpu_ash, oracle):
    num, capacity = 400_000, 600_000
    w, hm = _run_config2(gpu_ash, num, capacity)
    omap = _oracle_map(oracle, 3, capacity)
    stores = {"color": torch.zeros(capacity, 3), "depth": torch.zeros(capacity, 1)}
    omap.insert(w["keys"].cpu(), {"color": w["color"].cpu(), "depth": w["depth"].cpu()}, stores)
    masks, indices, values = hm.find(w["query_keys"], return_values=True)
    idx_cpu, masks_cpu = omap.find(w["query_keys"].cpu())
    assert torch.equal(masks.cpu(), masks_cpu)
    for name in ("color", "depth"):
        assert torch.equal(values[name][masks].cpu(), stores[name][idx_cpu][masks_cpu])
    keys_out, idx_out, vals_out = hm.items(return_values=True)
    k_cpu, i_cpu = omap.items()
    s_gpu = sort_rows(keys_out, vals_out["color"], vals_out["depth"])
    s_cpu = sort_rows(k_cpu, stores["color"][i_cpu], stores["depth"][i_cpu])
    assert all(torch.equal(a, b) for a, b in zip(s_gpu, s_cpu))


def test_config2_full_size_properties(gpu_ash):
    """16 M keys into capacity 24 M: every key found with its own value row,
    exactly the 70 % hit queries found, items() enumerates the key set with a
    bijective index assignment onto [0, 16 M)."""
    num, capacity = 16_000_000, 24_000_000
    w, hm = _run_config2(gpu_ash, num, capacity)
    assert hm.size() == num
    masks, indices, values = hm.find(w["keys"], return_values=True)
    assert bool(masks.all())
    assert torch.equal(values["color"], w["color"]) and torch.equal(values["depth"], w["depth"])
    del values
    qmask, qidx = hm.find(w["query_keys"])
    expect_hit = (w["query_keys"][:, 0] < 50_000)
    assert torch.equal(qmask, expect_hit)
    assert bool((qidx[~qmask] == 0).all())
    keys_out, idx_out = hm.items()
    assert torch.equal(torch.sort(idx_out)[0], torch.arange(num, device=DEV))
    assert torch.equal(
        torch.sort(workloads._pack21(keys_out))[0], torch.sort(workloads._pack21(w["keys"]))[0]
    )
    lookup, found = hm.engine.find(keys_out)
    assert bool(found.all()) and torch.equal(lookup, idx_out)


def test_first_rows_copy_equals_indexing(gpu_ash):
    """ash_gather_rows without indices copies the first n rows of every tensor
    (what a listing in index order asks for): equal to table[:n] for rows of
    4 to 64 bytes, tensors that do not start on a 16-byte boundary, n = 0, 1,
    odd and full."""
    backend = gpu_ash.core.backend
    gen = torch.Generator(device="cpu").manual_seed(5)
    base = torch.rand(7 + 1001 * 16, generator=gen).to(DEV)
    tables = {
        "a": torch.rand(1001, 3, generator=gen).to(DEV),
        "b": torch.rand(1001, 1, generator=gen).to(DEV),
        "c": torch.rand(1001, 4, 4, generator=gen).to(DEV),
        "d": base[3:3 + 1001 * 5].view(1001, 5),          # starts 12 bytes into its storage
        "e": torch.arange(1001 * 2, dtype=torch.int32, device=DEV).view(1001, 2),
    }
    for n in (0, 1, 2, 333, 1000, 1001):
        got = backend.gather_rows(tables, None, first=n)
        for name, table in tables.items():
            assert got[name].shape == (n,) + tuple(table.shape[1:])
            assert torch.equal(got[name], table[:n]), (name, n)
            if n:
                assert got[name].data_ptr() != table.data_ptr()


def test_listing_after_clears_that_left_the_key_log(gpu_ash, oracle):
    """clear() does not touch the log of stored keys while nothing was ever
    erased (a listing then reads no entry beyond the size); what earlier, larger
    fillings left there must be gone once an erase or a load makes listings
    read all of it."""
    dim, capacity = 3, 50_000
    rng = np.random.default_rng(77)

    def fresh(n, shift):
        k = torch.from_numpy(rng.integers(-40, 40, size=(n * 2, dim)).astype(np.int32))
        return (torch.unique(k, dim=0)[:n] + shift).to(DEV)

    engine = gpu_ash.ASHEngine(dim, capacity, DEV)
    for n in (30_001, 12_345, 20_000):           # fillings of different sizes
        engine.insert_keys(fresh(n, 0))
        engine.clear()
    keys = fresh(7_777, 1000)
    engine.insert_keys(keys)
    listed, idx = engine.items()
    assert torch.equal(sort_rows(listed)[0], sort_rows(keys)[0])
    assert torch.equal(torch.sort(idx)[0].cpu(), torch.arange(7_777))
    engine.erase(keys[:1_111])                  # an odd number of keys stays
    listed, idx = engine.items()
    assert torch.equal(sort_rows(listed)[0], sort_rows(keys[1_111:])[0])
    found, mask = engine.find(listed)
    assert bool(mask.all()) and torch.equal(found, idx)
    # once more, ending with a load instead of an erase
    engine.clear()
    engine.insert_keys(fresh(25_000, 0))
    engine.clear()
    engine.insert_keys(keys[:3_333])
    k_saved, i_saved = engine.items()
    other = gpu_ash.ASHEngine(dim, capacity, DEV)
    for n in (9_999, 28_000):
        other.insert_keys(fresh(n, 0))
        other.clear()
    other.insert_keys(fresh(5_001, -1000))
    other.load_state_dict(engine.state_dict())
    listed, idx = other.items()
    got, want = sort_rows(listed, idx), sort_rows(k_saved, i_saved)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    assert other.size() == 3_333


def test_config2_full_size_against_oracle(gpu_ash, oracle):
    """Configuration 2 at its full size against the oracle on the same keys,
    rows and queries: the same masks, the same value rows under the indices
    found, the same key set listed with the same rows."""
    num, capacity = 16_000_000, 24_000_000
    w, hm = _run_config2(gpu_ash, num, capacity)
    omap = _oracle_map(oracle, 3, capacity)
    stores = {"color": torch.zeros(capacity, 3), "depth": torch.zeros(capacity, 1)}
    omap.insert(w["keys"].cpu(), {"color": w["color"].cpu(), "depth": w["depth"].cpu()}, stores)
    assert hm.size() == omap.size() == num
    masks, indices, values = hm.find(w["query_keys"], return_values=True)
    idx_cpu, masks_cpu = omap.find(w["query_keys"].cpu())
    assert torch.equal(masks.cpu(), masks_cpu)
    for name in ("color", "depth"):
        assert torch.equal(values[name][masks].cpu(), stores[name][idx_cpu][masks_cpu])
    del values, masks, indices
    keys_out, idx_out, vals_out = hm.items(return_values=True)
    k_cpu, i_cpu = omap.items()
    s_gpu = sort_rows(keys_out, vals_out["color"], vals_out["depth"])
    s_cpu = sort_rows(k_cpu, stores["color"][i_cpu], stores["depth"][i_cpu])
    assert all(torch.equal(a.cpu(), b) for a, b in zip(s_gpu, s_cpu))


def test_config5_fusion_reduced_against_oracle(gpu_ash, oracle, monkeypatch):
    """Configuration 5 at reduced size (160x120 frames, three views): per frame
    unproject -> activate blocks with a one-block dilation through the hash map
    -> integrate TSDF and weight by cell index.  The same harness runs once on
    the device and once on the CPU with the oracle as backend; the active block
    sets must be identical and the fused cells equal (weights exactly, TSDF to
    fp32 rounding of the projection arithmetic)."""
    import ash.core
    import ash.grid
    import ash.grid_query

    scene = workloads.FusionScene(width=160, height=120)
    frames = []
    for f in (0, 10, 20):
        ext = scene.pose(f)
        depth = scene.depth(ext)
        frames.append((scene.unproject(depth, ext), depth, ext))

    def run(device):
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, 20000, 2, 8, cell_size=0.015, device=device)
        touched = []
        for points, depth, ext in frames:
            touched.append(
                workloads.fuse_frame(
                    grid, points.to(device), depth.to(device), scene.intrinsic.to(device),
                    ext.to(device), trunc=0.04,
                )
            )
        keys, idx = grid.engine.items()
        order = sort_rows(keys, idx)
        return touched, order[0], grid.embeddings.detach().cpu()[order[1]]

    touched_gpu, keys_gpu, cells_gpu = run(DEV)
    with monkeypatch.context() as m:
        for mod in (ash.core, ash.grid, ash.grid_query):
            m.setattr(mod, "backend", oracle)
        touched_cpu, keys_cpu, cells_cpu = run(torch.device("cpu"))
    assert touched_gpu == touched_cpu and len(keys_gpu) > 5000
    assert torch.equal(keys_gpu, keys_cpu)
    # The projection arithmetic (two small matmuls, a division, round()) is done
    # by torch on each device; a pixel coordinate landing on x.5 or a distance
    # landing on the truncation threshold may round differently there, which
    # flips single observations.  Everything the hash map decides (which blocks
    # exist, which row every cell lives in) is exact.
    same = cells_gpu[..., 1] == cells_cpu[..., 1]
    assert float((~same).float().mean()) < 5e-4
    assert torch.allclose(cells_gpu[..., 0][same], cells_cpu[..., 0][same], rtol=1e-3, atol=2e-4)
    assert float(cells_gpu[..., 1].sum()) > 1e5


@pytest.mark.parametrize("policy", ["auto", "always"])
def test_table_larger_than_4_gib(gpu_ash, monkeypatch, policy):
    """A bucket array of 6.4 GB (capacity 300 M): every byte offset into the
    table needs more than 32 bits.  Keys spread over the whole array are
    inserted (per key, and through the streaming path where it applies), found,
    listed and erased."""
    monkeypatch.setattr(gpu_ash.common, "BULK_INSERT", policy)
    capacity = 300_000_000
    hm = gpu_ash.HashMap(3, 1, capacity, DEV)
    table_bytes = hm.engine.backend._table.numel()
    assert table_bytes > 5 * 2**30
    g = torch.Generator().manual_seed(97)
    keys = torch.unique(torch.randint(-100_000, 100_000, (6_000_000, 3), generator=g,
                                      dtype=torch.int32), dim=0).to(DEV)
    n = len(keys)
    values = torch.arange(n, device=DEV, dtype=torch.float32).view(-1, 1)
    hm.insert(keys, values)
    assert hm.size() == n
    masks, indices, got = hm.find(keys, return_values=True)
    assert bool(masks.all()) and torch.equal(got, values)
    assert int(indices.min()) == 0 and int(indices.max()) == n - 1
    assert len(torch.unique(indices)) == n
    shifted = keys + torch.tensor([[250_000, 0, 0]], dtype=torch.int32, device=DEV)
    masks_absent, _ = hm.find(shifted)
    assert not bool(masks_absent.any())
    listed, listed_idx = hm.items()
    assert len(listed) == n
    assert torch.equal(sort_rows(listed, listed_idx)[0], sort_rows(keys, indices)[0])
    hm.erase(keys[: n // 2].contiguous())
    assert hm.size() == n - n // 2
    masks_after, _ = hm.find(keys)
    assert not bool(masks_after[: n // 2].any()) and bool(masks_after[n // 2:].all())
    hm.clear()
    assert hm.size() == 0 and not bool(hm.find(keys[:1000].contiguous())[0].any())
    del hm
    torch.cuda.empty_cache()


def test_heap_starts_over_after_clear(gpu_ash):
    """clear() gives the indices back in their first order: the heap array is
    rewritten when an erase or a load has written to it and left alone when
    nothing has; either way the next n distinct keys get the indices 0..n-1."""
    engine = gpu_ash.ASHEngine(3, 6000, DEV)
    g = torch.Generator().manual_seed(99)
    keys = torch.unique(torch.randint(-40, 40, (5000, 3), generator=g, dtype=torch.int32), dim=0).to(DEV)
    n = len(keys)

    def fresh_indices():
        engine.insert_keys(keys)
        indices, masks = engine.find(keys)
        assert bool(masks.all())
        return torch.sort(indices)[0]

    assert torch.equal(fresh_indices(), torch.arange(n, device=DEV))
    engine.clear()                                   # nothing wrote to the heap
    assert torch.equal(fresh_indices(), torch.arange(n, device=DEV))
    engine.erase(keys[::3].contiguous())             # freed indices go back in another order
    engine.insert_keys(keys[::3].contiguous())
    engine.clear()
    assert torch.equal(fresh_indices(), torch.arange(n, device=DEV))
    engine.erase(keys[::2].contiguous())             # the saved heap is out of order
    state = {k: v.clone() for k, v in engine.state_dict().items()}
    engine.clear()                                   # in order again, and marked so
    engine.load_state_dict(state)                    # the heap comes from the caller
    engine.clear()
    half = keys[: n // 2].contiguous()
    engine.insert_keys(half)
    indices, masks = engine.find(half)
    assert bool(masks.all())
    assert torch.equal(torch.sort(indices)[0], torch.arange(len(half), device=DEV))

"""GPU tests of the entry points that keep a table in order by themselves
(ash_map_insert_auto, ash_map_erase_auto, ash_map_counters) through the raw C
ABI -- what a binding with the reference's nine methods
(ash/src/pybind.cpp:9-23) calls -- against the oracle, of what the handle knows
of the counters while other calls go past it, of states a load has to refuse,
and of inserts captured into a HIP graph."""
import ctypes
import warnings

import numpy as np
import pytest
import torch

import workloads
from helpers import sort_rows
from test_gpu_hash import _assert_same_map, _oracle_map

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
AUTO, ALWAYS, NEVER = 0, 1, 2
NEEDS_GENERAL = 2


class RawMap:
    """A table driven through the C ABI alone: torch only owns the memory."""

    def __init__(self, ash, dim, capacity):
        self.lib = ash.core.backend.lib
        self.dim, self.capacity = dim, capacity
        self.heap = torch.arange(capacity, dtype=torch.int32, device=DEV)
        tb, gb = ctypes.c_int64(0), ctypes.c_int64(0)
        assert self.lib.ash_map_workspace_bytes(dim, capacity, ctypes.byref(tb), ctypes.byref(gb)) == 0
        self.table = torch.empty(tb.value, dtype=torch.uint8, device=DEV)
        self.general_bytes, self.general = gb.value, None
        self.stream = torch.cuda.current_stream(DEV).cuda_stream
        self.handle = ctypes.c_void_p()
        assert self.lib.ash_map_create(dim, capacity, self.heap.data_ptr(), self.table.data_ptr(),
                                       tb.value, 0, self.stream, ctypes.byref(self.handle)) == 0
        self.landing = torch.zeros(16, dtype=torch.int32, pin_memory=True)
        self.check(self.lib.ash_map_set_staging(self.handle, self.landing.data_ptr()))
        self.attached = 0

    def __del__(self):
        self.lib.ash_map_destroy(self.handle)

    def check(self, rc):
        assert rc == 0, self.lib.ash_last_error().decode()

    def insert(self, keys, policy=AUTO):
        """The whole binding of `insert_keys`: size the scratch, call, attach
        the second region and call again if asked to."""
        keys = keys.to(DEV).contiguous()
        for _ in range(2):
            nbytes = ctypes.c_int64(0)
            self.check(self.lib.ash_map_insert_scratch_bytes(
                self.handle, len(keys), 0, None, policy, ctypes.byref(nbytes)))
            scratch = torch.empty(max(nbytes.value, 1), dtype=torch.uint8, device=DEV)
            rc = self.lib.ash_map_insert_auto(
                self.handle, keys.data_ptr(), len(keys), 0, None, None, None, scratch.data_ptr(),
                nbytes.value, policy, None, self.stream)
            if rc != NEEDS_GENERAL:
                return self.check(rc)
            self.general = torch.empty(self.general_bytes, dtype=torch.uint8, device=DEV)
            self.check(self.lib.ash_map_attach_general(self.handle, self.general.data_ptr(),
                                                       self.general_bytes, self.stream))
            self.attached += 1
        raise AssertionError("asked for the second region twice")

    def erase(self, keys, policy=AUTO):
        keys = keys.to(DEV).contiguous()
        nbytes = ctypes.c_int64(0)
        self.check(self.lib.ash_map_erase_scratch_bytes(self.handle, len(keys), policy,
                                                        ctypes.byref(nbytes)))
        scratch = torch.empty(max(nbytes.value, 1), dtype=torch.uint8, device=DEV)
        self.check(self.lib.ash_map_erase_auto(self.handle, keys.data_ptr(), len(keys),
                                               scratch.data_ptr(), nbytes.value, policy, self.stream))

    def counters(self):
        out = (ctypes.c_int64 * 7)()
        self.check(self.lib.ash_map_counters(self.handle, None, out, self.stream))
        return dict(zip(("size", "dropped", "tombstones", "exotic", "refused", "touched", "general"),
                        out))

    def fresh_size(self):
        out = (ctypes.c_int64 * 5)()
        self.check(self.lib.ash_map_status(self.handle, out, self.stream))
        return out[0]

    def find(self, keys):
        keys = keys.to(DEV).contiguous()
        idx = torch.empty(len(keys), dtype=torch.int64, device=DEV)
        mask = torch.empty(len(keys), dtype=torch.bool, device=DEV)
        self.check(self.lib.ash_map_find(self.handle, keys.data_ptr(), len(keys), idx.data_ptr(),
                                         mask.data_ptr(), self.stream))
        return idx, mask

    def items(self):
        n = self.counters()["size"]
        keys = torch.empty((n, self.dim), dtype=torch.int32, device=DEV)
        idx = torch.empty(n, dtype=torch.int64, device=DEV)
        self.check(self.lib.ash_map_items(self.handle, keys.data_ptr(), idx.data_ptr(), n, self.stream))
        return keys, idx


def _keys(rng, n, span, dim=3):
    return torch.from_numpy(rng.integers(-span, span, size=(n, dim)).astype(np.int32))


def _same(raw, omap, probe):
    assert raw.counters()["size"] == raw.fresh_size() == omap.size()
    keys, idx = raw.items()
    assert torch.equal(sort_rows(keys)[0], sort_rows(omap.items()[0])[0])
    assert len(torch.unique(idx)) == len(idx)
    _, mask = raw.find(probe)
    assert torch.equal(mask.cpu(), omap.find(probe)[1])


@pytest.mark.parametrize("policy", [AUTO, ALWAYS, NEVER])
def test_two_calls_per_insert_keep_the_table_in_order(gpu_ash, oracle, policy):
    """Insert / erase cycles at full load through ash_map_insert_auto and
    ash_map_erase_auto only: the table is re-placed when tombstones pile up, a
    key that does not fit the packed code makes the call ask for the second
    region once, and the handle's counters equal the device's after every call."""
    capacity = 60_000
    rng = np.random.default_rng(4100 + policy)
    raw, omap = RawMap(gpu_ash, 3, capacity), _oracle_map(oracle, 3, capacity)
    pool = torch.unique(_keys(rng, 400_000, 60), dim=0)
    pool = pool[torch.from_numpy(rng.permutation(len(pool)))]
    live = pool[:capacity]
    raw.insert(live, policy)
    omap.insert_keys(live)
    pending = gpu_ash.core.backend.lib.ash_map_counters_pending(raw.handle)
    assert pending == (1 if policy == ALWAYS else 0)     # 60 000 keys: streaming only when forced
    _same(raw, omap, pool[: capacity + 3000])
    cursor = capacity
    for cycle in range(10):
        out = live[torch.from_numpy(rng.permutation(capacity)[: capacity // 3])]
        raw.erase(out, policy)
        omap.erase(out)
        new = pool[cursor: cursor + capacity // 3]
        cursor += capacity // 3
        raw.insert(new, policy)
        omap.insert_keys(new)
        live, _ = omap.items()
        _same(raw, omap, pool[: cursor + 2000])
    assert raw.counters()["tombstones"] < capacity // 2      # the upkeep has run
    assert raw.attached == 0
    odd = torch.tensor([[2**30, 1, -(2**30)], [5, 2**29, 7]], dtype=torch.int32)
    raw.erase(live[:100], policy)
    omap.erase(live[:100])
    batch = torch.cat([pool[cursor: cursor + 50], odd])
    raw.insert(batch, policy)
    omap.insert_keys(batch)
    assert raw.attached == 1 and raw.counters()["general"] == 2
    _same(raw, omap, torch.cat([batch, pool[:5000]]))
    # with the second region in use the entries are re-placed through scratch
    for cycle in range(4):
        live, _ = omap.items()
        out = live[torch.from_numpy(rng.permutation(len(live))[: capacity // 2])]
        raw.erase(out, policy)
        omap.erase(out)
        new = pool[cursor: cursor + capacity // 2]
        cursor += capacity // 2
        raw.insert(torch.cat([new, odd]), policy)
        omap.insert_keys(torch.cat([new, odd]))
        _same(raw, omap, torch.cat([odd, pool[: 4000]]))


def test_first_filling_of_a_new_table_streams(gpu_ash, oracle):
    """A table that has not been used since it was made (or emptied) still has
    its bucket array to fill: the managed insert then streams from 2^18 keys,
    where a table in use takes the per-key kernel at this size -- and either
    way the map is the oracle's.  Duplicates inside the batch included."""
    rng = np.random.default_rng(31)
    capacity, n = 700_000, 300_000
    raw, omap = RawMap(gpu_ash, 3, capacity), _oracle_map(oracle, 3, capacity)
    nbytes = ctypes.c_int64(-1)

    def wanted(count):
        raw.check(raw.lib.ash_map_insert_scratch_bytes(raw.handle, count, 0, None, AUTO,
                                                       ctypes.byref(nbytes)))
        return nbytes.value

    first = _keys(rng, n, 60)
    first[1::3] = first[::3][: len(first[1::3])]        # a third of the batch repeats another third
    probe = torch.cat([first[::7], _keys(rng, 50_000, 90)])
    assert wanted(n) > 0                                  # new table: the streaming passes
    assert wanted((1 << 18) - 1) == 0 and wanted(40 * capacity) == 0
    raw.insert(first)
    omap.insert_keys(first)
    _same(raw, omap, probe)
    assert wanted(n) == 0                                 # a table in use, and small: per key
    second = _keys(rng, n, 75)
    raw.insert(second)
    omap.insert_keys(second)
    _same(raw, omap, probe)
    raw.check(raw.lib.ash_map_clear(raw.handle, raw.stream))
    omap.clear()
    assert wanted(n) > 0                                  # emptied and not used since: streams again
    raw.insert(second)
    omap.insert_keys(second)
    _same(raw, omap, probe)


def test_the_handle_follows_calls_that_go_past_the_managed_entries(gpu_ash):
    """The size the handle reports is the device's whoever made the launches:
    the fine-grained entries invalidate what the handle knows."""
    rng = np.random.default_rng(4200)
    raw = RawMap(gpu_ash, 3, 50_000)
    lib = raw.lib
    keys = torch.unique(_keys(rng, 40_000, 40), dim=0).to(DEV)
    known = ctypes.c_int64(-1)
    assert lib.ash_map_known_size(raw.handle, ctypes.byref(known)) == 1 and known.value == 0
    raw.check(lib.ash_map_insert_keys(raw.handle, keys.data_ptr(), len(keys), raw.stream))
    assert lib.ash_map_known_size(raw.handle, ctypes.byref(known)) == 0      # would need the device
    assert raw.counters()["size"] == len(keys)
    assert lib.ash_map_known_size(raw.handle, ctypes.byref(known)) == 1 and known.value == len(keys)
    raw.check(lib.ash_map_erase(raw.handle, keys.data_ptr(), 1000, raw.stream))
    assert raw.counters()["size"] == len(keys) - 1000
    raw.check(lib.ash_map_clear(raw.handle, raw.stream))
    assert lib.ash_map_known_size(raw.handle, ctypes.byref(known)) == 1 and known.value == 0
    raw.insert(keys, ALWAYS)                       # counters queued behind the streaming insert
    assert lib.ash_map_counters_pending(raw.handle) == 1
    assert raw.counters()["size"] == len(keys) and lib.ash_map_counters_pending(raw.handle) == 0


def test_listing_stays_in_index_order_with_an_empty_second_region(gpu_ash):
    """A second region that holds no entry (attached ahead of time, as the
    frames without read-back do) does not switch the dense listing off; one
    entry in it does, and erasing that entry does not bring it back (the heap
    has been written to)."""
    hm = gpu_ash.HashMap(3, {"v": 2}, 30_000, DEV)
    backend = hm.engine.backend
    g = torch.Generator().manual_seed(4300)
    keys = torch.unique(torch.randint(-30, 30, (20_000, 3), generator=g, dtype=torch.int32), dim=0).to(DEV)
    backend._attach_general()
    hm.insert(keys, {"v": torch.rand(len(keys), 2, device=DEV)})
    k, i, v = hm.items(return_indices=True, return_values=True)
    assert backend.last_items_in_index_order and torch.equal(i, torch.arange(len(i), device=DEV))
    assert backend.counters()["general_live"] == 0 and torch.equal(v["v"], hm.v[i])
    odd = torch.tensor([[2**30, 0, 0]], dtype=torch.int32, device=DEV)
    hm.insert(odd, {"v": torch.ones(1, 2, device=DEV)})
    k, i, v = hm.items(return_indices=True, return_values=True)
    assert not backend.last_items_in_index_order and backend.counters()["general_live"] == 1
    assert len(k) == len(keys) + 1 and torch.equal(v["v"], hm.v[i])
    assert torch.equal(sort_rows(k)[0], sort_rows(torch.cat([keys, odd]))[0])
    hm.erase(odd)
    assert backend.counters()["general_live"] == 0
    k, i = hm.items(return_indices=True)
    assert not backend.last_items_in_index_order and len(k) == len(keys)


def test_second_region_of_the_callers_size(gpu_ash, oracle):
    """ash_map_attach_general takes a region smaller than what the capacity
    would need (attached ahead of time for keys that are not expected): keys
    that do not fit the packed code live there like in a full-sized one, and
    when it is full further ones are refused and counted, like keys that find
    the map full."""
    rng = np.random.default_rng(4500)
    wide = torch.from_numpy(rng.integers(2**22, 2**30, size=(300, 3)).astype(np.int32))
    wide = torch.unique(wide, dim=0)
    engine = gpu_ash.ASHEngine(3, 100_000, DEV)
    engine.backend._attach_general(just_in_case=True)
    assert engine.backend._general.numel() == 20 << 16 < engine.backend._general_bytes
    omap = _oracle_map(oracle, 3, 100_000)
    batch = torch.cat([_keys(rng, 20_000, 40), wide])
    engine.insert_keys(batch.to(DEV))
    omap.insert_keys(batch)
    _assert_same_map(engine, omap, torch.cat([wide, wide + 1, batch[:3000]]).to(DEV))
    assert engine.backend.counters()["general_live"] == len(wide)
    engine.erase(wide[:100].to(DEV))
    omap.erase(wide[:100])
    _assert_same_map(engine, omap, wide.to(DEV))
    # the smallest region: 64 slots
    raw = RawMap(gpu_ash, 3, 10_000)
    raw.general = torch.empty(64 * 20, dtype=torch.uint8, device=DEV)
    raw.check(raw.lib.ash_map_attach_general(raw.handle, raw.general.data_ptr(), 64 * 20, raw.stream))
    raw.insert(torch.cat([_keys(rng, 2000, 30), wide]), NEVER)
    c = raw.counters()
    assert c["general"] <= 64 and c["general"] + c["dropped"] == len(wide)
    _, mask = raw.find(wide)
    assert int(mask.sum()) == c["general"]
    assert raw.lib.ash_map_attach_general(raw.handle, raw.general.data_ptr(), 63 * 20, raw.stream) != 0


def test_states_that_address_no_row_are_refused(gpu_ash):
    """A state dict whose indices or heap entries lie outside 0 .. capacity-1
    would make later calls write outside the value rows and the key log
    (ash/src/hashmap_gpu.cuh:407-450 stores what it is given): the load is
    refused and the map left empty and usable."""
    capacity = 5000
    engine = gpu_ash.ASHEngine(3, capacity, DEV)
    keys = torch.unique(torch.randint(-20, 20, (3000, 3), dtype=torch.int32), dim=0).to(DEV)
    engine.insert_keys(keys)
    good = {k: v.clone() for k, v in engine.state_dict().items()}
    for what in ("index too large", "negative index", "heap entry"):
        state = {k: v.clone() for k, v in good.items()}
        if what == "index too large":
            state["_indices"][7] = capacity
        elif what == "negative index":
            state["_indices"][11] = -3
        else:
            state["_heap"][capacity - 1] = capacity + 5
        other = gpu_ash.ASHEngine(3, capacity, DEV)
        with pytest.raises(RuntimeError, match="refused"):
            other.load_state_dict(state)
        assert other.size() == 0
        other.insert_keys(keys[:100])          # still usable (its own heap is in place again)
        assert other.size() == 100 and bool(other.find(keys[:100])[1].all())
    other = gpu_ash.ASHEngine(3, capacity, DEV)
    other.load_state_dict(good)
    assert other.size() == len(keys) and bool(other.find(keys)[1].all())


def test_rows_of_indices_outside_the_table_read_as_zero(gpu_ash):
    """ash_gather_rows gives a zero row for an index outside the source table
    where torch's `values[name][indices]` (ash/hashmap.py:87-95) raises or wraps
    a negative index: protection against a fault, documented as a divergence."""
    backend = gpu_ash.core.backend
    table = {"v": torch.arange(30, dtype=torch.float32, device=DEV).view(10, 3) + 1}
    idx = torch.tensor([0, 9, 10, -1, 3, 10**9], device=DEV)
    got = backend.gather_rows(table, idx)["v"]
    inside = (idx >= 0) & (idx < 10)
    assert torch.equal(got[inside], table["v"][idx[inside]])
    assert float(got[~inside].abs().sum()) == 0.0


def test_insert_and_find_replay_in_a_hip_graph(gpu_ash, oracle):
    """ash_map_insert_auto on a stream that is being captured only queues
    launches: insert + find are recorded once and replayed with new keys in the
    same buffers, per-key and streaming, and equal the oracle after every replay
    (with eager calls and synchronisations between the replays).  From the
    capture on the handle trusts nothing it remembers of the map."""
    capacity, n = 200_000, 40_000
    rng = np.random.default_rng(4400)
    for policy in ("never", "always"):
        engine = gpu_ash.ASHEngine(3, capacity, DEV)
        backend = engine.backend
        omap = _oracle_map(oracle, 3, capacity)
        first = torch.unique(_keys(rng, 30_000, 50), dim=0)
        engine.insert_keys(first.to(DEV))         # eager: the table is settled, buffers exist
        omap.insert_keys(first)
        keys = torch.zeros((n, 3), dtype=torch.int32, device=DEV)
        probe = torch.zeros((n, 3), dtype=torch.int32, device=DEV)
        idx = torch.empty(n, dtype=torch.int64, device=DEV)
        mask = torch.empty(n, dtype=torch.bool, device=DEV)
        pol = {"never": NEVER, "always": ALWAYS}[policy]
        nbytes = ctypes.c_int64(0)
        lib, handle = backend._lib, backend._handle
        assert lib.ash_map_insert_scratch_bytes(handle, n, 0, None, pol, ctypes.byref(nbytes)) == 0
        scratch = torch.empty(max(nbytes.value, 256), dtype=torch.uint8, device=DEV)
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                rc = lib.ash_map_insert_auto(handle, keys.data_ptr(), n, 0, None, None, None,
                                             scratch.data_ptr(), nbytes.value, pol, None,
                                             side.cuda_stream)
                assert rc == 0, lib.ash_last_error().decode()
                assert lib.ash_map_find(handle, probe.data_ptr(), n, idx.data_ptr(),
                                        mask.data_ptr(), side.cuda_stream) == 0
                # a read of the counters would have to wait for the stream: it is
                # refused, by name, and leaves the capture as it is
                size = ctypes.c_int64(-1)
                assert lib.ash_map_size(handle, ctypes.byref(size), side.cuda_stream) != 0
                assert "being captured" in lib.ash_last_error().decode()
        torch.cuda.synchronize()
        assert engine.size() == omap.size()      # the capture itself inserted nothing
        for replay in range(3):
            batch = _keys(rng, n, 52 + replay)
            # a key that does not fit the packed code: the captured launches know
            # of no second region, so it is counted and not stored
            batch[-1] = torch.tensor([2**30, replay, 0])
            ask = torch.cat([batch[: n // 2], _keys(rng, n - n // 2, 60)])
            keys.copy_(batch.to(DEV))
            probe.copy_(ask.to(DEV))
            graph.replay()
            torch.cuda.synchronize()
            omap.insert_keys(batch[:-1])
            _, mask_ref = omap.find(ask)
            assert torch.equal(mask.cpu(), mask_ref), (policy, replay)
            assert bool((idx[~mask] == 0).all())
            assert backend.status()["exotic_pending"] == 1
            # an eager call between the replays: the first one attaches the
            # second region on the waiting key's account, later ones count the
            # key of the replay before them as refused
            extra = _keys(rng, 500, 70)
            with warnings.catch_warnings():
                warnings.simplefilter("ignore")
                engine.insert_keys(extra.to(DEV))
            omap.insert_keys(extra)
            _assert_same_map(engine, omap, ask.to(DEV))
            status = backend.status()
            assert status["exotic_pending"] == 0 and status["dropped"] == replay
        assert engine.size() == omap.size()


def test_fusion_frames_replay_in_a_hip_graph(gpu_ash):
    """One whole frame of ash.fusion.fuse_frame(count_blocks=False) --
    activation, listing, integration -- captured once and replayed for other
    frames by rewriting its input buffers: block sets and embedding rows equal
    the eager frames bit for bit after every replay."""
    scene = workloads.FusionScene(width=320, height=240)
    intrinsic = scene.intrinsic.to(DEV)
    frames = []
    for f in (0, 9, 18, 27):
        ext = scene.pose(f)
        depth = scene.depth(ext)
        frames.append((scene.unproject(depth, ext), depth, ext))
    most = max(len(p) for p, _, _ in frames)

    def padded(points):
        # (a graph has fixed shapes: frames are padded with copies of their last point)
        pad = points[-1:].expand(most - len(points), 3)
        return torch.cat([points, pad]).to(DEV)

    def fresh():
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, 30_000, 2, 8, cell_size=0.015, device=DEV)
        with torch.no_grad():
            grid.embeddings.zero_()
        return grid

    def snapshot(grid):
        keys, idx = sort_rows(*grid.engine.items())
        return keys, grid.embeddings.detach()[idx.to(DEV)].cpu()

    eager = fresh()
    expected = []
    for p, d, e in frames:
        gpu_ash.fusion.fuse_frame(eager, padded(p), d.to(DEV), intrinsic, e.to(DEV), 0.04, 6.0,
                                  count_blocks=False)
        expected.append(snapshot(eager))

    grid = fresh()
    points = padded(frames[0][0]).clone()
    depth, ext = frames[0][1].to(DEV).clone(), frames[0][2].to(DEV).clone()
    # the first frame runs eagerly: buffers, second region and the table's fill exist afterwards
    gpu_ash.fusion.fuse_frame(grid, points, depth, intrinsic, ext, 0.04, 6.0, count_blocks=False)
    assert all(torch.equal(a, b) for a, b in zip(snapshot(grid), expected[0]))
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        gpu_ash.fusion.fuse_frame(grid, points, depth, intrinsic, ext, 0.04, 6.0, count_blocks=False)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(snapshot(grid), expected[0]))   # captured, not run
    for (p, d, e), want in zip(frames[1:], expected[1:]):
        points.copy_(padded(p))
        depth.copy_(d.to(DEV))
        ext.copy_(e.to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        got = snapshot(grid)
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    assert grid.engine.size() == eager.engine.size() > 1000

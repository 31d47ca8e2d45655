"""Host-side logic of the package, run without a GPU by wiring the Python
layer to the CPU oracle (fixture `cpu_ash`): neighbour tables against closed
forms and brute force, the reference's unit tests of engine / set / map /
embedding / grid (unittests/*.py) re-expressed, state-dict layout, warnings."""
import itertools
import os
import warnings

import pytest
import torch

from helpers import assert_is_bijection_into, sort_rows

CPU = torch.device("cpu")


def _tiled_keys(dim, num, seed=0):
    g = torch.Generator().manual_seed(seed)
    keys = torch.arange(num, dtype=torch.int32).view(-1, 1).tile((1, dim))
    return keys[torch.randperm(num, generator=g)]


# ------------------------------------------------------------ neighbour offsets
@pytest.mark.parametrize("dim", [1, 2, 3])
@pytest.mark.parametrize("radius", [1, 2, 3])
@pytest.mark.parametrize("bidirectional", [False, True])
def test_neighbor_offsets_closed_form(dim, radius, bidirectional):
    """ash/grid_nns.py:5-47: first component fastest, offset2idx is the inverse."""
    from ash import enumerate_neighbor_coord_offsets

    offsets, offset2idx = enumerate_neighbor_coord_offsets(dim, radius, bidirectional, CPU)
    rng = range(-radius, radius + 1) if bidirectional else range(0, radius + 1)
    # itertools.product varies the LAST factor fastest; reverse to make x fastest
    expected = [tuple(reversed(p)) for p in itertools.product(rng, repeat=dim)]
    assert offsets.dtype == torch.int64
    assert [tuple(r) for r in offsets.tolist()] == expected
    assert torch.equal(offset2idx(offsets), torch.arange(len(expected)))


def test_neighbor_offsets_interpolation_window_is_the_bit_pattern():
    from ash import enumerate_neighbor_coord_offsets

    offsets, _ = enumerate_neighbor_coord_offsets(3, 1, False, CPU)
    for k in range(8):
        assert offsets[k].tolist() == [k & 1, (k >> 1) & 1, (k >> 2) & 1]


# ------------------------------------------------------------------ cell tables
@pytest.mark.parametrize("grid_dim", [1, 2, 3, 4, 8])
def test_cell_neighbor_tables_brute_force(cpu_ash, grid_dim):
    """ash/grid.py:525-564 for the interpolation window."""
    grid = cpu_ash.SparseDenseGrid(3, 4, 1, grid_dim, device=CPU)
    g = grid_dim
    assert grid.lut_cell_nb2cell_idx.shape == (g**3, 8) and grid.lut_cell_nb2cell_idx.dtype == torch.int64
    for cell in range(g**3):
        cx, cy, cz = cell % g, (cell // g) % g, cell // (g * g)
        assert grid.cell_coords[cell].tolist() == [cx, cy, cz]
        for k in range(8):
            nx, ny, nz = cx + (k & 1), cy + ((k >> 1) & 1), cz + ((k >> 2) & 1)
            want_cell = (nx % g) + g * (ny % g) + g * g * (nz % g)
            want_nb = (nx // g) + 2 * (ny // g) + 4 * (nz // g)
            assert grid.lut_cell_nb2cell_idx[cell, k].item() == want_cell
            assert grid.lut_cell_nb2grid_nb[cell, k].item() == want_nb


def test_cell_neighbor_tables_wide_window(cpu_ash):
    """Bidirectional radius-3 window on 2^3 cells (the convolution tables of
    the reference): block offsets up to +-2."""
    grid = cpu_ash.SparseDenseGrid(3, 4, 1, 2, device=CPU)
    nb, cell = grid.construct_cell_neighbor_lut(radius=3, bidirectional=True)
    assert nb.shape == (8, 343) and cell.shape == (8, 343)
    k = 0
    for oz in range(-3, 4):
        for oy in range(-3, 4):
            for ox in range(-3, 4):
                p = (1 + ox, 0 + oy, 1 + oz)  # neighbours of cell (1,0,1) = index 5
                want_cell = (p[0] % 2) + 2 * (p[1] % 2) + 4 * (p[2] % 2)
                b = [c // 2 + 2 for c in p]  # block radius 2 -> pad 2, width 5
                assert cell[5, k].item() == want_cell
                assert nb[5, k].item() == b[0] + 5 * b[1] + 25 * b[2]
                k += 1


def test_linearize_round_trip(cpu_ash):
    for g in (3, 4, 8, 16):
        grid = cpu_ash.SparseDenseGrid(3, 4, 1, g, device=CPU)
        idx = torch.randint(g**3, (100,))
        coords = grid._delinearize_cell_indices(idx)
        assert coords.dtype == torch.int32
        assert torch.equal(grid._linearize_cell_coords(coords), idx)


# ----------------------------------------------------------------- block tables
def test_grid_neighbor_table(cpu_ash):
    """ash/grid.py:566-617: rows of inactive blocks and missing neighbours are -1."""
    grid = cpu_ash.SparseDenseGrid(3, 16, 1, 2, device=CPU)
    blocks = torch.tensor([[0, 0, 0], [1, 0, 0], [0, 1, 0], [5, 5, 5]], dtype=torch.int32)
    grid.engine.insert_keys(blocks)
    coords, lut = grid.construct_grid_neighbor_lut(radius=1, bidirectional=False)
    idx, mask = grid.engine.find(blocks)
    assert mask.all()
    assert coords.dtype == torch.int32 and lut.dtype == torch.int64 and lut.shape == (16, 8)
    inactive = torch.ones(16, dtype=torch.bool)
    inactive[idx] = False
    assert (lut[inactive] == -1).all() and (coords[inactive] == -1).all()
    a, b, c, far = idx.tolist()
    assert coords[a].tolist() == [0, 0, 0] and coords[far].tolist() == [5, 5, 5]
    assert lut[a].tolist() == [a, b, c, -1, -1, -1, -1, -1]
    assert lut[b].tolist() == [b, -1, -1, -1, -1, -1, -1, -1]
    assert lut[far].tolist() == [far] + [-1] * 7
    # an empty grid gives all -1
    empty = cpu_ash.SparseDenseGrid(3, 4, 1, 2, device=CPU)
    coords, lut = empty.construct_grid_neighbor_lut(1, False)
    assert (lut == -1).all() and (coords == -1).all()


# ------------------------------------------------------- grid: reference tests
@pytest.mark.parametrize("embedding_dim,grid_dim", [(1, 2), (8, 4), (16, 8)])
def test_grid_items_and_query(cpu_ash, embedding_dim, grid_dim):
    """unittests/test_sparsedense_grid.py:79-137."""
    grid = cpu_ash.SparseDenseGrid(3, 1000, embedding_dim, grid_dim, device=CPU)
    assert grid.embeddings.shape == (1000, grid_dim**3, embedding_dim)
    torch.nn.init.uniform_(grid.embeddings, -1, 1)
    blocks = grid_dim * torch.arange(-1, 2, dtype=torch.int).view(-1, 1).tile((1, 3))
    gc, cc, gi, ci = grid.spatial_init_(blocks, dilation=0)
    assert gc.shape == (3, 1, 3) and cc.shape == (1, grid_dim**3, 3)
    gc, cc, gi, ci = grid.items()
    coords = (gc * grid_dim + cc).view(-1, 3)
    assert grid.embeddings[gi, ci].shape == (3, grid_dim**3, embedding_dim)
    q_gi, q_ci, offsets, masks = grid.query(coords)
    assert q_gi.shape == (3 * grid_dim**3,) and q_ci.shape == q_gi.shape
    assert torch.equal(offsets, torch.zeros_like(offsets)) and masks.all()
    feats, masks = grid(coords, interpolation="nearest")
    assert torch.equal(feats, grid.embeddings[q_gi, q_ci])
    feats.sum().backward()
    assert grid.embeddings.grad is not None
    with pytest.raises(ValueError):
        grid(coords.float(), interpolation="cubic")


def test_query_rounding_edge(cpu_ash):
    """A tiny negative coordinate makes x - floor(x/G)*G round to exactly G in
    fp32; it must resolve to cell 0 of the next block, never to a cell index
    out of range (the reference would read its tables out of bounds there)."""
    grid = cpu_ash.SparseDenseGrid(3, 64, 1, 8, device=CPU)
    r = torch.arange(-1, 1, dtype=torch.int32)
    grid.engine.insert_keys(torch.stack(torch.meshgrid(r, r, r, indexing="ij"), -1).view(-1, 3))
    x = torch.tensor([[-1e-9, 3.0, 3.0], [-1e-9, -1e-9, -1e-9], [7.9999995, 0.0, 0.0]])
    gi, ci, off, masks = grid.query(x)
    assert masks.all()
    assert int(ci.max()) < 512 and int(ci.min()) >= 0
    assert float(off.min()) >= 0.0 and float(off.max()) < 1.0
    k0, _ = grid.engine.find(torch.tensor([[0, 0, 0]], dtype=torch.int32))
    assert gi[1].item() == k0.item() and ci[1].item() == 0


@pytest.mark.parametrize("grid_dim", [1, 3, 8])
def test_query_decomposition_invariants(cpu_ash, grid_dim):
    """For every position, also one ulp below block boundaries:
    block * G + cell + offset reproduces x, cell in [0, G)^3, offset in [0, 1)."""
    grid = cpu_ash.SparseDenseGrid(3, 4, 1, grid_dim, device=CPU)
    g = torch.Generator().manual_seed(grid_dim)
    ints = torch.randint(-40 * grid_dim, 40 * grid_dim + 1, (4000, 3), generator=g).float()
    below = torch.nextafter(ints, torch.full_like(ints, -1e9))
    above = torch.nextafter(ints, torch.full_like(ints, 1e9))
    rand = (torch.rand(4000, 3, generator=g) * 2 - 1) * 40 * grid_dim
    x = torch.cat([ints, below, above, rand])
    _, ci, off, _ = grid.query(x)
    assert int(ci.min()) >= 0 and int(ci.max()) < grid_dim**3
    assert float(off.min()) >= 0.0 and float(off.max()) < 1.0
    cells = grid._delinearize_cell_indices(ci).double()
    within = cells + off.double()
    block = torch.round((x.double() - within) / grid_dim)
    assert torch.allclose(block * grid_dim + within, x.double(), rtol=0, atol=1e-4)


def test_spatial_init_dilation_and_bounds(cpu_ash):
    """ash/grid.py:121-159,850-852: dilation windows, out-of-box blocks dropped,
    few points with a wide window (more unique blocks than points)."""
    grid = cpu_ash.BoundedSparseDenseGrid(
        3, 4096, 1, grid_dim=4, sparse_grid_dim=8,
        bbox_min=torch.zeros(3), bbox_max=torch.ones(3), device=CPU,
    )
    assert abs(grid.cell_size - 1.0 / 31) < 1e-7
    pts = torch.tensor([[0.01, 0.01, 0.01], [0.99, 0.99, 0.99], [5.0, 5.0, 5.0]])
    gc, cc, gi, ci = grid.spatial_init_(pts, dilation=1, bidirectional=True)
    blocks = set(map(tuple, gc.view(-1, 3).tolist()))
    want = {(x, y, z) for x in (0, 1) for y in (0, 1) for z in (0, 1)} | {
        (x, y, z) for x in (6, 7) for y in (6, 7) for z in (6, 7)
    }
    assert blocks == want and grid.engine.size() == 16
    assert_is_bijection_into(gi.view(-1), 4096)
    world = grid.cell_to_world(gc, cc)
    assert world.shape == (16 * 64, 3)
    back = grid.transform_world_to_cell(world)
    assert torch.allclose(back, (gc * 4 + cc).view(-1, 3).float(), atol=1e-4)
    grid.dense_init_()
    assert grid.engine.size() == 512
    lo, hi = grid.get_bbox()
    assert torch.equal(lo, torch.zeros(3)) and torch.equal(hi, torch.ones(3))


def test_unbounded_grid_bbox_and_sampling(cpu_ash):
    grid = cpu_ash.UnBoundedSparseDenseGrid(3, 64, 2, 4, cell_size=0.5, device=CPU)
    grid.spatial_init_(torch.tensor([[0.1, 0.1, 0.1], [-3.0, 2.5, 9.0]]), dilation=0)
    lo, hi = grid.get_bbox()
    assert lo.tolist() == [-4.0, 0.0, 0.0] and hi.tolist() == [2.0, 4.0, 10.0]
    pts = grid.uniform_sample(500)
    feats, masks = grid(pts, "linear")
    assert masks.all() and feats.shape == (500, 2)


@pytest.mark.parametrize("embedding_dim,grid_dim", [(2, 1), (1, 2), (4, 4)])
def test_grid_gradcheck_through_autograd_functions(cpu_ash, embedding_dim, grid_dim):
    """unittests/test_sparsedense_grid.py:183-347 in float64 on the oracle:
    checks the autograd wiring of both Functions (argument order, which inputs
    get gradients, the chained double backward)."""
    torch.manual_seed(15213)
    grid = cpu_ash.SparseDenseGrid(3, 8, embedding_dim, grid_dim, device=CPU)
    r = torch.arange(0, 2, dtype=torch.int)
    grid.spatial_init_(grid_dim * torch.stack(torch.meshgrid(r, r, r, indexing="ij"), -1).view(-1, 3), dilation=0)
    grid.construct_grid_neighbor_lut_(1, False)
    cells = torch.randint(high=grid_dim * 2 - 1, size=(40, 3))
    x = cells + torch.rand(40, 3).clamp(0.05, 0.95)
    gi, ci, off, masks = grid.query(x)
    emb = (torch.rand(grid.embeddings.shape, dtype=torch.float64) * 2 - 1).requires_grad_(True)
    z = torch.rand(40, embedding_dim, dtype=torch.float64).requires_grad_(True)
    tables = (gi, ci, masks, grid.lut_grid_nb2grid_idx, grid.lut_cell_nb2cell_idx,
              grid.lut_cell_nb2grid_nb, grid.grid_dim)

    for interpolation in ("linear", "smooth_step"):
        fwd = lambda e: cpu_ash.SparseDenseGridQuery.apply(e, off, *tables, interpolation)
        torch.autograd.gradcheck(fwd, (emb,), eps=1e-6, atol=1e-6)
        bwd = lambda e, zz: cpu_ash.SparseDenseGridQueryBackward.apply(zz, e, off, *tables, interpolation)[1]
        torch.autograd.gradcheck(bwd, (emb, z), eps=1e-6, atol=1e-6)
    # default interpolation of the Function is smooth_step (ash/grid_query.py:35)
    a = cpu_ash.SparseDenseGridQuery.apply(emb, off, *tables)
    b = cpu_ash.SparseDenseGridQuery.apply(emb, off, *tables, "smooth_step")
    assert torch.equal(a, b)


def test_one_dense_gradient_per_backward_pass(cpu_ash, oracle, monkeypatch):
    """A value loss plus a gradient-norm loss reach the embeddings through the
    first- and the second-order backward in one pass.  As shipped every node
    produces a dense gradient of its own and autograd adds them, as in the
    reference.  Inside `with ash.dense_grad(grid):` both nodes add to
    `embeddings.grad` directly and return no gradient: the result is what
    separate passes give -- also with another user of the embeddings in the
    loss while a hook keeps a node's gradients (the case an implicit sharing
    cannot get right), on a second pass into an existing .grad, with a
    caller's buffer, and not at all while a graph of the backward is being
    recorded or for tensors that were not registered."""
    import ash.grid_query as gq

    torch.manual_seed(7)
    g_dim = 2
    grid = cpu_ash.SparseDenseGrid(3, 8, 3, g_dim, device=CPU)
    r = torch.arange(0, 2, dtype=torch.int)
    grid.spatial_init_(g_dim * torch.stack(torch.meshgrid(r, r, r, indexing="ij"), -1).view(-1, 3), dilation=0)
    grid.construct_grid_neighbor_lut_(1, False)
    with torch.no_grad():
        grid.embeddings.copy_(torch.rand(grid.embeddings.shape) * 2 - 1)
    x = (torch.randint(high=g_dim * 2 - 1, size=(50, 3)) + torch.rand(50, 3).clamp(0.05, 0.95))

    in_place_calls = []
    for name in ("query_backward_forward", "query_backward_backward"):
        real = getattr(oracle, name)

        def spy(*args, _real=real, _name=name, **kwargs):
            if kwargs.get("accumulate_into") is not None:
                in_place_calls.append(_name)
            return _real(*args, **kwargs)

        monkeypatch.setattr(oracle, name, spy, raising=False)

    def losses(xq):
        feats, _ = grid(xq, "smooth_step")
        (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
        return (feats[:, 1:] ** 2).mean(), (gx.norm(dim=-1) - 1).abs().mean()

    def separate():
        total = torch.zeros_like(grid.embeddings)
        for which in (0, 1):
            grid.embeddings.grad = None
            losses(x.clone().requires_grad_(True))[which].backward()
            total += grid.embeddings.grad
        return total

    expected = separate()
    grid.embeddings.grad = None
    value, eikonal = losses(x.clone().requires_grad_(True))
    (value + eikonal).backward()
    assert in_place_calls == [] and gq.LAST_GRADIENT_PATH == "own"
    assert torch.allclose(grid.embeddings.grad, expected, rtol=1e-5, atol=1e-7)

    def hooked_step(inside_block):
        """A hook that keeps the gradients of the query node + a third
        contribution to the parameter."""
        kept = []
        grid.embeddings.grad = None
        xq = x.clone().requires_grad_(True)
        feats, _ = grid(xq, "smooth_step")
        feats.grad_fn.register_hook(lambda grad_inputs, grad_outputs: kept.append(grad_inputs))
        (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
        loss = ((feats[:, 1:] ** 2).mean() + (gx.norm(dim=-1) - 1).abs().mean()
                + 0.5 * (grid.embeddings ** 2).sum())
        if inside_block:
            with cpu_ash.dense_grad(grid):
                loss.backward()
        else:
            loss.backward()
        assert len(kept) >= 1
        return grid.embeddings.grad.clone()

    want = expected + grid.embeddings.detach()
    assert torch.allclose(hooked_step(False), want, rtol=1e-5, atol=1e-6)
    assert in_place_calls == []
    assert torch.allclose(hooked_step(True), want, rtol=1e-5, atol=1e-6)
    assert sorted(in_place_calls) == ["query_backward_backward", "query_backward_forward"]
    assert gq._DENSE_TARGETS == {}          # the block has ended

    # the plain step inside the block; a second pass adds to the existing .grad
    del in_place_calls[:]
    grid.embeddings.grad = None
    with cpu_ash.dense_grad(grid.embeddings):
        value, eikonal = losses(x.clone().requires_grad_(True))
        (value + eikonal).backward()
        assert len(in_place_calls) == 2 and gq.LAST_GRADIENT_PATH == "contract"
        assert torch.allclose(grid.embeddings.grad, expected, rtol=1e-5, atol=1e-7)
        held = grid.embeddings.grad
        value, eikonal = losses(x.clone().requires_grad_(True))
        (value + eikonal).backward()
        assert len(in_place_calls) == 4 and grid.embeddings.grad is held
        assert torch.allclose(grid.embeddings.grad, 2 * expected, rtol=1e-5, atol=1e-6)

    # a caller's buffer becomes .grad (zero-filled on entry) when there is none
    mine = torch.full_like(grid.embeddings, 7.0)
    grid.embeddings.grad = None
    with cpu_ash.dense_grad(grid, buffers={grid.embeddings: mine}):
        assert grid.embeddings.grad is mine and float(mine.abs().max()) == 0.0
        value, eikonal = losses(x.clone().requires_grad_(True))
        (value + eikonal).backward()
    assert grid.embeddings.grad is mine
    assert torch.allclose(mine, expected, rtol=1e-5, atol=1e-7)

    # while a graph of the backward pass is recorded nothing is added in place
    before = len(in_place_calls)
    grid.embeddings.grad = None
    value, eikonal = losses(x.clone().requires_grad_(True))
    with cpu_ash.dense_grad(grid):
        (got,) = torch.autograd.grad(value + eikonal, grid.embeddings, create_graph=True)
    assert len(in_place_calls) == before
    assert torch.allclose(got.detach(), expected, rtol=1e-5, atol=1e-7)

    # another leaf over the same storage, and a tensor computed from the
    # parameter, are not the registered parameter: autograd gets their gradients
    grid.embeddings.grad = None
    alias = grid.embeddings.detach().requires_grad_(True)
    tables = (grid.lut_grid_nb2grid_idx, grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, g_dim)
    gi, ci, off, masks = grid.query(x)
    before = len(in_place_calls)
    a = cpu_ash.SparseDenseGridQuery.apply(grid.embeddings, off, gi, ci, masks, *tables)
    b = cpu_ash.SparseDenseGridQuery.apply(alias, off, gi, ci, masks, *tables)
    with cpu_ash.dense_grad(grid):
        (a.sum() + 2 * b.sum()).backward()
    assert len(in_place_calls) == before + 1
    assert torch.allclose(alias.grad, 2 * grid.embeddings.grad)

    scaled = grid.embeddings * 1.0
    xq = x.clone().requires_grad_(True)
    gi, ci, off, masks = grid.query(xq)
    feats = cpu_ash.SparseDenseGridQuery.apply(scaled, off, gi, ci, masks, *tables, "smooth_step")
    (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
    grid.embeddings.grad = None
    before = len(in_place_calls)
    with cpu_ash.dense_grad(grid):
        ((feats[:, 1:] ** 2).mean() + (gx.norm(dim=-1) - 1).abs().mean()).backward()
    assert len(in_place_calls) == before and gq.LAST_GRADIENT_PATH == "own"
    assert torch.allclose(grid.embeddings.grad, expected, rtol=1e-5, atol=1e-7)


# ---------------------------------------------- engine / set / map / embedding
@pytest.mark.parametrize("dim", [1, 2, 3, 4])
def test_engine_state_dict_layout_and_round_trip(cpu_ash, dim, tmp_path):
    """ash/core.py:69-135 and unittests/test_engine.py:85-106."""
    capacity = 2000
    for num in (0, 1500):
        engine = cpu_ash.ASHEngine(dim, capacity, CPU)
        keys = _tiled_keys(dim, num, seed=dim)
        if num:
            engine.insert_keys(keys)
        state = engine.state_dict()
        assert list(state) == ["_heap", "_keys", "_indices", "_size"]
        assert state["_heap"].dtype == torch.int32 and state["_heap"].shape == (capacity,)
        assert state["_keys"].dtype == torch.int32 and state["_keys"].shape == (capacity, dim)
        assert state["_indices"].dtype == torch.int64 and state["_indices"].shape == (capacity,)
        assert state["_size"].dtype == torch.int32 and state["_size"].item() == num
        path = os.path.join(tmp_path, f"e{num}.pt")
        torch.save(state, path)
        other = cpu_ash.ASHEngine(dim, capacity, CPU)
        other.load_state_dict(torch.load(path))
        k, i = other.items()
        assert len(k) == num
        assert all(torch.equal(a, b) for a, b in zip(sort_rows(k, i), sort_rows(*engine.items())))


def test_engine_resize_multivalue_and_warnings(cpu_ash):
    """unittests/test_engine.py:108-159 plus the warning paths of ash/core.py."""
    dim, old, new, num = 3, 4000, 2000, 2000
    engine = cpu_ash.ASHEngine(dim, old, CPU)
    stores = {"0": torch.zeros(old, dim, dtype=torch.int64), "1": torch.zeros(old, dim)}
    keys = _tiled_keys(dim, num, seed=3)
    engine.insert(keys, {"0": keys.long() * 2, "1": keys.float() * 4}, stores)
    grown = {"0": torch.zeros(new, dim, dtype=torch.int64), "1": torch.zeros(new, dim)}
    engine.resize(new, stores, grown)
    idx, mask = engine.find(keys)
    assert mask.all() and torch.equal(grown["0"][idx], keys.long() * 2)
    assert torch.equal(grown["1"][idx], keys.float() * 4)
    with pytest.raises(AssertionError):
        engine.resize(num - 1)
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        engine.insert_keys(torch.tensor([[9000, 9000, 9000]], dtype=torch.int32))
    assert engine.size() == new
    with pytest.warns(UserWarning, match="empty keys"):
        engine.find(torch.zeros((0, 3), dtype=torch.int32))
    with pytest.warns(UserWarning, match="not int32"):
        engine.find(torch.zeros((1, 3), dtype=torch.int64))
    with pytest.raises(AssertionError):
        engine.find(torch.zeros((1, 2), dtype=torch.int32))
    assert "ASHEngine (dim=3, capacity=2000, size=2000)" in repr(engine)
    engine.clear()
    assert engine.size() == 0 and torch.equal(engine._heap, torch.arange(new, dtype=torch.int32))


def test_hashset_and_hashmap_wrappers(cpu_ash):
    """unittests/test_hashset.py and test_hashmap.py: return orders and value
    naming (mask first; "default", "default_<i>", or the caller's names)."""
    keys = _tiled_keys(2, 500, seed=8)
    hs = cpu_ash.HashSet(2, 1000, CPU)
    hs.insert(keys)
    assert hs.find(keys).all() and hs.size() == 500
    hs.erase(keys[:250])
    assert int(hs.find(keys).sum()) == 250
    hs.resize(5000)
    assert int(hs.find(keys).sum()) == 250 and hs.engine.capacity == 5000
    assert torch.equal(sort_rows(hs.keys())[0], sort_rows(keys[250:])[0])

    for value_dims, names in ((2, ["default"]), ([1, 3], ["default_0", "default_1"]), ({"a": 4, "b": 1}, ["a", "b"])):
        hm = cpu_ash.HashMap(2, value_dims, 1000, CPU)
        assert list(hm.values) == names and all(n in dict(hm.named_buffers()) for n in names)
        named = {n: torch.rand(500, hm.values[n].shape[1]) for n in names}
        hm.insert(keys, hm.reinterpret_value_dict(named))
        masks, indices, values = hm.find(keys, return_indices=True, return_values=True)
        assert masks.dtype == torch.bool and masks.all()
        back = values if isinstance(values, dict) else ({"default": values} if torch.is_tensor(values) else {f"default_{i}": v for i, v in enumerate(values)})
        for n in names:
            assert torch.equal(back[n], named[n])
        only_values = hm.find(keys, return_indices=False, return_values=True)
        assert len(only_values) == 2
        with pytest.raises(AssertionError):
            hm.find(keys, return_indices=False, return_values=False)
        hm.resize(3000)
        k, i, v = hm.items(return_values=True)
        assert len(k) == 500 and all(hm.values[n].shape[0] == 3000 for n in names)
        state = hm.state_dict()
        assert set(state) == {"engine._heap", "engine._keys", "engine._indices", "engine._size", *names}
        hm2 = cpu_ash.HashMap(2, value_dims, 3000, CPU)
        hm2.load_state_dict(state, strict=False)
        m2, _, v2 = hm2.find(keys, return_values=True)
        back2 = v2 if isinstance(v2, dict) else ({"default": v2} if torch.is_tensor(v2) else {f"default_{i}": x for i, x in enumerate(v2)})
        assert m2.all() and all(torch.equal(back2[n], named[n]) for n in names)
        hm.clear()
        assert hm.size() == 0 and all(float(s.abs().sum()) == 0 for s in hm.values.values())
    with pytest.raises(ValueError):
        cpu_ash.HashMap(2, "bad", 10, CPU)


def test_hash_embedding_forward(cpu_ash):
    """unittests/test_embedding.py:29-39: zeros for keys never inserted."""
    emb = cpu_ash.HashEmbedding(3, 100, 16, CPU)
    keys = _tiled_keys(3, 200, seed=4)
    emb.spatial_init_(keys[:100])
    out = emb(keys)
    assert out.shape == (200, 16) and torch.equal(out[100:], torch.zeros(100, 16))
    idx, _ = emb.engine.find(keys[:100])
    assert torch.equal(out[:100], emb.embedding[idx])
    out.sum().backward()
    assert emb.embedding.grad is not None
    assert set(emb.state_dict()) == {"embedding", "engine._heap", "engine._keys", "engine._indices", "engine._size"}

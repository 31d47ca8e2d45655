"""GPU parity tests of the sparse convolution (ash_convolution_forward) against
the oracle on identical inputs: taps are accumulated in the same order with one
fused multiply-add each on both sides, so the outputs are bit-exact."""
import pytest
import torch

import workloads

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _tables(grid, radius):
    c2g, c2c = grid.construct_cell_neighbor_lut(radius, bidirectional=True)
    _, g2g = grid.construct_grid_neighbor_lut((radius + grid.grid_dim - 1) // grid.grid_dim,
                                              bidirectional=True)
    _, _, gi, ci = grid.items()
    return c2g, c2c, g2g, gi, ci


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("radius,channels", [(1, 4), (2, 3), (1, 16), (3, 1)])
def test_convolution_matches_oracle(gpu_ash, oracle, dtype, radius, channels):
    grid, _, _ = workloads.build_grid(gpu_ash, 700, channels, 8, 32, device=DEV)
    g = torch.Generator().manual_seed(800 + radius)
    inputs = torch.randn(grid.embeddings.shape, generator=g, dtype=dtype).to(DEV)
    size = 2 * radius + 1
    weights = torch.randn(size, size, size, channels, generator=g, dtype=dtype).to(DEV)
    out = grid.convolution(inputs, weights)
    c2g, c2c, g2g, gi, ci = _tables(grid, radius)
    masks = torch.ones(inputs.shape[:2], dtype=torch.bool)
    ref = oracle.convolution_forward(inputs, weights.view(size**3, channels), masks, gi, ci,
                                     g2g, c2c, c2g, 8)
    assert out.dtype == dtype and torch.equal(out.cpu(), ref)
    assert float(ref.abs().max()) > 1.0


def test_masked_cells_and_unlisted_blocks_stay_zero(gpu_ash, oracle):
    grid, _, _ = workloads.build_grid(gpu_ash, 300, 2, 8, 32, device=DEV)
    g = torch.Generator().manual_seed(810)
    inputs = torch.randn(grid.embeddings.shape, generator=g).to(DEV)
    weights = torch.randn(27, 2, generator=g).to(DEV)
    c2g, c2c, g2g, gi, ci = _tables(grid, 1)
    listed = gi.view(-1)[::2].contiguous()  # every other block
    masks = (torch.rand(listed.numel() * 512, generator=g) < 0.7).to(DEV)
    backend = gpu_ash.grid.backend
    out = backend.convolution_forward(inputs, weights, masks, listed, ci, g2g, c2c, c2g, 8)
    ref = oracle.convolution_forward(inputs, weights, masks, listed, ci, g2g, c2c, c2g, 8)
    assert torch.equal(out.cpu(), ref)
    skipped = torch.ones(inputs.shape[0], dtype=torch.bool)
    skipped[listed.cpu()] = False
    assert bool((out.cpu()[skipped] == 0).all())
    rows = out[listed].view(-1, 2)
    assert bool((rows[~masks] == 0).all()) and bool((rows[masks] != 0).any())
    # nothing listed: all zeros
    none = backend.convolution_forward(inputs, weights, masks[:0], listed[:0], ci, g2g, c2c, c2g, 8)
    assert bool((none == 0).all())


@pytest.mark.parametrize("channels,radius,reorder", [(16, 1, False), (4, 1, False), (3, 2, False),
                                                     (5, 1, True), (8, 3, False)])
def test_entries_with_and_without_block_scratch_agree(gpu_ash, oracle, channels, radius, reorder):
    """ash_convolution_forward clears the whole output and leaves skipped cells
    alone; ash_convolution_forward_listed clears the rows of unlisted blocks
    only and writes zeros into skipped cells of listed ones.  Both from an
    output full of NaNs, half of the blocks listed, a third of the cells masked
    out, also with the taps in another order (cells then go through the
    tables): equal to the oracle bit for bit."""
    import ctypes

    from ash.common import _DTYPE, _stream_of

    grid, _, _ = workloads.build_grid(gpu_ash, 300, channels, 8, 32, device=DEV)
    g = torch.Generator().manual_seed(870 + channels)
    inputs = torch.randn(grid.embeddings.shape, generator=g).to(DEV)
    k = (2 * radius + 1) ** 3
    weights = torch.randn(k, channels, generator=g).to(DEV)
    c2g, c2c, g2g, gi, ci = _tables(grid, radius)
    if reorder:
        perm = torch.randperm(k, generator=g).to(DEV)
        c2g, c2c, weights = c2g[:, perm].contiguous(), c2c[:, perm].contiguous(), weights[perm].contiguous()
    listed = gi.view(-1)[1::2].contiguous()
    masks = (torch.rand(listed.numel() * 512, generator=g) < 0.67).to(DEV)
    ref = oracle.convolution_forward(inputs, weights, masks, listed, ci, g2g, c2c, c2g, 8)
    lib = gpu_ash.grid.backend.lib
    b, m, e = inputs.shape
    ci = ci.view(-1).contiguous()
    common = (inputs.data_ptr(), weights.data_ptr(), masks.data_ptr(), listed.data_ptr(),
              ci.data_ptr(), g2g.data_ptr(), c2c.data_ptr(), c2g.data_ptr())
    sizes = (listed.numel(), b, m, e, k, g2g.shape[1], _DTYPE[inputs.dtype])
    plain = torch.full_like(inputs, float("nan"))
    assert lib.ash_convolution_forward(*common, plain.data_ptr(), *sizes, _stream_of(DEV)) == 0
    scratch = torch.full((b,), 7, dtype=torch.uint8, device=DEV)
    with_scratch = torch.full_like(inputs, float("nan"))
    assert lib.ash_convolution_forward_listed(*common, with_scratch.data_ptr(), *sizes,
                                              scratch.data_ptr(), _stream_of(DEV)) == 0
    assert torch.equal(plain.cpu(), ref)
    assert torch.equal(with_scratch.cpu(), ref)
    assert lib.ash_convolution_forward_listed(*common, with_scratch.data_ptr(), *sizes,
                                              None, _stream_of(DEV)) != 0


def test_window_tables_follow_the_table(gpu_ash, oracle):
    """grid.convolution keeps its tables between calls: the per-cell pair per
    radius, the per-block one while the table holds the same keys.  After more
    blocks are dropped or activated the result has to follow."""
    grid, _, _ = workloads.build_grid(gpu_ash, 200, 2, 8, 32, device=DEV)
    g = torch.Generator().manual_seed(880)
    weights = torch.randn(3, 3, 3, 2, generator=g).to(DEV)

    def check():
        inputs = torch.randn(grid.embeddings.shape, generator=g).to(DEV)
        out = grid.convolution(inputs, weights)
        c2g, c2c, g2g, gi, ci = _tables(grid, 1)
        masks = torch.ones(inputs.shape[:2], dtype=torch.bool)
        ref = oracle.convolution_forward(inputs, weights.view(27, 2), masks, gi, ci, g2g, c2c, c2g, 8)
        assert torch.equal(out.cpu(), ref)
        return out

    check()
    first_tables = grid._window_tables(1)
    check()
    assert all(a is b for a, b in zip(first_tables, grid._window_tables(1)))
    keys, _ = grid.engine.items()
    grid.engine.erase(keys[:40].contiguous())
    assert grid.engine.size() == len(keys) - 40
    check()
    grid.engine.insert_keys((keys[:25] + torch.tensor([[1, 0, 0]], device=DEV, dtype=keys.dtype)).clamp(0, 31))
    check()
    assert grid._window_tables(1)[2] is not first_tables[2]
    assert grid._window_tables(1)[0] is first_tables[0]


def test_gaussian_filter_device_equals_oracle_backend(gpu_ash, oracle, monkeypatch):
    """SparseDenseGrid.gaussian_filter_ (ash/grid.py:435-476) end to end: the
    same blocks and the same field, filtered on the device and on the CPU with
    the oracle as backend, compared block by block."""
    import ash.core
    import ash.grid
    import ash.grid_query

    blocks, _, _ = workloads.surface_blocks(400, 8, 32, device="cpu", seed=9)
    g = torch.Generator().manual_seed(820)
    field = torch.randn(len(blocks), 512, 3, generator=g)

    def run(device):
        grid = gpu_ash.BoundedSparseDenseGrid(
            3, 400, 3, grid_dim=8, sparse_grid_dim=32, bbox_min=torch.zeros(3),
            bbox_max=torch.ones(3), device=device)
        grid.engine.insert_keys(blocks.to(device))
        rows, found = grid.engine.find(blocks.to(device))
        assert bool(found.all())
        with torch.no_grad():
            grid.embeddings[rows] = field.to(device)
        grid.gaussian_filter_(3, 1.0)
        return grid.embeddings.detach()[rows].cpu()

    on_device = run(DEV)
    with monkeypatch.context() as m:
        for mod in (ash.core, ash.grid, ash.grid_query):
            m.setattr(mod, "backend", oracle)
        on_cpu = run(torch.device("cpu"))
    assert torch.equal(on_device, on_cpu)
    assert not torch.equal(on_device, field)


def test_few_blocks_take_the_per_cell_kernel(gpu_ash, oracle):
    """Fewer than 64 listed blocks: the launch that maps one lane to one cell
    (also with a row width that is not a multiple of four, and one above 16)."""
    for channels in (3, 8, 20):
        grid, _, _ = workloads.build_grid(gpu_ash, 48, min(channels, 16), 8, 16, device=DEV)
        g = torch.Generator().manual_seed(840 + channels)
        inputs = torch.randn(*grid.embeddings.shape[:2], channels, generator=g).to(DEV)
        weights = torch.randn(3, 3, 3, channels, generator=g).to(DEV)
        out = grid.convolution(inputs, weights)
        c2g, c2c, g2g, gi, ci = _tables(grid, 1)
        masks = torch.ones(inputs.shape[:2], dtype=torch.bool)
        ref = oracle.convolution_forward(inputs, weights.view(27, channels), masks, gi, ci,
                                         g2g, c2c, c2g, 8)
        assert torch.equal(out.cpu(), ref)


def test_tables_in_another_order_take_the_table_path(gpu_ash, oracle):
    """The tiled kernel assumes the layout the Python layer builds and checks
    the tables against it; taps listed in another order must give the same
    result through the tables (weights permuted alike, so the sums differ only
    in the order of their terms -- and that order is the tables')."""
    grid, _, _ = workloads.build_grid(gpu_ash, 300, 5, 8, 32, device=DEV)
    g = torch.Generator().manual_seed(820)
    inputs = torch.randn(grid.embeddings.shape, generator=g).to(DEV)
    weights = torch.randn(27, 5, generator=g).to(DEV)
    c2g, c2c, g2g, gi, ci = _tables(grid, 1)
    perm = torch.randperm(27, generator=g).to(DEV)
    masks = torch.ones(inputs.shape[:2], dtype=torch.bool)
    backend = gpu_ash.grid.backend
    args = (masks, gi, ci, g2g, c2c[:, perm].contiguous(), c2g[:, perm].contiguous(), 8)
    out = backend.convolution_forward(inputs, weights[perm].contiguous(), *args)
    ref = oracle.convolution_forward(inputs, weights[perm].contiguous(), *args)
    assert torch.equal(out.cpu(), ref)
    # five channels through the tile: one pass of eight with three idle
    plain = backend.convolution_forward(inputs, weights, masks, gi, ci, g2g, c2c, c2g, 8)
    plain_ref = oracle.convolution_forward(inputs, weights, masks, gi, ci, g2g, c2c, c2g, 8)
    assert torch.equal(plain.cpu(), plain_ref)
    assert torch.allclose(out, plain, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("radius,channels", [(3, 5), (2, 16), (3, 16), (1, 8), (1, 6), (1, 12), (2, 8)])
def test_wide_windows_and_rows(gpu_ash, oracle, radius, channels):
    grid, _, _ = workloads.build_grid(gpu_ash, 200, channels, 8, 32, device=DEV)
    g = torch.Generator().manual_seed(830 + radius)
    inputs = torch.randn(grid.embeddings.shape, generator=g).to(DEV)
    size = 2 * radius + 1
    weights = torch.randn(size**3, channels, generator=g).to(DEV)
    c2g, c2c, g2g, gi, ci = _tables(grid, radius)
    masks = (torch.rand(inputs.shape[:2], generator=g) < 0.9)
    args = (masks, gi, ci.view(-1)[torch.randperm(512, generator=g).to(DEV)], g2g, c2c, c2g, 8)
    out = gpu_ash.grid.backend.convolution_forward(inputs, weights, *args)
    ref = oracle.convolution_forward(inputs, weights, *args)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("radius", [1, 3])
def test_impulse_and_constant_field_on_a_dense_volume(gpu_ash, radius):
    """Independent of the oracle: on a dense volume an impulse at cell p gives
    out[p - o_k] = w[k] (tap k reads the cell at offset o_k), and a field of
    ones gives the sum of the weights, added in table order, at every cell
    whose window lies inside the volume."""
    s, g_dim, e = 5, 8, 4
    grid = gpu_ash.BoundedSparseDenseGrid(
        3, s**3, e, grid_dim=g_dim, sparse_grid_dim=s, bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3), device=DEV)
    grid.dense_init_()
    keys, idx = grid.engine.items()
    size = 2 * radius + 1
    g = torch.Generator().manual_seed(840 + radius)
    weights = torch.randn(size, size, size, e, generator=g).to(DEV)
    n = s * g_dim
    # dense view of a (B, M, E) tensor: vol[x, y, z, :]
    cells = (keys.view(-1, 1, 3) * g_dim + grid.cell_coords.view(1, -1, 3)).long()

    def densify(t):
        vol = torch.zeros(n, n, n, e, device=DEV)
        vol[cells[..., 0], cells[..., 1], cells[..., 2]] = t[idx]
        return vol

    p = torch.tensor([17, 22, 19], device=DEV)
    inputs = torch.zeros(grid.embeddings.shape, device=DEV)
    block = (keys == (p // g_dim).int()).all(dim=1).nonzero().item()
    local = p % g_dim
    inputs[idx[block], local[0] + g_dim * local[1] + g_dim**2 * local[2]] = 1.0
    vol = densify(grid.convolution(inputs, weights))
    lo, hi = p - radius, p + radius + 1
    patch = vol[lo[0]:hi[0], lo[1]:hi[1], lo[2]:hi[2]]
    # weights[i, j, k] belongs to the offset (k, j, i) - radius: x varies fastest
    expect = weights.permute(2, 1, 0, 3).flip(0, 1, 2)
    assert torch.equal(patch, expect)
    assert int((vol != 0).sum()) == int((expect != 0).sum())

    ones = torch.ones(grid.embeddings.shape, device=DEV)
    vol = densify(grid.convolution(ones, weights))
    total = torch.zeros(e)
    for row in weights.view(-1, e).cpu():
        total = total + row          # fma(1, w, acc) in table order
    inner = vol[radius:n - radius, radius:n - radius, radius:n - radius]
    assert torch.equal(inner.reshape(-1, e).cpu(), total.expand(inner.numel() // e, e))


@pytest.mark.parametrize("grid_dim,radius,channels", [(4, 1, 3), (4, 2, 2), (16, 1, 2), (6, 2, 4),
                                                      (12, 3, 1)])
def test_other_block_edges(gpu_ash, oracle, grid_dim, radius, channels, monkeypatch):
    """Block edges that are and are not multiples of four (the latter compute
    one cell per lane), windows reaching two blocks deep into a small block.
    Outputs start as NaNs and a fifth of the cells is masked out: every cell
    has to be written, by the clear or by the kernel."""
    monkeypatch.setattr(torch, "empty_like", lambda t, **kw: torch.full_like(t, float("nan")))
    s = 5
    g = torch.Generator().manual_seed(850 + grid_dim)
    blocks = torch.stack(torch.meshgrid(*[torch.arange(s)] * 3, indexing="ij"), -1).view(-1, 3)
    blocks = blocks[torch.rand(len(blocks), generator=g) < 0.8]
    grid = gpu_ash.BoundedSparseDenseGrid(
        3, len(blocks) + 3, channels, grid_dim=grid_dim, sparse_grid_dim=s,
        bbox_min=torch.zeros(3), bbox_max=torch.ones(3), device=DEV)
    grid.engine.insert_keys(blocks.int().to(DEV))
    assert grid.engine.size() >= 64
    inputs = torch.randn(grid.embeddings.shape, generator=g).to(DEV)
    size = 2 * radius + 1
    weights = torch.randn(size**3, channels, generator=g).to(DEV)
    c2g, c2c, g2g, gi, ci = _tables(grid, radius)
    masks = torch.rand(inputs.shape[:2], generator=g) < 0.8
    out = gpu_ash.grid.backend.convolution_forward(inputs, weights, masks, gi, ci, g2g, c2c, c2g,
                                                   grid_dim)
    ref = oracle.convolution_forward(inputs, weights, masks, gi, ci, g2g, c2c, c2g, grid_dim)
    assert torch.equal(out.cpu(), ref) and float(ref.abs().max()) > 1.0

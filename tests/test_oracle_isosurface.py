"""Pins of the oracle's iso-surface point extraction (restating
ash/src/grid.cu:453-531 behind the `vertices_only` branch of
SparseDenseGrid.marching_cubes, ash/grid.py:654-678): a sphere's distance field
sampled on a fully active grid must give points on the sphere, as many as a
brute-force count of sign changes on the densified volume, and the reference's
handling of missing neighbour blocks is checked on a hand-made case."""
import numpy as np
import torch

G, S = 4, 4  # cells per block edge, blocks per axis


def _grid(cpu_ash, blocks):
    grid = cpu_ash.BoundedSparseDenseGrid(
        3, 64, 1, grid_dim=G, sparse_grid_dim=S, bbox_min=torch.zeros(3), bbox_max=torch.ones(3),
        device="cpu")
    grid.engine.insert_keys(blocks.int())
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    return grid


def _all_blocks():
    return torch.stack(torch.meshgrid(*[torch.arange(S)] * 3, indexing="ij"), -1).view(-1, 3)


def _cell_positions(grid):
    """(B, M, 3) integer cell positions of the active rows (others zero)."""
    keys, idx = grid.engine.items()
    pos = torch.zeros(grid.embeddings.shape[0], G**3, 3)
    pos[idx] = keys.view(-1, 1, 3).float() * G + grid.cell_coords.view(1, -1, 3).float()
    return pos, keys, idx


def test_sphere_points_lie_on_the_sphere_and_match_a_dense_count(cpu_ash):
    grid = _grid(cpu_ash, _all_blocks())
    pos, keys, idx = _cell_positions(grid)
    centre, radius = torch.tensor([7.3, 8.1, 7.7]), 5.2
    sdf = (pos - centre).norm(dim=-1) - radius
    weights = torch.ones_like(sdf)
    pts = cpu_ash.grid.backend.isosurface_extraction(
        sdf, weights, idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
        grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, G, 0.0, 1.0)
    # linear interpolation of a distance field along an edge of length 1:
    # the crossing is within ~1/(8 r) of the sphere
    err = ((pts - centre).norm(dim=-1) - radius).abs()
    assert len(pts) > 300 and float(err.max()) < 0.03
    # every point sits on a grid edge: two integer coordinates, one in between
    frac = pts - pts.floor()
    assert bool(((frac > 0).sum(dim=1) == 1).all())
    # brute force on the dense volume
    n = G * S
    vol = np.zeros((n, n, n))
    ip = pos[idx].view(-1, 3).long().numpy()
    vol[ip[:, 0], ip[:, 1], ip[:, 2]] = sdf[idx].view(-1).numpy()
    count = 0
    for axis in range(3):
        a = np.moveaxis(vol, axis, 0)
        count += int(((a[:-1] * a[1:]) < 0).sum())
    assert len(pts) == count
    # iso value: a larger sphere
    pts2 = cpu_ash.grid.backend.isosurface_extraction(
        sdf, weights, idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
        grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, G, 1.0, 1.0)
    err2 = ((pts2 - centre).norm(dim=-1) - (radius + 1.0)).abs()
    assert len(pts2) > len(pts) and float(err2.max()) < 0.03


def test_weights_and_missing_blocks(cpu_ash):
    """Plane x = 5.5 through blocks (1, *, *).  (a) a cell or neighbour below
    the weight threshold gives no point; (b) when the +x neighbour block of a
    cell is missing the reference stops scanning that cell, so the cell's +y /
    +z crossings are lost as well."""
    blocks = torch.tensor([[0, 0, 0], [1, 0, 0], [0, 1, 0]])  # no block (1, 1, 0), none at z = 1
    grid = _grid(cpu_ash, blocks)
    pos, keys, idx = _cell_positions(grid)
    sdf = pos[..., 0] - 5.5
    weights = torch.ones_like(sdf)
    args = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, G)
    pts = cpu_ash.grid.backend.isosurface_extraction(sdf, weights, *args, 0.0, 1.0)
    # crossings between x = 5 and x = 6 inside block (1, 0, 0): 16 edges, all at x = 5.5
    assert pts.shape == (16, 3) and bool((pts[:, 0] == 5.5).all())
    assert sorted(map(tuple, pts[:, 1:].long().tolist())) == [(y, z) for y in range(4) for z in range(4)]
    # (a) drop the weight of the cells at x = 6, y = 0
    low = weights.clone()
    row = int(idx[(keys == torch.tensor([1, 0, 0])).all(dim=1)][0])
    cells = (grid.cell_coords[:, 0] == 2) & (grid.cell_coords[:, 1] == 0)
    low[row, cells] = 0.5
    pts = cpu_ash.grid.backend.isosurface_extraction(sdf, low, *args, 0.0, 1.0)
    assert pts.shape == (12, 3) and int(pts[:, 1].min()) == 1
    # (b) plane y = 2.5 crosses blocks (0,0,0) and (1,0,0); cells of block
    # (0, 0, 0) at x = 3 have their +x neighbour in block (1, 0, 0): present.
    # Cells of block (1, 0, 0) at x = 7 have theirs in block (2, 0, 0): missing,
    # so their +y crossings are not reported: 4 x-positions in block 0 and 3 in
    # block 1, times 4 z-positions.
    sdf_y = pos[..., 1] - 2.5
    pts = cpu_ash.grid.backend.isosurface_extraction(sdf_y, weights, *args, 0.0, 1.0)
    assert pts.shape == (28, 3) and bool((pts[:, 1] == 2.5).all())
    assert sorted(set(pts[:, 0].long().tolist())) == [0, 1, 2, 3, 4, 5, 6]


def test_grid_method_returns_world_positions(cpu_ash):
    grid = _grid(cpu_ash, _all_blocks())
    pos, keys, idx = _cell_positions(grid)
    world = grid.transform_cell_to_world(pos)
    centre, radius = torch.tensor([0.5, 0.45, 0.55]), 0.3
    sdf = (world - centre).norm(dim=-1) - radius
    out = grid.marching_cubes(sdf.unsqueeze(-1), torch.ones_like(sdf).unsqueeze(-1), None,
                              lambda p: (p - centre) / radius, vertices_only=True)
    pts = out["positions"] if isinstance(out, dict) else torch.from_numpy(out.point["positions"].numpy())
    err = ((pts - centre).norm(dim=-1) - radius).abs()
    assert len(pts) > 200 and float(err.max()) < 0.03 * grid.cell_size * 4
    assert grid.marching_cubes(sdf + 10.0, torch.ones_like(sdf), None, None, vertices_only=True) is None

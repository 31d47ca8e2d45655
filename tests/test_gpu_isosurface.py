"""GPU parity tests of the iso-surface point extraction
(ash_isosurface_extraction) against the oracle: the same set of points, bit for
bit (the order of the output is free on both sides)."""
import pytest
import torch

import workloads
from helpers import sort_rows

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _sorted_points(p):
    p = p.detach().cpu()
    key = p.double()
    order = torch.from_numpy(__import__("numpy").lexsort(key.numpy().T[::-1]))
    return p[order]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("iso,thr", [(0.0, 1.0), (0.004, 0.5)])
def test_points_match_oracle(gpu_ash, oracle, dtype, iso, thr):
    grid, radii, centres = workloads.build_grid(gpu_ash, 3000, 1, 8, 64, device=DEV)
    keys, idx = grid.engine.items()
    cells = keys.view(-1, 1, 3) * 8 + grid.cell_coords.view(1, -1, 3)
    world = grid.transform_cell_to_world(cells.float())  # (n, M, 3)
    dist = (world.unsqueeze(2) - centres.to(DEV).view(1, 1, -1, 3)).norm(dim=-1) - radii.to(DEV)
    sdf = torch.zeros(grid.embeddings.shape[:2], dtype=dtype, device=DEV)
    sdf[idx] = dist.min(dim=2)[0].to(dtype)
    g = torch.Generator().manual_seed(830)
    weights = torch.zeros_like(sdf)
    weights[idx] = (torch.rand(len(idx), 512, generator=g) * 2).to(DEV, dtype)
    args = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, 8, iso, thr)
    got = gpu_ash.grid.backend.isosurface_extraction(sdf, weights, *args)
    ref = oracle.isosurface_extraction(sdf, weights, *args)
    assert got.dtype == torch.float32 and got.shape == ref.shape and len(ref) > 5000
    assert torch.equal(_sorted_points(got), _sorted_points(ref))


def test_grid_method_on_device(gpu_ash):
    grid, radii, centres = workloads.build_grid(gpu_ash, 3000, 1, 8, 64, device=DEV)
    keys, idx = grid.engine.items()
    cells = keys.view(-1, 1, 3) * 8 + grid.cell_coords.view(1, -1, 3)
    world = grid.transform_cell_to_world(cells.float())
    dist = (world.unsqueeze(2) - centres.to(DEV).view(1, 1, -1, 3)).norm(dim=-1) - radii.to(DEV)
    sdf = torch.zeros(grid.embeddings.shape[:2], device=DEV)
    sdf[idx] = dist.min(dim=2)[0]
    pts = grid.isosurface_points(sdf, torch.ones_like(sdf))
    d = ((pts.unsqueeze(1) - centres.to(DEV).view(1, -1, 3)).norm(dim=-1) - radii.to(DEV)).min(dim=1)[0]
    assert len(pts) > 10_000 and float(d.abs().max()) < grid.cell_size
    # nothing above the weight threshold, and an empty listing
    assert grid.marching_cubes(sdf, torch.zeros_like(sdf), None, None, vertices_only=True) is None


@pytest.mark.parametrize("grid_dim", [1, 2, 3, 5, 16, 20])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_block_sizes_match_oracle(gpu_ash, oracle, grid_dim, dtype):
    """Block edges from one cell over sizes whose cell count is no multiple of
    the kernels' chunking to edges beyond the LDS-tiled path, with missing
    blocks, light cells and exact zeros of the field."""
    s = max(3, min(12, 40 // grid_dim))
    g = torch.Generator().manual_seed(860 + grid_dim)
    blocks = torch.stack(torch.meshgrid(*[torch.arange(s)] * 3, indexing="ij"), -1).view(-1, 3)
    blocks = blocks[torch.rand(len(blocks), generator=g) < 0.85]
    grid = gpu_ash.BoundedSparseDenseGrid(
        3, len(blocks) + 7, 1, grid_dim=grid_dim, sparse_grid_dim=s, bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3), device=DEV)
    grid.engine.insert_keys(blocks.int().to(DEV))
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    _, idx = grid.engine.items()
    shape = grid.embeddings.shape[:2]
    sdf = torch.rand(shape, generator=g, dtype=dtype) - 0.45
    sdf[torch.rand(shape, generator=g) < 0.02] = 0.02      # exactly on the iso value
    sdf = sdf.to(DEV)
    weights = (torch.rand(shape, generator=g, dtype=dtype) * 10).to(DEV)
    args = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, grid_dim, 0.02, 0.4)
    got = gpu_ash.grid.backend.isosurface_extraction(sdf, weights, *args)
    ref = oracle.isosurface_extraction(sdf, weights, *args)
    assert got.shape == ref.shape and len(ref) > 200
    assert torch.equal(_sorted_points(got), _sorted_points(ref))

"""GPU parity tests of marching cubes (ash_marching_cubes_classify / _extract)
against the oracle.  Vertex and triangle numbering follow the scheduling on
both sides, so meshes are compared as sets: the vertex positions bit for bit,
and the triangles as triples of positions in the smallest of their three
rotations (which keeps the orientation)."""
import numpy as np
import pytest
import torch

import workloads

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _sorted_rows(x):
    x = x.detach().cpu().numpy()
    return x[np.lexsort(x.T[::-1])]


def _lex_min(a, b):
    """Row-wise lexicographic minimum of two (T, 9) arrays."""
    differ = a != b
    first = differ.argmax(axis=1)
    rows = np.arange(len(a))
    take_b = differ.any(axis=1) & (b[rows, first] < a[rows, first])
    return np.where(take_b[:, None], b, a)


def _triangle_set(tri, pts):
    """(T, 9) float32: corner positions of every triangle in the smallest of
    its three rotations (which keeps the orientation), rows sorted."""
    p = pts.detach().cpu()[tri.detach().cpu().long()].numpy()      # (T, 3, 3)
    rot = [np.concatenate([p[:, k:], p[:, :k]], axis=1).reshape(-1, 9) for k in range(3)]
    return _sorted_rows(torch.from_numpy(_lex_min(_lex_min(rot[0], rot[1]), rot[2])))


def _scene(gpu_ash, dtype, seed):
    grid, radii, centres = workloads.build_grid(gpu_ash, 3000, 1, 8, 64, device=DEV)
    keys, idx = grid.engine.items()
    cells = keys.view(-1, 1, 3) * 8 + grid.cell_coords.view(1, -1, 3)
    world = grid.transform_cell_to_world(cells.float())  # (n, M, 3)
    dist = (world.unsqueeze(2) - centres.to(DEV).view(1, 1, -1, 3)).norm(dim=-1) - radii.to(DEV)
    sdf = torch.zeros(grid.embeddings.shape[:2], dtype=dtype, device=DEV)
    sdf[idx] = dist.min(dim=2)[0].to(dtype)
    g = torch.Generator().manual_seed(seed)
    weights = torch.zeros_like(sdf)
    weights[idx] = (torch.rand(len(idx), 512, generator=g) * 8).to(DEV, dtype)
    return grid, idx, sdf, weights


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("iso,thr", [(0.0, 1.0), (0.004, 0.25)])
def test_mesh_matches_oracle(gpu_ash, oracle, dtype, iso, thr):
    grid, idx, sdf, weights = _scene(gpu_ash, dtype, 840)
    args = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, 8, iso, thr)
    tri, pts = gpu_ash.grid.backend.marching_cubes(sdf, weights, *args)
    tri_ref, pts_ref = oracle.marching_cubes(sdf, weights, *args)
    assert tri.dtype == torch.int32 and pts.dtype == torch.float32
    assert pts.shape == pts_ref.shape and tri.shape == tri_ref.shape and len(tri_ref) > 5000
    assert int(tri.min()) == 0 and int(tri.max()) == len(pts) - 1
    assert np.array_equal(_sorted_rows(pts), _sorted_rows(pts_ref))
    assert np.array_equal(_triangle_set(tri, pts), _triangle_set(tri_ref, pts_ref))
    # a second extraction on the same inputs gives the same mesh
    tri2, pts2 = gpu_ash.grid.backend.marching_cubes(sdf, weights, *args)
    assert np.array_equal(_triangle_set(tri2, pts2), _triangle_set(tri_ref, pts_ref))


def test_random_field_matches_oracle(gpu_ash, oracle):
    """Every case of the table, on a field without structure."""
    grid, idx, sdf, weights = _scene(gpu_ash, torch.float32, 841)
    g = torch.Generator().manual_seed(842)
    sdf[idx] = (torch.rand(len(idx), 512, generator=g) - 0.5).to(DEV)
    # a part of the blocks only: the rows that the neighbour table reaches from
    # a listed row must be listed as well, so take the closure of a fifth
    closure = idx[: len(idx) // 5]
    while True:
        lut = grid.lut_grid_nb2grid_idx[closure].view(-1)
        grown = torch.unique(torch.cat([closure, lut[lut >= 0]]))
        if len(grown) == len(closure):
            break
        closure = grown
    args = (closure, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, 8, 0.0, 0.5)
    tri, pts = gpu_ash.grid.backend.marching_cubes(sdf, weights, *args)
    tri_ref, pts_ref = oracle.marching_cubes(sdf, weights, *args)
    assert len(tri_ref) > 100_000 and tri.shape == tri_ref.shape
    assert np.array_equal(_sorted_rows(pts), _sorted_rows(pts_ref))
    assert np.array_equal(_triangle_set(tri, pts), _triangle_set(tri_ref, pts_ref))


def test_sphere_mesh_through_the_grid_method(gpu_ash):
    """One large sphere well inside a dense set of blocks, at full device
    size: closed, oriented, Euler characteristic 2, the sphere's volume."""
    grid = gpu_ash.BoundedSparseDenseGrid(
        3, 20 ** 3, 1, grid_dim=8, sparse_grid_dim=20, bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3), device=DEV)
    grid.dense_init_()
    keys, idx = grid.engine.items()
    cells = (keys.view(-1, 1, 3) * 8 + grid.cell_coords.view(1, -1, 3)).float()
    centre, radius = torch.tensor([80.3, 79.1, 81.7], device=DEV), 61.4
    sdf = torch.zeros(grid.embeddings.shape[:2], device=DEV)
    sdf[idx] = (cells - centre).norm(dim=-1) - radius
    tri, pts = grid.surface_mesh(sdf, torch.ones_like(sdf))
    assert len(tri) > 100_000
    v, f = len(pts), len(tri)
    t = tri.long()
    edges = torch.cat([t[:, [0, 1]], t[:, [1, 2]], t[:, [2, 0]]])
    code = edges[:, 0] * v + edges[:, 1]
    assert len(torch.unique(code)) == len(code)                       # each directed edge once
    back = edges[:, 1] * v + edges[:, 0]
    assert torch.equal(torch.sort(code)[0], torch.sort(back)[0])      # and its reverse once
    assert v - len(code) // 2 + f == 2
    p = pts.double()[t] / grid.cell_size
    vol = float((p[:, 0] * torch.cross(p[:, 1], p[:, 2], dim=1)).sum() / 6)
    assert abs(vol / (4 / 3 * np.pi * radius ** 3) - 1) < 2e-3
    out = grid.marching_cubes(sdf, torch.ones_like(sdf), None, normal_fn=lambda x: x * 0 + 1.0)
    if isinstance(out, dict):
        assert out["triangles"].shape == tri.shape and out["normals"].shape == pts.shape
    assert grid.marching_cubes(sdf, torch.zeros_like(sdf), None, None) is None


@pytest.mark.parametrize("grid_dim", [1, 2, 3, 5, 16, 20])
def test_block_sizes_match_oracle(gpu_ash, oracle, grid_dim):
    """Block edges from one cell (every corner in another block) over sizes whose
    cell count is no multiple of the kernels' chunking to edges beyond the
    LDS-tiled path, with missing blocks and light cells."""
    s = max(3, min(12, 40 // grid_dim))
    g = torch.Generator().manual_seed(850 + grid_dim)
    blocks = torch.stack(torch.meshgrid(*[torch.arange(s)] * 3, indexing="ij"), -1).view(-1, 3)
    blocks = blocks[torch.rand(len(blocks), generator=g) < 0.85]
    grid = gpu_ash.BoundedSparseDenseGrid(
        3, len(blocks) + 7, 1, grid_dim=grid_dim, sparse_grid_dim=s, bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3), device=DEV)
    grid.engine.insert_keys(blocks.int().to(DEV))
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    _, idx = grid.engine.items()
    shape = grid.embeddings.shape[:2]
    sdf = (torch.rand(shape, generator=g) - 0.45).to(DEV)
    weights = (torch.rand(shape, generator=g) * 10).to(DEV)
    args = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, grid_dim, 0.02, 0.4)
    tri, pts = gpu_ash.grid.backend.marching_cubes(sdf, weights, *args)
    tri_ref, pts_ref = oracle.marching_cubes(sdf, weights, *args)
    assert len(tri_ref) > 300 and tri.shape == tri_ref.shape and pts.shape == pts_ref.shape
    assert np.array_equal(_sorted_rows(pts), _sorted_rows(pts_ref))
    assert np.array_equal(_triangle_set(tri, pts), _triangle_set(tri_ref, pts_ref))


@pytest.mark.parametrize("grid_dim", [8, 20])
def test_cells_numbered_in_another_order(gpu_ash, oracle, grid_dim):
    """The kernels work the corners of a cell out when the per-cell tables are
    the usual ones (cell = x + G y + G^2 z) and follow the tables otherwise:
    with the cells renumbered by a random permutation, consistently in the
    field, the weights and the three per-cell tables, mesh and points still
    equal the oracle's, which only ever follows the tables."""
    s = 4 if grid_dim == 8 else 3
    g = torch.Generator().manual_seed(890 + grid_dim)
    blocks = torch.stack(torch.meshgrid(*[torch.arange(s)] * 3, indexing="ij"), -1).view(-1, 3)
    blocks = blocks[torch.rand(len(blocks), generator=g) < 0.9]
    grid = gpu_ash.BoundedSparseDenseGrid(
        3, len(blocks) + 5, 1, grid_dim=grid_dim, sparse_grid_dim=s, bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3), device=DEV)
    grid.engine.insert_keys(blocks.int().to(DEV))
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    _, idx = grid.engine.items()
    shape = grid.embeddings.shape[:2]
    m = shape[1]
    sdf = (torch.rand(shape, generator=g) - 0.45).to(DEV)
    weights = (torch.rand(shape, generator=g) * 10).to(DEV)
    perm = torch.randperm(m, generator=g).to(DEV)            # old cell c becomes cell perm[c]
    sdf_p, weights_p = torch.empty_like(sdf), torch.empty_like(weights)
    sdf_p[:, perm], weights_p[:, perm] = sdf, weights
    coords_p = torch.empty_like(grid.cell_coords)
    coords_p[perm] = grid.cell_coords
    c2c_p = torch.empty_like(grid.lut_cell_nb2cell_idx)
    c2c_p[perm] = perm[grid.lut_cell_nb2cell_idx]
    c2g_p = torch.empty_like(grid.lut_cell_nb2grid_nb)
    c2g_p[perm] = grid.lut_cell_nb2grid_nb
    backend = gpu_ash.grid.backend
    usual = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
             grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, grid_dim, 0.02, 0.4)
    renumbered = (idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, coords_p, c2c_p, c2g_p,
                  grid_dim, 0.02, 0.4)
    tri, pts = backend.marching_cubes(sdf_p, weights_p, *renumbered)
    tri_ref, pts_ref = oracle.marching_cubes(sdf_p, weights_p, *renumbered)
    assert len(tri_ref) > 300 and tri.shape == tri_ref.shape
    assert np.array_equal(_sorted_rows(pts), _sorted_rows(pts_ref))
    assert np.array_equal(_triangle_set(tri, pts), _triangle_set(tri_ref, pts_ref))
    tri_u, pts_u = backend.marching_cubes(sdf, weights, *usual)
    assert np.array_equal(_triangle_set(tri, pts), _triangle_set(tri_u, pts_u))
    points = backend.isosurface_extraction(sdf_p, weights_p, *renumbered)
    points_ref = oracle.isosurface_extraction(sdf_p, weights_p, *renumbered)
    assert len(points_ref) > 200
    assert np.array_equal(_sorted_rows(points), _sorted_rows(points_ref))
    assert np.array_equal(_sorted_rows(points),
                          _sorted_rows(backend.isosurface_extraction(sdf, weights, *usual)))


def test_spatial_listing_follows_the_table(gpu_ash):
    """The Z-order listing of the blocks is kept while the table is unchanged
    and rebuilt after every call that can change its keys."""
    from helpers import sort_rows

    grid = gpu_ash.BoundedSparseDenseGrid(
        3, 17 ** 3 + 10, 1, grid_dim=2, sparse_grid_dim=20, bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3), device=DEV)
    r = torch.arange(17, dtype=torch.int32)
    blocks = torch.stack(torch.meshgrid(r, r, r, indexing="ij"), -1).view(-1, 3)
    # inserted in a random order: items() lists by index, i.e. roughly as inserted
    blocks = blocks[torch.randperm(len(blocks), generator=torch.Generator().manual_seed(3))].to(DEV)
    grid.engine.insert_keys(blocks)

    def same_set(listing):
        keys, idx = grid.engine.items()
        a, b = sort_rows(listing[0], listing[1]), sort_rows(keys, idx)
        return torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])

    first = grid._blocks_in_spatial_order()
    assert same_set(first) and len(first[1]) == 17 ** 3
    # neighbours in the listing are neighbours in space far more often than in items() order
    step = (first[0][1:] - first[0][:-1]).abs().sum(dim=1).float().mean()
    table_step = (grid.engine.items()[0][1:] - grid.engine.items()[0][:-1]).abs().sum(dim=1).float().mean()
    assert float(step) < 0.3 * float(table_step)
    again = grid._blocks_in_spatial_order()
    assert again[0] is first[0] and again[1] is first[1]
    grid.engine.insert_keys(torch.tensor([[18, 18, 18], [19, 0, 3]], dtype=torch.int32, device=DEV))
    grown = grid._blocks_in_spatial_order()
    assert len(grown[1]) == 17 ** 3 + 2 and same_set(grown)
    grid.engine.erase(blocks[:100])
    shrunk = grid._blocks_in_spatial_order()
    assert len(shrunk[1]) == 17 ** 3 - 98 and same_set(shrunk)
    # a resized engine is a new table (possibly at the old one's address) that
    # hands the same keys other indices
    grid.engine.resize(grid.engine.capacity + 64)
    resized = grid._blocks_in_spatial_order()
    assert len(resized[1]) == 17 ** 3 - 98 and same_set(resized)

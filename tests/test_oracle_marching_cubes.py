"""Pins of the marching-cubes case table and of the oracle's mesh extraction
(restating ash/src/grid.cu:606-946 behind SparseDenseGrid.marching_cubes,
ash/grid.py:680-711).

The library's case table is written by torch-ash_amd/csrc/gen_mc_table.py.  It
is pinned (a) against the reference: for every case the set of oriented
triangles, and with it the outline of the emitted patch and the number of
triangles, equal those of the reference's table
(tests/golden/mc_case_boundaries.json, written by
tests/golden/make_mc_case_fixture.py from ash/src/mc_macros.h:32-288 and the
reversed order of ash/src/grid.cu:818-841); the oracle takes its table from
that fixture, the library from the generator; (b) by geometry: meshes of closed surfaces
are closed, oriented, have the Euler characteristic of the surface and
enclose its volume, and a random field gives a mesh whose only open edges lie
on the border of the volume -- a wrong entry in any of the 256 rows tears it.

The oracle's passes are pinned by the same mesh properties, by its vertex set
against the iso-surface point extraction, and by a numpy count over the
densified volume for missing blocks and low weights."""
import importlib.util
import json
import os

import numpy as np
import torch

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), os.pardir)
G, S = 4, 4  # cells per block edge, blocks per axis
N = G * S


def _gen():
    path = os.path.join(ROOT, "torch-ash_amd", "csrc", "gen_mc_table.py")
    spec = importlib.util.spec_from_file_location("gen_mc_table", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _outline(tris):
    sides = []
    for a, b, c in tris:
        sides += [(a, b), (b, c), (c, a)]
    return sorted(s for s in sides if (s[1], s[0]) not in sides)


def test_table_outlines_equal_the_reference_for_all_cases():
    gen = _gen()
    with open(os.path.join(ROOT, "tests", "golden", "mc_case_boundaries.json")) as f:
        golden = json.load(f)
    assert len(golden) == 256
    for case in range(256):
        tris = gen.case_triangles(case)
        ref = golden[str(case)]
        assert len(tris) == ref["triangles"], case
        assert _outline(tris) == [tuple(s) for s in ref["outline"]], case


def test_table_triangles_equal_the_reference_for_all_cases():
    """Every row of the library's table holds the reference's triangles: same
    oriented triples (up to where a triple starts), for all 256 cases; and the
    oracle's table, read from the fixture, is that set as well."""
    import ash_oracle

    gen = _gen()
    with open(os.path.join(ROOT, "tests", "golden", "mc_case_boundaries.json")) as f:
        golden = json.load(f)

    def as_set(row):
        tris = [row[i:i + 3] for i in range(0, 15, 3) if row[i] >= 0]
        return sorted(tuple(gen.from_lowest_edge(list(t))) for t in tris)

    table, oracle_table = gen.build_table(), ash_oracle._mc_table()
    polygons = 0
    for case in range(256):
        want = [tuple(t) for t in golden[str(case)]["set"]]
        assert as_set(table[case]) == want, case
        assert as_set(oracle_table[case]) == want, case
        polygons += sum(len(loop) > 3 for loop in gen.case_loops(case))
    assert polygons > 200     # the cuts were a choice in most cases
    # the generator's enumeration really offers a choice: another cut differs
    loop = gen.from_lowest_edge(gen.case_loops(3)[0])
    assert len(loop) == 4 and len(gen.triangulations(loop)) == 2
    assert sorted(gen.triangulations(loop)[0]) != sorted(gen.triangulations(loop)[1])


def test_table_rows_use_exactly_the_crossed_edges():
    gen = _gen()
    table = gen.build_table()
    for case, row in enumerate(table):
        used = {e for e in row if e >= 0}
        crossed = set()
        for e in range(12):
            lo, hi = gen.edge_corners(e)
            assert hi == lo | (1 << (e // 4)) and not lo & (1 << (e // 4))
            if (case >> lo ^ case >> hi) & 1:
                crossed.add(e)
        assert used == crossed, case
        n = sum(1 for v in row if v >= 0)
        assert n % 3 == 0 and all(v == -1 for v in row[n:])
    # complementary cases join the same edges unless a face is ambiguous
    assert len(table[1][:3]) == 3 and sorted(table[1][:3]) == sorted(table[254][:3])


def test_committed_header_is_the_generators_output():
    gen = _gen()
    with open(gen.HEADER) as f:
        assert f.read() == gen.header_text()


# ------------------------------------------------------------------ meshes
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
    keys, idx = grid.engine.items()
    pos = torch.zeros(grid.embeddings.shape[0], G**3, 3)
    pos[idx] = keys.view(-1, 1, 3).float() * G + grid.cell_coords.view(1, -1, 3).float()
    return pos, idx


def _mesh(cpu_ash, grid, sdf, weights, idx, iso=0.0, thr=1.0):
    return cpu_ash.grid.backend.marching_cubes(
        sdf, weights, idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
        grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, G, iso, thr)


def _edge_use(tri):
    """directed edge -> number of triangles that have it"""
    use = {}
    for a, b, c in tri.tolist():
        for e in ((a, b), (b, c), (c, a)):
            use[e] = use.get(e, 0) + 1
    return use


def _closed_and_oriented(tri):
    use = _edge_use(tri)
    return all(n == 1 and use.get((b, a), 0) == 1 for (a, b), n in use.items())


def _signed_volume(tri, pts):
    p = pts.double()[tri.long()]
    return float((p[:, 0] * torch.cross(p[:, 1], p[:, 2], dim=1)).sum() / 6)


def _sort_rows(x):
    x = x.numpy()
    return x[np.lexsort(x.T[::-1])]


def test_sphere_mesh_is_a_closed_outward_sphere(cpu_ash):
    grid = _grid(cpu_ash, _all_blocks())
    pos, idx = _cell_positions(grid)
    centre, radius = torch.tensor([7.3, 8.1, 7.7]), 5.2
    sdf = (pos - centre).norm(dim=-1) - radius
    weights = torch.ones_like(sdf)
    tri, pts = _mesh(cpu_ash, grid, sdf, weights, idx)
    v, f = len(pts), len(tri)
    assert f > 500 and int(tri.min()) == 0 and int(tri.max()) == v - 1
    assert _closed_and_oriented(tri)
    e = len(_edge_use(tri)) // 2
    assert v - e + f == 2
    # normals point out of the sphere (towards larger distances): positive volume
    vol = _signed_volume(tri, pts)
    assert abs(vol / (4 / 3 * np.pi * radius**3) - 1) < 0.03
    # the vertices are the edge crossings of the point extraction
    ref = cpu_ash.grid.backend.isosurface_extraction(
        sdf, weights, idx, grid.grid_coords, grid.lut_grid_nb2grid_idx, grid.cell_coords,
        grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, G, 0.0, 1.0)
    assert np.array_equal(_sort_rows(pts), _sort_rows(ref))
    # a shifted iso value gives the larger sphere
    tri2, pts2 = _mesh(cpu_ash, grid, sdf, weights, idx, iso=1.0)
    assert _closed_and_oriented(tri2)
    assert abs(_signed_volume(tri2, pts2) / (4 / 3 * np.pi * (radius + 1) ** 3) - 1) < 0.03
    # float64 fields give the same connectivity
    tri3, pts3 = _mesh(cpu_ash, grid, sdf.double(), weights.double(), idx)
    assert torch.equal(tri3, tri) and torch.allclose(pts3, pts, atol=1e-5)


def test_torus_mesh_has_genus_one(cpu_ash):
    grid = _grid(cpu_ash, _all_blocks())
    pos, idx = _cell_positions(grid)
    q = pos - torch.tensor([7.6, 7.4, 7.5])
    sdf = torch.sqrt((q[..., :2].norm(dim=-1) - 4.6) ** 2 + q[..., 2] ** 2) - 1.7
    tri, pts = _mesh(cpu_ash, grid, sdf, torch.ones_like(sdf), idx)
    assert _closed_and_oriented(tri)
    v, f, e = len(pts), len(tri), len(_edge_use(tri)) // 2
    assert v - e + f == 0
    # chords of a tube only 1.7 cells thick cut off a noticeable part of it
    assert 0.88 < _signed_volume(tri, pts) / (2 * np.pi**2 * 4.6 * 1.7**2) < 1.0


def test_random_field_mesh_is_open_only_on_the_border(cpu_ash):
    """Exercises every case, ambiguous faces included: surfaces of neighbouring
    cells must meet along shared faces, so an edge that is not shared by two
    opposite triangles can only lie on the border of the volume."""
    grid = _grid(cpu_ash, _all_blocks())
    pos, idx = _cell_positions(grid)
    g = torch.Generator().manual_seed(77)
    sdf = torch.rand(pos.shape[:2], generator=g) - 0.5
    tri, pts = _mesh(cpu_ash, grid, sdf, torch.ones_like(sdf), idx)
    # all 254 surface cases occur
    vol = np.zeros((N, N, N))
    ip = pos[idx].view(-1, 3).long().numpy()
    vol[ip[:, 0], ip[:, 1], ip[:, 2]] = sdf[idx].view(-1).numpy()
    codes = np.zeros((N - 1,) * 3, dtype=np.int64)
    for c in range(8):
        sl = tuple(slice(o, N - 1 + o) for o in (c & 1, c >> 1 & 1, c >> 2 & 1))
        codes |= (vol[sl] < 0).astype(np.int64) << c
    assert len(np.unique(codes)) == 256
    counts = np.array(_gen().triangle_counts())
    assert len(tri) == int(counts[codes].sum())
    use = _edge_use(tri)
    assert max(use.values()) == 1
    on_border = ((pts == 0) | (pts == N - 1)).any(dim=1)
    open_edges = [(a, b) for (a, b) in use if (b, a) not in use]
    assert 0 < len(open_edges) < len(use) // 4
    for a, b in open_edges:
        shared = ((pts[a] == pts[b]) & ((pts[a] == 0) | (pts[a] == N - 1))).any()
        assert bool(on_border[a]) and bool(on_border[b]) and bool(shared)


def test_weights_and_missing_blocks_against_a_dense_count(cpu_ash):
    """A cell takes part only if all eight corners exist and weigh enough
    (ash/src/grid.cu:641-666); vertices are the crossed edges of such cells."""
    g = torch.Generator().manual_seed(78)
    blocks = _all_blocks()
    keep = torch.rand(len(blocks), generator=g) < 0.7
    grid = _grid(cpu_ash, blocks[keep])
    pos, idx = _cell_positions(grid)
    sdf = torch.rand(pos.shape[:2], generator=g) - 0.4
    weights = (torch.rand(pos.shape[:2], generator=g) < 0.9).float() * 3.0
    tri, pts = _mesh(cpu_ash, grid, sdf, weights, idx, iso=0.05, thr=2.0)
    vol = np.full((N, N, N), np.nan)
    ok = np.zeros((N, N, N), dtype=bool)
    ip = pos[idx].view(-1, 3).long().numpy()
    vol[ip[:, 0], ip[:, 1], ip[:, 2]] = sdf[idx].view(-1).numpy() - np.float32(0.05)
    ok[ip[:, 0], ip[:, 1], ip[:, 2]] = (weights[idx].view(-1) >= 2.0).numpy()
    codes = np.zeros((N - 1,) * 3, dtype=np.int64)
    valid = np.ones((N - 1,) * 3, dtype=bool)
    for c in range(8):
        sl = tuple(slice(o, N - 1 + o) for o in (c & 1, c >> 1 & 1, c >> 2 & 1))
        codes |= (np.nan_to_num(vol[sl]) < 0).astype(np.int64) << c
        valid &= ok[sl]
    codes[~valid] = 0
    gen = _gen()
    counts = np.array(gen.triangle_counts())
    assert 200 < len(tri) == int(counts[codes].sum())
    edges = set()
    for x, y, z in zip(*np.nonzero((codes != 0) & (codes != 255))):
        code = int(codes[x, y, z])
        for e in range(12):
            lo, hi = gen.edge_corners(e)
            if (code >> lo ^ code >> hi) & 1:
                edges.add((x + (lo & 1), y + (lo >> 1 & 1), z + (lo >> 2 & 1), e // 4))
    assert len(pts) == len(edges)
    got = set()
    for p in pts.tolist():
        axis = [i for i in range(3) if p[i] != int(p[i])]
        assert len(axis) == 1
        got.add((int(p[0]), int(p[1]), int(p[2]), axis[0]))
    assert got == edges
    assert int(tri.min()) >= 0 and int(tri.max()) == len(pts) - 1


def test_marching_cubes_method_returns_mesh_fields(cpu_ash):
    grid = _grid(cpu_ash, _all_blocks())
    pos, idx = _cell_positions(grid)
    sdf = (pos - torch.tensor([7.3, 8.1, 7.7])).norm(dim=-1) - 5.2
    out = grid.marching_cubes(sdf.unsqueeze(-1), torch.ones_like(sdf).unsqueeze(-1),
                              color_fn=lambda p: p * 0 + 0.5, normal_fn=None)
    if isinstance(out, dict):
        assert set(out) == {"positions", "triangles", "colors"}
        assert out["triangles"].dtype == torch.int32 and out["positions"].shape[1] == 3
        assert out["colors"].shape == out["positions"].shape
        # world units: the unit box holds N cells per axis
        r = (out["positions"] - torch.tensor([7.3, 8.1, 7.7]) * grid.cell_size).norm(dim=-1)
        assert float((r - 5.2 * grid.cell_size).abs().max()) < 0.03 * grid.cell_size
    assert grid.marching_cubes(sdf + 10.0, torch.ones_like(sdf), None, None) is None

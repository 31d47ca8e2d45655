"""GPU parity tests of the fused fusion step: block activation
(ash_grid_activate behind SparseDenseGrid.spatial_init_) and depth integration
(ash_grid_integrate_depth behind ash.fusion) against the reference's statement
of the same step -- candidate expansion + scratch set + insert + find, and the
torch expressions of demo/rgbd_fusion.py:76-110,216-254 -- on the device and,
through the oracle, on the CPU."""
import numpy as np
import pytest
import torch

import workloads
from helpers import sort_rows

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _unfused(gpu_ash, monkeypatch):
    """Makes spatial_init_ take the reference's formulation."""
    monkeypatch.setattr(gpu_ash.grid, "FUSED_ACTIVATION", False)


def _touched(result):
    gc, _, gi, _ = result
    return sort_rows(gc.view(-1, 3), gi.view(-1))


@pytest.mark.parametrize("dilation,bidirectional", [(0, False), (1, False), (1, True), (2, True)])
@pytest.mark.parametrize("bounded", [False, True])
def test_spatial_init_fused_equals_expansion(gpu_ash, monkeypatch, dilation, bidirectional, bounded):
    g = torch.Generator().manual_seed(300 + dilation)
    # image-like ordering: neighbouring rows are neighbouring positions
    pts = (torch.rand(40_000, 3, generator=g).cumsum(0) * 0.002) % 1.6 - 0.3
    pts = pts.to(DEV)

    def make():
        if bounded:
            return gpu_ash.BoundedSparseDenseGrid(
                3, 60_000, 2, grid_dim=8, sparse_grid_dim=24,
                bbox_min=torch.zeros(3), bbox_max=torch.ones(3), device=DEV)
        return gpu_ash.UnBoundedSparseDenseGrid(3, 60_000, 2, 8, cell_size=0.006, device=DEV)

    fused = make()
    first = fused.spatial_init_(pts[:25_000], dilation=dilation, bidirectional=bidirectional)
    second = fused.spatial_init_(pts[15_000:], dilation=dilation, bidirectional=bidirectional)
    with monkeypatch.context() as m:
        _unfused(gpu_ash, m)
        plain = make()
        first_ref = plain.spatial_init_(pts[:25_000], dilation=dilation, bidirectional=bidirectional)
        second_ref = plain.spatial_init_(pts[15_000:], dilation=dilation, bidirectional=bidirectional)
    assert fused.engine.size() == plain.engine.size() > 100
    k_f, _ = fused.engine.items()
    k_p, _ = plain.engine.items()
    assert torch.equal(sort_rows(k_f)[0], sort_rows(k_p)[0])
    for got, ref in ((first, first_ref), (second, second_ref)):
        coords, idx = _touched(got)
        coords_ref, _ = _touched(ref)
        assert torch.equal(coords, coords_ref)
        # every returned index is the row of its block
        found, mask = fused.engine.find(coords.to(DEV))
        assert bool(mask.all()) and torch.equal(found.cpu(), idx)
        assert got[1].shape == ref[1].shape and got[3].shape == ref[3].shape
    if bounded:
        assert int(k_f.min()) >= 0 and int(k_f.max()) < 24


def test_spatial_init_fused_overflow_warns(gpu_ash):
    grid = gpu_ash.UnBoundedSparseDenseGrid(3, 500, 2, 8, cell_size=0.01, device=DEV)
    g = torch.Generator().manual_seed(310)
    pts = (torch.rand(20_000, 3, generator=g) * 4).to(DEV)
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        gc, _, gi, _ = grid.spatial_init_(pts, dilation=1, bidirectional=True)
    assert grid.engine.size() == 500 and gi.shape[0] == 500
    assert gi.min() >= 0 and gi.max() < 500


def _torch_integrate(grid, gc, gi, depth, color, intrinsic, extrinsic, trunc, depth_max):
    """demo/rgbd_fusion.py:76-110 and :232-254 with the embedding layout
    [sdf, (r, g, b,) weight]."""
    cc, ci = grid.cell_coords.view(1, -1, 3), grid.cell_indices.view(1, -1)
    positions = grid.cell_to_world(gc, cc)
    xyz = positions @ extrinsic[:3, :3].t() + extrinsic[:3, 3:].t()
    uvd = xyz @ intrinsic.t()
    d = uvd[:, 2]
    h, w = depth.shape
    u = (uvd[:, 0] / d).round().long()
    v = (uvd[:, 1] / d).round().long()
    inside = (d > 0) & (u >= 0) & (v >= 0) & (u < w) & (v < h)
    reading = torch.zeros_like(d)
    reading[inside] = depth[v[inside], u[inside]]
    sdf = reading - d
    ok = inside & (reading > 0) & (reading < depth_max) & (sdf >= -trunc)
    sdf[sdf >= trunc] = trunc
    weight = ok.float()
    with torch.no_grad():
        emb = grid.embeddings[gi, ci]
        e = emb.shape[-1]
        w_sum = emb[..., e - 1 : e]
        wv = weight.view(w_sum.shape)
        w_new = w_sum + wv
        emb[..., 0:1] = (emb[..., 0:1] * w_sum + sdf.view(w_sum.shape) * wv) / (w_new + 1e-6)
        if color is not None:
            rgb = torch.zeros((len(d), 3), device=d.device)
            rgb[inside] = color[v[inside], u[inside], :]
            emb[..., 1:4] = (emb[..., 1:4] * w_sum + rgb.view(*w_sum.shape[:2], 3) * wv) / (w_new + 1e-6)
        emb[..., e - 1 : e] = w_new
        grid.embeddings[gi, ci] = emb
    return u, v, d


@pytest.mark.parametrize("with_color,bounded", [(False, False), (True, False), (True, True)])
def test_integrate_depth_equals_torch_expressions(gpu_ash, with_color, bounded):
    scene = workloads.FusionScene(width=320, height=240)
    e = 5 if with_color else 2
    g = torch.Generator().manual_seed(320)

    def make():
        if bounded:
            grid = gpu_ash.BoundedSparseDenseGrid(
                3, 30_000, e, grid_dim=8, sparse_grid_dim=32,
                bbox_min=-1.7 * torch.ones(3), bbox_max=1.7 * torch.ones(3), device=DEV)
        else:
            grid = gpu_ash.UnBoundedSparseDenseGrid(3, 30_000, e, 8, cell_size=0.015, device=DEV)
        with torch.no_grad():
            grid.embeddings.zero_()
        return grid

    fused, plain = make(), make()
    intrinsic = scene.intrinsic.to(DEV)
    n_cells = flips = 0
    for frame in (0, 7, 14, 21):
        ext = scene.pose(frame)
        depth = scene.depth(ext)
        color = torch.rand(*depth.shape, 3, generator=g) if with_color else None
        pts = scene.unproject(depth, ext).to(DEV)
        depth, ext = depth.to(DEV), ext.to(DEV)
        color = color.to(DEV) if with_color else None
        gc, _, gi, _ = fused.spatial_init_(pts, dilation=1, bidirectional=True)
        gc2, _, gi2, _ = plain.spatial_init_(pts, dilation=1, bidirectional=True)
        assert torch.equal(_touched((gc, None, gi, None))[0], _touched((gc2, None, gi2, None))[0])
        gpu_ash.fusion.integrate_depth(fused, gc, gi, depth, intrinsic, ext, 0.04, 6.0, color)
        _torch_integrate(plain, gc2, gi2, depth, color, intrinsic, ext, 0.04, 6.0)
    # rows are allocated in parallel, so the two grids are compared block by block

    def by_key(grid):
        keys, idx = grid.engine.items()
        order = sort_rows(keys, idx)
        return order[0], grid.embeddings.detach().cpu()[order[1]]

    (keys_a, a), (keys_b, b) = by_key(fused), by_key(plain)
    assert torch.equal(keys_a, keys_b)
    # Observations decided by a rounding (pixel coordinate on x.5, distance on
    # the truncation threshold) may differ between the fused projection and
    # torch's matrix products; all others must agree to fp32 rounding.
    same = a[..., -1] == b[..., -1]
    n_cells, flips = same.numel(), int((~same).sum())
    assert int(b[..., -1].sum()) > 100_000
    assert flips < 5e-4 * n_cells
    close = torch.isclose(a[..., 0], b[..., 0], rtol=1e-3, atol=2e-4)
    assert int((~close & same).sum()) < 5e-4 * n_cells
    if with_color:
        close_rgb = torch.isclose(a[..., 1:4], b[..., 1:4], rtol=1e-3, atol=1e-3).all(-1)
        assert int((~close_rgb & same).sum()) < 2e-3 * n_cells


@pytest.mark.parametrize("width,height,poses,capacity",
                         [(160, 120, (0, 10, 20), 20_000), (640, 480, (0, 33, 66), 80_000)])
def test_fused_fusion_against_oracle_harness(gpu_ash, oracle, monkeypatch, width, height, poses,
                                             capacity):
    """Configuration 5, at reduced size and at its full frame size (640 x 480
    depth frames, 307 200 positions and 8.3 M candidate keys per frame,
    capacity 80 000 as in the reference's demo): the fused step on the device
    against the reference's formulation run on the CPU with the oracle as
    backend."""
    import ash.core
    import ash.grid
    import ash.grid_query

    scene = workloads.FusionScene(width=width, height=height)
    frames = []
    for f in poses:
        ext = scene.pose(f)
        depth = scene.depth(ext)
        frames.append((scene.unproject(depth, ext), depth, ext))

    def run(device, fused):
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, capacity, 2, 8, cell_size=0.015, device=device)
        touched = [
            workloads.fuse_frame(grid, p.to(device), d.to(device), scene.intrinsic.to(device),
                                 e.to(device), trunc=0.04, fused=fused)
            for p, d, e in frames
        ]
        keys, idx = grid.engine.items()
        order = sort_rows(keys, idx)
        return touched, order[0], grid.embeddings.detach().cpu()[order[1]]

    touched_gpu, keys_gpu, cells_gpu = run(DEV, True)
    with monkeypatch.context() as m:
        for mod in (ash.core, ash.grid, ash.grid_query):
            m.setattr(mod, "backend", oracle)
        touched_cpu, keys_cpu, cells_cpu = run(torch.device("cpu"), False)
    assert touched_gpu == touched_cpu and len(keys_gpu) > 5000
    assert torch.equal(keys_gpu, keys_cpu)
    # A cell whose projection falls on a pixel boundary (x.5) may read the
    # neighbouring pixel on the other side (fused multiply-adds against torch's
    # matrix products): its weight flips when one of the two pixels has no
    # valid reading, its distance changes when both have.  Their fraction is
    # bounded; every other cell agrees to fp32 rounding.
    same = cells_gpu[..., 1] == cells_cpu[..., 1]
    flipped = float((~same).float().mean())
    assert flipped < 5e-4, flipped
    close = torch.isclose(cells_gpu[..., 0], cells_cpu[..., 0], rtol=1e-3, atol=2e-4)
    other_pixel = float((same & ~close).float().mean())
    assert other_pixel < 5e-4, other_pixel
    assert float(cells_gpu[..., 1].sum()) > 1e5


def test_frames_without_read_back_equal_counted_frames(gpu_ash):
    """ash.fusion.fuse_frame(count_blocks=False): activation, listing and
    integration are queued with the number of touched blocks left on the device
    (ash_grid_integrate_depth_touched).  Same blocks and, block by block, the
    same embedding rows bit for bit as the frames that read the number back;
    an overfull table shows at the next call that reads the counters."""
    scene = workloads.FusionScene(width=320, height=240)
    intrinsic = scene.intrinsic.to(DEV)
    frames = []
    for f in (0, 9, 18, 27, 36):
        ext = scene.pose(f)
        depth = scene.depth(ext)
        frames.append((scene.unproject(depth, ext).to(DEV), depth.to(DEV), ext.to(DEV)))

    def run(count_blocks, capacity=30_000):
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, capacity, 2, 8, cell_size=0.015, device=DEV)
        with torch.no_grad():
            grid.embeddings.zero_()
        touched = [gpu_ash.fusion.fuse_frame(grid, p, d, intrinsic, e, 0.04, 6.0,
                                             count_blocks=count_blocks) for p, d, e in frames]
        keys, idx = grid.engine.items()
        order = sort_rows(keys, idx)
        return grid, touched, order[0], grid.embeddings.detach()[order[1].to(DEV)].cpu()

    _, touched, keys_a, cells_a = run(True)
    grid, nothing, keys_b, cells_b = run(False)
    assert all(t > 100 for t in touched) and nothing == [None] * len(frames)
    assert torch.equal(keys_a, keys_b) and len(keys_a) > 1000
    assert torch.equal(cells_a, cells_b)
    assert float(cells_a[..., 1].sum()) > 1e5
    # the count of the last listing is still in the counters
    assert grid.engine.backend.status()["touched"] == touched[-1]
    # too small a table: the frames run, the table is full, the next insert warns
    small, _, keys_c, _ = run(False, capacity=1500)
    assert small.engine.size() == 1500 and len(keys_c) == 1500
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        small.engine.insert_keys(torch.tensor([[900, 900, 900]], dtype=torch.int32, device=DEV))


@pytest.mark.parametrize("capacity", [5, 1000, 80_000, 131_073, 200_000, 1_048_576])
def test_touched_rows_are_listed_in_order(gpu_ash, capacity):
    """ash_grid_collect_touched against torch.nonzero: ascending rows, their
    coordinates, flags cleared, count in the sixth status value -- for tables of
    one workgroup's chunk and of many, with one and with two words of flags per
    thread, that end inside a word, and for flags that start at a 4-byte but not
    at a 16-byte boundary.  Three calls in a row on one table: the workgroups'
    ticket counter has to be back at zero after each."""
    engine = gpu_ash.ASHEngine(3, capacity, DEV)
    backend = engine.backend
    g = torch.Generator().manual_seed(capacity)
    for density, shift in ((0.0, 0), (0.05, 4), (1.0, 0)):
        store = torch.zeros(capacity + 16, dtype=torch.uint8, device=DEV)
        flags = store[shift : shift + capacity]
        flags.copy_((torch.rand(capacity, generator=g) < density).to(torch.uint8))
        flags.mul_(torch.randint(1, 255, (capacity,), generator=g, dtype=torch.uint8).to(DEV))
        coords = torch.randint(-1000, 1000, (capacity, 3), generator=g, dtype=torch.int32).to(DEV)
        expected = flags.nonzero().view(-1)
        rows = torch.full((capacity,), -1, dtype=torch.int64, device=DEV)
        out_coords = torch.zeros((capacity, 3), dtype=torch.int32, device=DEV)
        rc = backend._lib.ash_grid_collect_touched(
            backend._handle, flags.data_ptr(), coords.data_ptr(), rows.data_ptr(),
            out_coords.data_ptr(), backend._stream())
        assert rc == 0, backend._lib.ash_last_error().decode()
        n = backend.status()["touched"]
        assert n == len(expected)
        assert torch.equal(rows[:n], expected) and torch.equal(out_coords[:n], coords[expected])
        assert bool((rows[n:] == -1).all()) and int(flags.sum()) == 0

"""GPU parity tests of the fused fusion step: block activation
(ash_grid_activate behind SparseDenseGrid.spatial_init_) and depth integration
(ash_grid_integrate_depth behind ash.fusion) against the reference's statement
of the same step -- candidate expansion + scratch set + insert + find, and the
torch expressions of demo/rgbd_fusion.py:76-110,216-254 -- on the device and,
through the oracle, on the CPU."""
import numpy as np
import pytest
import torch

import ctypes

import workloads
from ash import common
from helpers import RawBlockMap, sort_rows

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


# What a cell observes in a frame is decided by roundings of its projection:
# the pixel it reads (coordinates rounded to the nearest integer), whether it
# lies in front of the camera, whether its distance passes the truncation
# threshold.  The fused kernel projects with fused multiply-adds where torch
# calls matrix products; either way every product and partial sum is rounded
# (up to eighteen roundings on the way to a coordinate on the two sides
# together, each at most 2^-24 of the sum of |terms|, adding up like a random
# walk: K_PROJ = 16 is more than six standard deviations).  A cell is "decided"
# when no such error changes its observation: with `slack` = K_PROJ * 2^-24 *
# (sum of |terms|) of numerator and depth, the projected coordinates stay clear
# of x.5 by what that slack moves them, and depth and signed distance stay clear
# of zero and of the truncation threshold.  Decided cells read the same pixel
# on both sides and their update is the same arithmetic on inputs that differ by
# at most `slack` in the distance: weights and colours equal bit for bit, the
# distance channel within the stated fp32 tolerance plus `slack`.  The others
# may differ; their number is what the geometry makes it (bounded here at 5 %),
# and those of them that do differ stay below 5e-4 of the cells.
K_PROJ = 16.0
RTOL32, ATOL32 = 1e-5, 1e-6


def _decided(positions, intrinsic, extrinsic, depth, trunc):
    """float64 projection of world positions (n, 3): (decided bool[n],
    slack of the distance float64[n])."""
    p = positions.detach().double().cpu()
    rot, shift = extrinsic[:3, :3].double().cpu(), extrinsic[:3, 3].double().cpu()
    k = intrinsic.double().cpu()
    cam = p @ rot.t() + shift
    slack = K_PROJ * 2.0**-24 * ((p.abs() @ rot.abs().t() + shift.abs()) @ k.abs().t())
    uvd = cam @ k.t()
    d = uvd[:, 2]
    u, v = uvd[:, 0] / d, uvd[:, 1] / d
    h, w = depth.shape
    ui, vi = u.round(), v.round()
    inside = (d > 0) & (ui >= 0) & (vi >= 0) & (ui < w) & (vi < h)
    reading = torch.zeros_like(d)
    reading[inside] = depth.double().cpu()[vi[inside].long(), ui[inside].long()]

    def off_half(c, slack_c):
        # numerator and denominator each off by their slack, and the quotient rounded
        moved = (slack_c + c.abs() * slack[:, 2]) / d.abs() + 2.0**-22 * c.abs()
        return ((c - c.floor()) - 0.5).abs() > moved

    decided = (d.abs() > slack[:, 2]) & ((d < 0) | (off_half(u, slack[:, 0]) & off_half(v, slack[:, 1])))
    decided &= ((reading - d) + trunc).abs() > slack[:, 2]
    return decided, slack[:, 2]


def _assert_same_update(got, ref, decided, slack, what):
    """got / ref (cells, E) after one frame from the same state."""
    got, ref = got.detach().cpu(), ref.detach().cpu()
    e = got.shape[-1]
    assert torch.equal(got[decided, e - 1], ref[decided, e - 1]), f"{what}: weights"
    if e >= 5:
        assert torch.equal(got[decided, 1:4], ref[decided, 1:4]), f"{what}: colours"
    diff = (got[:, 0].double() - ref[:, 0].double()).abs()
    within = diff <= RTOL32 * ref[:, 0].double().abs() + ATOL32 + slack
    worst = int((diff * decided).argmax())
    assert bool(within[decided].all()), (what, float(diff[worst]), float(slack[worst]))
    assert float((~decided).float().mean()) < 0.05, what
    differ = ~decided & (~within | (got[:, e - 1] != ref[:, e - 1]))
    assert float(differ.float().mean()) < 5e-4, (what, float(differ.float().mean()))


@pytest.mark.parametrize("with_color,bounded", [(False, False), (True, False), (True, True)])
def test_integrate_depth_equals_torch_expressions(gpu_ash, with_color, bounded):
    """ash_grid_integrate_depth against the torch expressions of
    demo/rgbd_fusion.py:76-110,232-254, frame by frame from the same state:
    same observation and fp32-rounding agreement on every decided cell."""
    scene = workloads.FusionScene(width=320, height=240)
    e = 5 if with_color else 2
    g = torch.Generator().manual_seed(320)
    if bounded:
        grid = gpu_ash.BoundedSparseDenseGrid(
            3, 30_000, e, grid_dim=8, sparse_grid_dim=32,
            bbox_min=-1.7 * torch.ones(3), bbox_max=1.7 * torch.ones(3), device=DEV)
    else:
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, 30_000, e, 8, cell_size=0.015, device=DEV)
    with torch.no_grad():
        grid.embeddings.zero_()
    intrinsic = scene.intrinsic.to(DEV)
    observed = 0
    for frame in (0, 7, 14, 21):
        ext = scene.pose(frame)
        depth = scene.depth(ext)
        color = torch.rand(*depth.shape, 3, generator=g) if with_color else None
        pts = scene.unproject(depth, ext).to(DEV)
        depth, ext = depth.to(DEV), ext.to(DEV)
        color = color.to(DEV) if with_color else None
        gc, cc, gi, _ = grid.spatial_init_(pts, dilation=1, bidirectional=True)
        before = grid.embeddings.detach().clone()
        gpu_ash.fusion.integrate_depth(grid, gc, gi, depth, intrinsic, ext, 0.04, 6.0, color)
        fused = grid.embeddings.detach()[gi.view(-1)].reshape(-1, e).clone()
        untouched = torch.ones(len(before), dtype=torch.bool, device=DEV)
        untouched[gi.view(-1)] = False
        assert torch.equal(grid.embeddings.detach()[untouched], before[untouched])
        with torch.no_grad():
            grid.embeddings.copy_(before)
        _torch_integrate(grid, gc, gi, depth, color, intrinsic, ext, 0.04, 6.0)
        plain = grid.embeddings.detach()[gi.view(-1)].reshape(-1, e)
        decided, slack = _decided(grid.cell_to_world(gc, cc), intrinsic, ext, depth, 0.04)
        _assert_same_update(fused, plain, decided, slack, f"frame {frame}")
        observed += int((plain[:, -1] != before[gi.view(-1)].reshape(-1, e)[:, -1]).sum())
    assert observed > 100_000


@pytest.mark.parametrize("width,height,poses,capacity",
                         [(160, 120, (0, 10, 20), 20_000), (640, 480, (0, 33, 66), 80_000)])
def test_fused_fusion_against_oracle_harness(gpu_ash, oracle, monkeypatch, width, height, poses,
                                             capacity):
    """Configuration 5, at reduced size and at its full frame size (640 x 480
    depth frames, 307 200 positions and 8.3 M candidate keys per frame,
    capacity 80 000 as in the reference's demo): the fused step on the device
    against the reference's formulation run on the CPU with the oracle as
    backend, frame by frame.  Same blocks touched and stored; every decided
    cell (see above) updated alike; after each frame the device's rows are set
    to the CPU's, block by block, so that every frame starts from one state."""
    import ash.core
    import ash.grid
    import ash.grid_query

    scene = workloads.FusionScene(width=width, height=height)
    cpu = torch.device("cpu")

    class on_oracle:
        def __enter__(self):
            self.m = monkeypatch.context()
            m = self.m.__enter__()
            for mod in (ash.core, ash.grid, ash.grid_query):
                m.setattr(mod, "backend", oracle)

        def __exit__(self, *exc):
            return self.m.__exit__(*exc)

    grid_gpu = gpu_ash.UnBoundedSparseDenseGrid(3, capacity, 2, 8, cell_size=0.015, device=DEV)
    with on_oracle():
        grid_cpu = gpu_ash.UnBoundedSparseDenseGrid(3, capacity, 2, 8, cell_size=0.015, device=cpu)
    observed = 0
    for f in poses:
        ext = scene.pose(f)
        depth = scene.depth(ext)
        pts = scene.unproject(depth, ext)
        touched_gpu = workloads.fuse_frame(grid_gpu, pts.to(DEV), depth.to(DEV),
                                           scene.intrinsic.to(DEV), ext.to(DEV), trunc=0.04,
                                           fused=True)
        with on_oracle():
            before = grid_cpu.embeddings.detach().clone()
            touched_cpu = workloads.fuse_frame(grid_cpu, pts, depth, scene.intrinsic, ext,
                                               trunc=0.04, fused=False)
            keys_cpu, idx_cpu = sort_rows(*grid_cpu.engine.items())
        keys_gpu, idx_gpu = sort_rows(*grid_gpu.engine.items())
        assert touched_gpu == touched_cpu and torch.equal(keys_gpu, keys_cpu)
        cells_cpu = grid_cpu.embeddings.detach()[idx_cpu]
        cells_gpu = grid_gpu.embeddings.detach()[idx_gpu.to(DEV)].cpu()
        # every active block is compared: the blocks the frame did not touch
        # hold what they held before on both sides
        positions = grid_cpu.cell_to_world(keys_cpu.view(-1, 1, 3),
                                           grid_cpu.cell_coords.view(1, -1, 3))
        decided, slack = _decided(positions, scene.intrinsic, ext, depth, 0.04)
        _assert_same_update(cells_gpu.reshape(-1, 2), cells_cpu.reshape(-1, 2), decided, slack,
                            f"pose {f}")
        observed += int((cells_cpu[..., 1] != before[idx_cpu][..., 1]).sum())
        with torch.no_grad():
            grid_gpu.embeddings[idx_gpu.to(DEV)] = cells_cpu.to(DEV)
    assert len(keys_gpu) > 5000 and observed > 1e5


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

    def run(count_blocks, capacity=30_000, listing=False):
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, capacity, 2, 8, cell_size=0.015, device=DEV)
        if listing:
            # a transform of the user's: the frame cannot apply it inside its
            # kernels and takes the activation that lists the touched rows
            own = grid.transform_world_to_cell
            grid.transform_world_to_cell = lambda x: own(x)
        with torch.no_grad():
            grid.embeddings.zero_()
        touched = [gpu_ash.fusion.fuse_frame(grid, p, d, intrinsic, e, 0.04, 6.0,
                                             count_blocks=count_blocks) for p, d, e in frames]
        keys, idx = grid.engine.items()
        order = sort_rows(keys, idx)
        return grid, touched, order[0], grid.embeddings.detach()[order[1].to(DEV)].cpu()

    _, touched, keys_a, cells_a = run(True)
    assert all(t > 100 for t in touched) and float(cells_a[..., 1].sum()) > 1e5
    for listing in (False, True):
        grid, nothing, keys_b, cells_b = run(False, listing=listing)
        assert nothing == [None] * len(frames)
        assert torch.equal(keys_a, keys_b) and len(keys_a) > 1000
        assert torch.equal(cells_a, cells_b)
        table = grid.engine.backend
        if listing:
            # the count of the last listing is still in the counters
            assert table.status()["touched"] == touched[-1]
        # no flag is left standing either way
        assert int(table._touched.sum()) == 0
    # too small a table: the frames run, the table is full, the next insert warns
    small, _, keys_c, _ = run(False, capacity=1500)
    assert small.engine.size() == 1500 and len(keys_c) == 1500
    with pytest.warns(UserWarning, match="exceeds the hash map capacity"):
        small.engine.insert_keys(torch.tensor([[900, 900, 900]], dtype=torch.int32, device=DEV))


def test_activation_from_world_positions_equals_activation_from_cells(gpu_ash):
    """ash_grid_activate_positions (world positions, run heads found per
    workgroup, no scratch) against ash_grid_activate on torch's
    (x - origin) / cell_size, through the C ABI on two identical maps, call
    after call: same blocks stored, same rows' coordinates flagged, same
    answers to look-ups.  Batches that end inside a workgroup's share of the
    positions, every dilation, bounds that cut candidates off, positions in
    cell units; positions in no order at all (every workgroup then meets blocks
    that others are storing at that moment, and has to leave their flags to
    them) and, before the last batches, an erase of every second block, which
    leaves tombstones and slots whose index word still names an earlier
    tenant."""
    lib = common.load_library()
    capacity = 60_000
    plain, direct = RawBlockMap(lib, capacity, DEV), RawBlockMap(lib, capacity, DEV)
    g = torch.Generator().manual_seed(77)
    cases = (  # n, dilation, two-sided, origin, cell size, bounds
        (40_001, 1, 1, (-1.5, 0.25, 3.0), 0.015, (-1000, 1000)),
        (9_000, 2, 1, (-1.5, 0.25, 3.0), 0.015, (-1000, 1000)),
        (5_003, 0, 0, None, 1.0, (-1000, 1000)),
        (127, 1, 0, (0.5, 0.5, 0.5), 0.1, (-1000, 1000)),
        (20_000, 1, 1, (-2.0, -2.0, -2.0), 0.02, (0, 11)),
        (30_000, 1, 1, (4.0, 4.0, 4.0), 0.015, (-1000, 1000)),     # shuffled, new ground
        (30_000, 1, 1, (-1.5, 0.25, 3.0), 0.015, (-1000, 1000)),   # shuffled, after the erase
        (40_001, 1, 1, (-1.5, 0.25, 3.0), 0.015, (-1000, 1000)),
        (12_000, 2, 1, (9.0, 9.0, 9.0), 0.015, (-1000, 1000)),     # shuffled, new ground, 125 each
    )
    seen = []
    try:
        for case, (n, dilation, two_sided, origin, cell_size, (lo, hi)) in enumerate(cases):
            # image-like ordering: neighbouring rows are neighbouring positions
            cells = ((torch.rand(n, 3, generator=g).cumsum(0) * 0.3) % 260.0) - 50.0
            if case in (5, 6, 8):
                cells = cells[torch.randperm(n, generator=g)]
            if case == 6:
                stored = torch.unique(torch.cat(seen), dim=0)[::2].to(DEV).contiguous()
                for m in (plain, direct):
                    assert lib.ash_map_erase(m.handle, stored.data_ptr(), stored.shape[0], m.stream) == 0
                assert plain.size() == direct.size()
            x = (cells * cell_size + (torch.tensor(origin) if origin else 0.0)).to(DEV).contiguous()
            o = torch.tensor(origin, device=DEV) if origin else None
            cells = ((x - o) / cell_size if origin else x / cell_size).contiguous()
            heads = torch.empty(64 + 3 * n, dtype=torch.int32, device=DEV)
            rc = lib.ash_grid_activate(plain.handle, cells.data_ptr(), n, 8, dilation, two_sided,
                                       lo, hi, plain.touched.data_ptr(), plain.coords.data_ptr(),
                                       heads.data_ptr(), plain.stream)
            assert rc == 0, lib.ash_last_error()
            rc = lib.ash_grid_activate_positions(
                direct.handle, x.data_ptr(), n, o.data_ptr() if origin else None,
                ctypes.c_float(cell_size), 8, dilation, two_sided, lo, hi,
                direct.touched.data_ptr(), direct.coords.data_ptr(), direct.stream)
            assert rc == 0, lib.ash_last_error()
            torch.cuda.synchronize()
            size = plain.size()
            assert direct.size() == size and 20 < size < capacity
            coords_p, rows_p = plain.touched_blocks()
            coords_d, rows_d = direct.touched_blocks()
            assert coords_p.shape[0] > 20 and torch.equal(coords_d, coords_p)
            assert int(coords_p.min()) >= lo and int(coords_p.max()) <= hi
            for m, rows in ((plain, rows_p), (direct, rows_d)):
                idx, mask = m.find(coords_p.to(DEV))
                assert bool(mask.all()) and torch.equal(idx.cpu(), rows.cpu())
            probe = torch.cat([coords_p[::3] + 1, coords_p[::5]]).to(DEV).contiguous()
            assert torch.equal(plain.find(probe)[1], direct.find(probe)[1])
            seen.append(coords_p)
    finally:
        plain.close()
        direct.close()


@pytest.mark.parametrize("grid_dim,e,bounded", [(8, 2, False), (8, 5, False), (4, 2, True), (8, 2, True)])
def test_integration_by_flags_equals_integration_by_listing(gpu_ash, grid_dim, e, bounded):
    """ash_grid_integrate_depth_flagged (after ash_grid_activate_positions)
    against ash_grid_integrate_depth over the listing spatial_init_ returns, on
    two grids from the same state, frame after frame: the same blocks and,
    block by block, the same rows bit for bit; rows of untouched blocks keep
    what they held; no flag is left standing.  Block edges of 8 with
    distance + weight rows take kernels of their own; the others the general
    ones."""
    scene = workloads.FusionScene(width=320, height=240)
    rnd = torch.Generator().manual_seed(5)
    intrinsic = scene.intrinsic.to(DEV)
    cell_size = 0.015 * 8 / grid_dim

    def new_grid():
        if bounded:
            grid = gpu_ash.BoundedSparseDenseGrid(
                3, 30_000, e, grid_dim=grid_dim, sparse_grid_dim=32,
                bbox_min=-1.7 * torch.ones(3), bbox_max=1.7 * torch.ones(3), device=DEV)
        else:
            grid = gpu_ash.UnBoundedSparseDenseGrid(3, 30_000, e, grid_dim, cell_size=cell_size,
                                                    device=DEV)
        with torch.no_grad():
            # (zeros: the two grids hand out their rows in different orders)
            grid.embeddings.zero_()
        return grid

    listed, flagged = new_grid(), new_grid()
    for frame in (0, 11, 22):
        ext = scene.pose(frame)
        depth = scene.depth(ext)
        color = torch.rand(*depth.shape, 3, generator=rnd).to(DEV) if e >= 5 else None
        pts = scene.unproject(depth, ext).to(DEV)
        depth, ext = depth.to(DEV), ext.to(DEV)
        gc, _, gi, _ = listed.spatial_init_(pts, dilation=1, bidirectional=True)
        gpu_ash.fusion.integrate_depth(listed, gc, gi, depth, intrinsic, ext, 0.04, 6.0, color)
        assert gpu_ash.fusion.fuse_frame(flagged, pts, depth, intrinsic, ext, 0.04, 6.0, color,
                                         count_blocks=False) is None
        keys_l, idx_l = sort_rows(*listed.engine.items())
        keys_f, idx_f = sort_rows(*flagged.engine.items())
        assert torch.equal(keys_l, keys_f) and len(gi) > 100
        assert torch.equal(listed.embeddings.detach()[idx_l.to(DEV)],
                           flagged.embeddings.detach()[idx_f.to(DEV)])
        assert int(flagged.engine.backend._touched.sum()) == 0
    # rows no block owns were not written
    free = torch.ones(30_000, dtype=torch.bool, device=DEV)
    free[idx_f.to(DEV)] = False
    assert int(flagged.embeddings.detach()[free].count_nonzero()) == 0


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

"""Seeded synthetic workloads of the benchmark configurations, shared by
bench.py and the parity tests.  Every generator takes the sizes as arguments so
that the tests can run the same construction at sizes the CPU oracle finishes
in seconds; the defaults are the full benchmark sizes.

The generators only use torch and run on any device; nothing here touches the
hash map or the oracle except `build_grid`, which drives the package's own
modules.
"""
import math
from typing import Dict, Tuple

import torch


def _gen(device, seed: int) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    return g


# --------------------------------------------------------------------- cfg 1
def hashset_uniform_keys(
    num_unique: int = 500_000, lo: int = -256, hi: int = 256, device="cpu", seed: int = 1
) -> Dict[str, torch.Tensor]:
    """Configuration 1: `num_unique` draws from [lo, hi)^3, every draw present
    twice (50 % deliberate duplicates) in random order; queries are half
    re-draws from the inserted rows and half fresh uniform draws."""
    g = _gen(device, seed)
    base = torch.randint(lo, hi, (num_unique, 3), generator=g, device=device, dtype=torch.int32)
    insert = torch.cat([base, base])[torch.randperm(2 * num_unique, generator=g, device=device)]
    hits = base[torch.randint(num_unique, (num_unique,), generator=g, device=device)]
    fresh = torch.randint(lo, hi, (num_unique, 3), generator=g, device=device, dtype=torch.int32)
    queries = torch.cat([hits, fresh])[torch.randperm(2 * num_unique, generator=g, device=device)]
    return {"insert_keys": insert.contiguous(), "query_keys": queries.contiguous()}


# --------------------------------------------------------------------- cfg 2
def _sphere_scene(num_spheres, r_lo, r_hi, c_lo, c_hi, device, g):
    radii = torch.rand(num_spheres, generator=g, device=device) * (r_hi - r_lo) + r_lo
    centres = torch.rand(num_spheres, 3, generator=g, device=device) * (c_hi - c_lo) + c_lo
    return radii, centres


def _surface_points(radii, centres, n, g):
    """n points on the union of sphere surfaces, spheres drawn by area."""
    device = radii.device
    pick = torch.multinomial(radii * radii, n, replacement=True, generator=g)
    d = torch.randn(n, 3, generator=g, device=device)
    d = d / d.norm(dim=1, keepdim=True).clamp_min(1e-12)
    return centres[pick] + radii[pick].unsqueeze(1) * d


def _pack21(k: torch.Tensor) -> torch.Tensor:
    k = k.long() + (1 << 20)
    return k[:, 0] | (k[:, 1] << 21) | (k[:, 2] << 42)


def _unpack21(p: torch.Tensor) -> torch.Tensor:
    m = (1 << 21) - 1
    return torch.stack([(p & m), (p >> 21) & m, (p >> 42) & m], dim=1).sub_(1 << 20).int()


def hashmap_sphere_voxels(
    num_keys: int = 16_000_000,
    num_spheres: int = 64,
    voxel_size: float = 0.01,
    hit_fraction: float = 0.7,
    device="cpu",
    seed: int = 2,
) -> Dict[str, torch.Tensor]:
    """Configuration 2: `num_keys` distinct voxel coordinates of points on 64
    random spheres (radii U[0.5,3], centres U[-20,20]^3, voxel 0.01), fp32
    values color[.,3] and depth[.,1], and as many queries: 70 % drawn from the
    keys, 30 % keys moved far outside the scene (certain misses)."""
    g = _gen(device, seed)
    radii, centres = _sphere_scene(num_spheres, 0.5, 3.0, -20.0, 20.0, device, g)
    packed = torch.empty(0, dtype=torch.int64, device=device)
    chunk = max(min(num_keys, 8_000_000), 1024)
    while packed.numel() < num_keys:
        pts = _surface_points(radii, centres, chunk, g)
        vox = torch.floor(pts / voxel_size).int()
        packed = torch.unique(torch.cat([packed, _pack21(vox)]))
    packed = packed[torch.randperm(packed.numel(), generator=g, device=device)[:num_keys]]
    keys = _unpack21(packed).contiguous()
    color = torch.rand(num_keys, 3, generator=g, device=device)
    depth = torch.rand(num_keys, 1, generator=g, device=device)
    n_hit = int(round(hit_fraction * num_keys))
    hits = keys[torch.randint(num_keys, (n_hit,), generator=g, device=device)]
    misses = keys[torch.randint(num_keys, (num_keys - n_hit,), generator=g, device=device)]
    misses = misses + torch.tensor([100_000, 0, 0], dtype=torch.int32, device=device)
    queries = torch.cat([hits, misses])[torch.randperm(num_keys, generator=g, device=device)]
    return {
        "keys": keys,
        "color": color,
        "depth": depth,
        "query_keys": queries.contiguous(),
    }


# ----------------------------------------------------------------- cfg 3 / 4
def surface_blocks(
    num_blocks: int = 200_000,
    num_spheres: int = 32,
    sparse_grid_dim: int = 128,
    device="cpu",
    seed: int = 3,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Block coordinates (int32[num_blocks,3], inside [0,sparse_grid_dim)^3)
    around the union of `num_spheres` random spheres in the unit cube, each
    surface block dilated by its +1 neighbours so that interpolation finds its
    corner blocks.  Spheres are added one by one until `num_blocks` is reached;
    the last sphere is cut (in key order) to land exactly on it.  Also returns
    the sphere radii and centres."""
    g = _gen(device, seed)
    s = sparse_grid_dim
    # radii scale with the block budget so that small test grids still get
    # several spheres: area ~ num_blocks / (num_spheres * 8) blocks per sphere
    r_blocks = math.sqrt(max(num_blocks, 64) / (num_spheres * 8.0 * 4 * math.pi)) * 1.9
    r_blocks = min(r_blocks, s * 0.22)
    have = torch.empty(0, dtype=torch.int64, device=device)
    radii_all, centres_all = [], []
    corner = torch.tensor(
        [[(c >> d) & 1 for d in range(3)] for c in range(8)], dtype=torch.int64, device=device
    )
    guard = 0
    while have.numel() < num_blocks:
        guard += 1
        assert guard < 100000, "surface_blocks cannot reach the requested block count"
        r = (torch.rand(1, generator=g, device=device) * 0.8 + 0.6) * r_blocks
        c = torch.rand(1, 3, generator=g, device=device) * (s - 2 * (r + 2)) + (r + 2)
        n_pts = int(60 * float(r) ** 2) + 64
        pts = _surface_points(r, c, n_pts, g)
        blk = torch.floor(pts).long().clamp_(0, s - 2)
        blk = (blk.view(-1, 1, 3) + corner.view(1, 8, 3)).view(-1, 3)
        new = torch.unique(_pack21(blk))
        fresh = new[~torch.isin(new, have)]
        room = num_blocks - have.numel()
        have = torch.cat([have, fresh[:room]])
        radii_all.append(r / s)
        centres_all.append(c / s)
    coords = _unpack21(have).contiguous()
    return coords, torch.cat(radii_all), torch.cat(centres_all)


def build_grid(
    ash,
    num_blocks: int = 200_000,
    embedding_dim: int = 16,
    grid_dim: int = 8,
    sparse_grid_dim: int = 128,
    device="cuda",
    seed: int = 3,
    embedding_std: float = 0.01,
):
    """Configuration 3/4 grid: BoundedSparseDenseGrid over the unit cube with
    exactly `num_blocks` active blocks and N(0, std) embeddings; the per-block
    neighbour table is built.  Returns (grid, radii, centres)."""
    coords, radii, centres = surface_blocks(
        num_blocks, sparse_grid_dim=sparse_grid_dim, device=device, seed=seed
    )
    grid = ash.BoundedSparseDenseGrid(
        3,
        num_blocks,
        embedding_dim,
        grid_dim=grid_dim,
        sparse_grid_dim=sparse_grid_dim,
        bbox_min=torch.zeros(3),
        bbox_max=torch.ones(3),
        device=device,
    )
    grid.engine.insert_keys(coords)
    g = _gen(device, seed + 1000)
    with torch.no_grad():
        grid.embeddings.copy_(
            torch.randn(grid.embeddings.shape, generator=g, device=device) * embedding_std
        )
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    return grid, radii, centres


def sphere_distance_field(grid, radii, centres) -> torch.Tensor:
    """Signed distance to the union of the scene's spheres at every cell of the
    grid's active blocks, (num_embeddings, cells_per_grid) in world units; zero
    in rows of inactive blocks.  The field the surface extraction of the demos
    runs on after fusion."""
    dev = grid.embeddings.device
    keys, idx = grid.engine.items()
    field = torch.zeros(grid.embeddings.shape[:2], device=dev)
    cell_coords = grid.cell_coords.view(1, -1, 3)
    centres, radii = centres.to(dev), radii.to(dev)
    for s in range(0, len(idx), 16384):
        cells = (keys[s : s + 16384].view(-1, 1, 3) * grid.grid_dim + cell_coords).float()
        world = grid.transform_cell_to_world(cells)
        best = None
        for c in range(0, len(centres), 8):
            d = (world.unsqueeze(2) - centres[c : c + 8].view(1, 1, -1, 3)).norm(dim=-1)
            d = (d - radii[c : c + 8]).min(dim=2)[0]
            best = d if best is None else torch.minimum(best, d)
        field[idx[s : s + 16384]] = best
    return field


def uniform_queries(
    grid, num_inside: int = 4_000_000, empty_fraction: float = 0.1, seed: int = 4
) -> torch.Tensor:
    """Configuration 3 queries (world coordinates): `num_inside` points uniform
    inside randomly chosen active blocks plus 10 % points whose block is
    inactive (they must come back masked), shuffled together."""
    device = grid.device
    g = _gen(device, seed)
    active, _ = grid.engine.items()
    pick = torch.randint(len(active), (num_inside,), generator=g, device=device)
    inside = (active[pick].float() + torch.rand(num_inside, 3, generator=g, device=device)) * grid.grid_dim
    n_empty = int(num_inside * empty_fraction)
    empties = []
    need = n_empty
    while need > 0:
        cand = torch.rand(2 * need + 64, 3, generator=g, device=device) * (
            grid.sparse_grid_dim * grid.grid_dim - 1
        )
        blocks = torch.floor(cand / grid.grid_dim).int()
        _, found = grid.engine.find(blocks)
        cand = cand[~found][:need]
        empties.append(cand)
        need -= len(cand)
    cells = torch.cat([inside] + empties)
    cells = cells[torch.randperm(len(cells), generator=g, device=device)]
    return grid.transform_cell_to_world(cells).contiguous()


def ray_queries(
    grid,
    radii: torch.Tensor,
    centres: torch.Tensor,
    num_rays: int = 32768,
    samples_per_ray: int = 128,
    band_cells: float = 12.0,
    seed: int = 5,
) -> torch.Tensor:
    """Configuration 4 queries (world coordinates), ray-major: every ray aims
    at a random point of a sphere surface from a random outside direction and
    carries `samples_per_ray` stratified samples in the band of +-band_cells
    cells around the hit, i.e. through the activated shell."""
    device = grid.device
    g = _gen(device, seed)
    target = _surface_points(radii.to(device), centres.to(device), num_rays, g)
    d = torch.randn(num_rays, 3, generator=g, device=device)
    d = d / d.norm(dim=1, keepdim=True).clamp_min(1e-12)
    band = band_cells * grid.cell_size
    jitter = torch.rand(num_rays, samples_per_ray, generator=g, device=device)
    t = (torch.arange(samples_per_ray, device=device).view(1, -1) + jitter) / samples_per_ray
    t = (t * 2 - 1) * band
    x = target.view(-1, 1, 3) + t.unsqueeze(-1) * d.view(-1, 1, 3)
    return x.view(-1, 3).contiguous()


def camera_rays(grid, radii, centres, num_rays: int = 32768, seed: int = 5):
    """Rays for the sampler (world coordinates): origins inside the grid's box,
    each aimed at a random point of a sphere surface.  Returns (origins,
    unit directions)."""
    device = grid.device
    g = _gen(device, seed)
    target = _surface_points(radii.to(device), centres.to(device), num_rays, g)
    lo, hi = grid.get_bbox()
    origin = lo + (hi - lo) * (0.05 + 0.9 * torch.rand(num_rays, 3, generator=g, device=device))
    d = target - origin
    d = d / d.norm(dim=1, keepdim=True).clamp_min(1e-12)
    return origin.contiguous(), d.contiguous()


# --------------------------------------------------------------------- cfg 5
class FusionScene:
    """Configuration 5: synthetic RGB-D stream.  48 random spheres, a pinhole
    camera (fx = fy = 525, cx = 319.5, cy = 239.5 at 640x480; scaled with the
    resolution) on a seeded orbit of radius 3 m looking at the origin, depth
    images (fp32 metres) by analytic ray casting.  Everything is computed on
    the CPU in float32 so that every backend is fed identical inputs."""

    def __init__(self, num_spheres: int = 48, width: int = 640, height: int = 480, seed: int = 6):
        g = _gen("cpu", seed)
        self.width, self.height = width, height
        sx, sy = width / 640.0, height / 480.0
        self.intrinsic = torch.tensor(
            [[525.0 * sx, 0.0, 319.5 * sx], [0.0, 525.0 * sy, 239.5 * sy], [0.0, 0.0, 1.0]]
        )
        self.radii = torch.rand(num_spheres, generator=g) * 0.35 + 0.1
        self.centres = (torch.rand(num_spheres, 3, generator=g) * 2 - 1) * 1.2
        self.phase = float(torch.rand(1, generator=g)) * 2 * math.pi
        self.depth_max = 6.0

    def pose(self, frame: int, num_frames: int = 100) -> torch.Tensor:
        """world-to-camera 4x4 (camera looks along +z at the origin)."""
        a = self.phase + 2 * math.pi * frame / num_frames
        eye = torch.tensor([3.0 * math.cos(a), 0.6 * math.sin(2 * a), 3.0 * math.sin(a)])
        fwd = -eye / eye.norm()
        right = torch.linalg.cross(torch.tensor([0.0, 1.0, 0.0]), fwd)
        right = right / right.norm()
        up = torch.linalg.cross(fwd, right)
        rot = torch.stack([right, up, fwd])  # rows: camera axes in world coordinates
        ext = torch.eye(4)
        ext[:3, :3] = rot
        ext[:3, 3] = -rot @ eye
        return ext

    def depth(self, extrinsic: torch.Tensor) -> torch.Tensor:
        """(H, W) depth along the camera z axis, 0 where no sphere is hit."""
        v, u = torch.meshgrid(
            torch.arange(self.height, dtype=torch.float32),
            torch.arange(self.width, dtype=torch.float32),
            indexing="ij",
        )
        k = self.intrinsic
        d_cam = torch.stack([(u - k[0, 2]) / k[0, 0], (v - k[1, 2]) / k[1, 1], torch.ones_like(u)], -1)
        rot, t = extrinsic[:3, :3], extrinsic[:3, 3]
        origin = -rot.t() @ t
        d = d_cam.view(-1, 3) @ rot  # camera ray directions in world coordinates
        oc = origin.view(1, 1, 3) - self.centres.view(1, -1, 3)
        b = (d.view(-1, 1, 3) * oc).sum(-1)
        a = (d * d).sum(-1, keepdim=True)
        c = (oc * oc).sum(-1) - self.radii.view(1, -1) ** 2
        disc = b * b - a * c
        s = (-b - disc.clamp_min(0).sqrt()) / a
        s = torch.where((disc > 0) & (s > 0), s, torch.full_like(s, float("inf")))
        z = s.min(dim=1)[0]  # parameter along d_cam == depth, since d_cam.z == 1
        z = torch.where(torch.isfinite(z) & (z < self.depth_max), z, torch.zeros_like(z))
        return z.view(self.height, self.width)

    def unproject(self, depth: torch.Tensor, extrinsic: torch.Tensor) -> torch.Tensor:
        """World-space points of the valid depth pixels (N, 3)."""
        v, u = torch.nonzero(depth > 0, as_tuple=True)
        z = depth[v, u]
        k = self.intrinsic
        cam = torch.stack([(u.float() - k[0, 2]) / k[0, 0] * z, (v.float() - k[1, 2]) / k[1, 1] * z, z], -1)
        rot, t = extrinsic[:3, :3], extrinsic[:3, 3]
        return ((cam - t) @ rot).contiguous()


def fuse_frame(grid, points, depth, intrinsic, extrinsic, trunc: float, depth_max: float = 6.0,
               fused: bool = False, count_blocks: bool = True):
    """One fusion step on `grid` (embedding channels: tsdf, weight), following
    the reference demo (demo/rgbd_fusion.py:200-254 and :76-110): activate the
    blocks around `points` with a one-block two-sided dilation, project every
    cell of the touched blocks into the depth image, and update the running
    weighted mean.  All tensors must live on the grid's device.  Returns the
    number of touched blocks.  `fused` takes the library's integration kernel
    instead of the torch expressions below (the reference's statement), and
    with `count_blocks=False` runs the frame without a read-back (returns
    None)."""
    if fused:
        import ash.fusion

        return ash.fusion.fuse_frame(grid, points, depth, intrinsic, extrinsic, trunc, depth_max,
                                     count_blocks=count_blocks)
    import ash.grid

    switch, ash.grid.FUSED_ACTIVATION = ash.grid.FUSED_ACTIVATION, False
    try:
        gc, cc, gi, ci = grid.spatial_init_(points, dilation=1, bidirectional=True)
    finally:
        ash.grid.FUSED_ACTIVATION = switch
    if gi.numel() == 0:
        return 0
    positions = grid.cell_to_world(gc, cc)
    xyz = positions @ extrinsic[:3, :3].t() + extrinsic[:3, 3]
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
    sdf = sdf.clamp(max=trunc)
    weight = ok.float().view(gi.shape[0], ci.shape[1], 1)
    sdf = sdf.view(gi.shape[0], ci.shape[1], 1)
    with torch.no_grad():
        cur = grid.embeddings[gi, ci]
        w_sum, mean = cur[..., 1:2], cur[..., 0:1]
        w_new = w_sum + weight
        cur[..., 0:1] = (mean * w_sum + sdf * weight) / (w_new + 1e-6)
        cur[..., 1:2] = w_new
        grid.embeddings[gi, ci] = cur
    return int(gi.shape[0])

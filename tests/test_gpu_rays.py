"""GPU parity tests of the ray functions (ash_ray_find_near_far,
ash_ray_sample) against the oracle on identical seeded inputs: every output is
bit-exact (the marches are sequences of fp32 operations with one fused
multiply-add per position, written the same way on both sides)."""
import math

import pytest
import torch

import workloads

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _scene(gpu_ash, oracle, n_blocks=6000, seed=700):
    blocks, _, _ = workloads.surface_blocks(n_blocks, 12, 64, device="cpu", seed=seed)
    blocks = blocks.int()
    cap = len(blocks) + 64
    engine = gpu_ash.ASHEngine(3, cap, DEV)
    engine.insert_keys(blocks.to(DEV))
    omap = oracle.HashMap(3, cap, torch.arange(cap, dtype=torch.int32))
    omap.insert_keys(blocks)
    return engine, omap, blocks, torch.Generator().manual_seed(seed)


def _rays(g, n, extent, blocks=None):
    """Random origins in the box; directions random, or (three quarters of
    them) towards a random active block so that most rays meet the surface."""
    o = torch.rand(n, 3, generator=g) * extent
    d = torch.randn(n, 3, generator=g)
    if blocks is not None and n:
        target = (blocks[torch.randint(len(blocks), (n,), generator=g)].float() + 0.5) * 8.0
        aimed = torch.rand(n, generator=g) < 0.75
        d = torch.where(aimed.unsqueeze(1), target - o, d)
    d = d / d.norm(dim=1, keepdim=True).clamp_min(1e-6)
    return o.contiguous(), d.contiguous()


@pytest.mark.parametrize("n", [0, 1, 5000])
def test_near_far_and_samples_match_oracle(gpu_ash, oracle, n):
    engine, omap, blocks, g = _scene(gpu_ash, oracle)
    backend = gpu_ash.grid.backend
    extent = 64 * 8.0
    o, d = _rays(g, n, extent, blocks)
    lo, hi = torch.zeros(3), torch.full((3,), extent)
    near, far = backend.ray_find_near_far(engine.backend, o.to(DEV), d.to(DEV), lo.to(DEV),
                                          hi.to(DEV), 0.5, 700.0, 1.0, 8.0)
    near_ref, far_ref = oracle.ray_find_near_far(omap, o, d, lo, hi, 0.5, 700.0, 1.0, 8.0)
    assert torch.equal(near.cpu(), near_ref) and torch.equal(far.cpu(), far_ref)
    if n > 1:
        assert int((near_ref >= 0).sum()) > n // 4  # the case is not trivial
    for max_samples in (8, 64, 4096):
        got = backend.ray_sample(engine.backend, o.to(DEV), d.to(DEV), near, far, lo.to(DEV),
                                 hi.to(DEV), max_samples, 8.0)
        ref = oracle.ray_sample(omap, o, d, near_ref, far_ref, lo, hi, max_samples, 8.0)
        for a, b in zip(got, ref):
            assert a.dtype == b.dtype and torch.equal(a.cpu(), b)
        if n > 1 and max_samples == 4096:
            assert ref[0].numel() > 10 * n


def test_many_rays_match_oracle(gpu_ash, oracle):
    """Enough rays for the sampler's one-lane-per-ray kernel (the cases above
    run the variant for few rays)."""
    engine, omap, blocks, g = _scene(gpu_ash, oracle, seed=705)
    backend = gpu_ash.grid.backend
    extent = 64 * 8.0
    n = 70_000
    o, d = _rays(g, n, extent, blocks)
    lo, hi = torch.zeros(3), torch.full((3,), extent)
    near, far = backend.ray_find_near_far(engine.backend, o.to(DEV), d.to(DEV), lo.to(DEV),
                                          hi.to(DEV), 0.5, 700.0, 1.0, 8.0)
    near_ref, far_ref = oracle.ray_find_near_far(omap, o, d, lo, hi, 0.5, 700.0, 1.0, 8.0)
    assert torch.equal(near.cpu(), near_ref) and torch.equal(far.cpu(), far_ref)
    got = backend.ray_sample(engine.backend, o.to(DEV), d.to(DEV), near, far, lo.to(DEV),
                             hi.to(DEV), 48, 8.0)
    ref = oracle.ray_sample(omap, o, d, near_ref, far_ref, lo, hi, 48, 8.0)
    assert ref[0].numel() > 10 * n
    for a, b in zip(got, ref):
        assert a.dtype == b.dtype and torch.equal(a.cpu(), b)


@pytest.mark.parametrize("mode", ["two_marches", "stage_overflow"])
def test_sample_paths_agree(gpu_ash, oracle, monkeypatch, mode):
    """ray_sample keeps the samples of its allocation pass and copies them; the
    reference's second march remains for staging areas that would be too large
    and for rays with more samples than the staging stride."""
    engine, omap, blocks, g = _scene(gpu_ash, oracle)
    backend = gpu_ash.grid.backend
    extent = 64 * 8.0
    o, d = _rays(g, 3000, extent, blocks)
    lo, hi = torch.zeros(3, device=DEV), torch.full((3,), extent, device=DEV)
    near, far = backend.ray_find_near_far(engine.backend, o.to(DEV), d.to(DEV), lo, hi,
                                          0.5, 700.0, 1.0, 8.0)
    staged = backend.ray_sample(engine.backend, o.to(DEV), d.to(DEV), near, far, lo, hi, 64, 8.0)
    if mode == "two_marches":
        monkeypatch.setattr(gpu_ash.common, "RAY_STAGE_LIMIT", 0)
    else:
        monkeypatch.setattr(gpu_ash.common, "RAY_STAGE_EXTRA", -60)   # stride 4
    other = backend.ray_sample(engine.backend, o.to(DEV), d.to(DEV), near, far, lo, hi, 64, 8.0)
    assert staged[0].numel() > 20_000 and int(torch.diff(staged[3]).max()) > 4
    for a, b in zip(staged, other):
        assert torch.equal(a, b)


def test_samples_start_inside_active_blocks(gpu_ash, oracle):
    """Property at a larger size: every interval starts in an active block,
    intervals of a ray are ordered, counts agree with the prefix sum."""
    engine, omap, blocks, g = _scene(gpu_ash, oracle, n_blocks=20000, seed=710)
    backend = gpu_ash.grid.backend
    extent = 64 * 8.0
    o, d = _rays(g, 200_000, extent, blocks)
    o, d = o.to(DEV), d.to(DEV)
    lo, hi = torch.zeros(3, device=DEV), torch.full((3,), extent, device=DEV)
    near, far = backend.ray_find_near_far(engine.backend, o, d, lo, hi, 0.0, 900.0, 1.0, 8.0)
    idx, tn, tf, prefix = backend.ray_sample(engine.backend, o, d, near, far, lo, hi, 128, 8.0)
    assert prefix.shape == (200_000,) and int(prefix[-1]) == idx.numel() > 10**6
    counts = torch.diff(prefix, prepend=prefix.new_zeros(1))
    assert torch.equal(torch.repeat_interleave(torch.arange(200_000, device=DEV), counts), idx)
    assert bool((tf > tn).all())
    same_ray = idx[1:] == idx[:-1]
    assert bool((tn[1:][same_ray] == tf[:-1][same_ray]).all())
    # Position where the sample was accepted: origin + t_accept * direction with
    # t_accept = t_far - step; recomputed in float64 and skipped within 1e-3
    # cells of a block face, it must lie in an active block.
    step = torch.clamp((far - near) / 128, min=0.7)[idx]
    pos = o[idx].double() + (tf - step).double().unsqueeze(1) * d[idx].double()
    frac = pos / 8.0 - torch.floor(pos / 8.0)
    clear = ((frac > 1e-3) & (frac < 1 - 1e-3)).all(dim=1)
    _, found = engine.find(torch.floor(pos[clear] / 8.0).int())
    assert bool(found.all())


def test_grid_methods_follow_the_reference_wrappers(gpu_ash):
    """SparseDenseGrid.ray_find_near_far / ray_sample (ash/grid.py:322-403):
    world units in, world units out, samples inside the surface shell."""
    grid, radii, centres = workloads.build_grid(gpu_ash, 3000, 4, 8, 64, device=DEV)
    g = torch.Generator().manual_seed(720)
    o = torch.rand(4000, 3, generator=g).to(DEV) * 0.2 + 0.4
    d = torch.randn(4000, 3, generator=g)
    d = (d / d.norm(dim=1, keepdim=True)).to(DEV)
    near, far = grid.ray_find_near_far(o, d, 0.0, 2.0, 0.01)
    hit = near >= 0
    assert int(hit.sum()) > 200 and bool((far[hit] > near[hit]).all())
    idx, tn, tf, prefix = grid.ray_sample(o, d, near, far, 64)
    assert int(prefix[-1]) == idx.numel() > 0
    x = o[idx] + ((tn + tf) / 2).unsqueeze(1) * d[idx]
    _, masks = grid(x, interpolation="linear")
    # midpoints of accepted intervals sit in active blocks, except for the
    # intervals that bridge a skipped gap
    assert float(masks.float().mean()) > 0.6
    assert math.isclose(float(tn.min()), float(near[hit].min()), rel_tol=0, abs_tol=grid.cell_size * 8)


def test_ranges_beyond_fp32_resolution_end(gpu_ash, oracle):
    """A sampling range so far out that a step no longer changes t must end
    (the reference would not return); near/far refuses such a range."""
    engine, omap, blocks, g = _scene(gpu_ash, oracle, n_blocks=500, seed=730)
    backend = gpu_ash.grid.backend
    o = torch.tensor([[10.0, 10.0, 10.0]] * 3)
    d = torch.tensor([[1.0, 0.0, 0.0]] * 3)
    lo, hi = torch.zeros(3), torch.full((3,), 512.0)
    nears = torch.tensor([1.0e9, 0.0, 3.0e7])
    fars = torch.tensor([2.0e9, 40.0, 3.0e7 + 64])
    got = backend.ray_sample(engine.backend, o.to(DEV), d.to(DEV), nears.to(DEV), fars.to(DEV),
                             lo.to(DEV), hi.to(DEV), 10**9, 8.0)
    ref = oracle.ray_sample(omap, o, d, nears, fars, lo, hi, 10**9, 8.0)
    for a, b in zip(got, ref):
        assert torch.equal(a.cpu(), b)
    with pytest.raises(RuntimeError, match="step is too small"):
        backend.ray_find_near_far(engine.backend, o.to(DEV), d.to(DEV), lo.to(DEV), hi.to(DEV),
                                  0.0, 1.0e12, 1.0, 8.0)

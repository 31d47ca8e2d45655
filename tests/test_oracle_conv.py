"""Pins of the oracle's sparse convolution (restating ash/src/grid.cu:948-1043
behind SparseDenseGrid.convolution, ash/grid.py:478-520): on a grid that is
densified into a volume it must equal torch.nn.functional.conv3d with zero
padding (missing blocks and the outside count as zero), per channel."""
import pytest
import torch
import torch.nn.functional as F


def _grid(cpu_ash, e, dtype, seed, n_blocks=40, g=4, s=4):
    gen = torch.Generator().manual_seed(seed)
    grid = cpu_ash.BoundedSparseDenseGrid(
        3, 64, e, grid_dim=g, sparse_grid_dim=s, bbox_min=torch.zeros(3), bbox_max=torch.ones(3),
        device="cpu")
    all_blocks = torch.stack(torch.meshgrid(*[torch.arange(s)] * 3, indexing="ij"), -1).view(-1, 3)
    pick = all_blocks[torch.randperm(len(all_blocks), generator=gen)[:n_blocks]].int()
    grid.engine.insert_keys(pick)
    with torch.no_grad():
        grid.embeddings.copy_(torch.randn(grid.embeddings.shape, generator=gen))
    inputs = grid.embeddings.detach().to(dtype).contiguous()
    return grid, inputs, gen


def _densify(grid, rows, g, s):
    """(B, M, E) rows of the active blocks -> volume (E, Z, Y, X); cell index is
    cx + G cy + G^2 cz, block coordinates are (bx, by, bz)."""
    keys, idx = grid.engine.items()
    e = rows.shape[-1]
    vol = torch.zeros(e, s * g, s * g, s * g, dtype=rows.dtype)
    for (bx, by, bz), i in zip(keys.tolist(), idx.tolist()):
        block = rows[i].view(g, g, g, e).permute(3, 0, 1, 2)  # (E, cz, cy, cx)
        vol[:, bz * g:(bz + 1) * g, by * g:(by + 1) * g, bx * g:(bx + 1) * g] = block
    return vol, keys, idx


@pytest.mark.parametrize("size", [3, 5])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.float64, 1e-12)])
def test_convolution_equals_dense_conv3d(cpu_ash, size, dtype, tol):
    g, s, e = 4, 4, 3
    grid, inputs, gen = _grid(cpu_ash, e, dtype, seed=40 + size)
    weights = torch.randn(size, size, size, e, generator=gen).to(dtype).contiguous()
    out = grid.convolution(inputs, weights)
    assert out.shape == inputs.shape and out.dtype == dtype
    vol, keys, idx = _densify(grid, inputs, g, s)
    # weights[z, y, x, c]: tap at offset (x, y, z) - R; conv3d is a correlation
    kernel = weights.permute(3, 0, 1, 2).unsqueeze(1)  # (E, 1, kz, ky, kx)
    dense = F.conv3d(vol.unsqueeze(0), kernel, padding=size // 2, groups=e)[0]
    got, _, _ = _densify(grid, out, g, s)
    active = torch.zeros(s * g, s * g, s * g, dtype=torch.bool)
    for bx, by, bz in keys.tolist():
        active[bz * g:(bz + 1) * g, by * g:(by + 1) * g, bx * g:(bx + 1) * g] = True
    assert torch.allclose(got[:, active], dense[:, active], rtol=tol, atol=tol)
    # rows of blocks that are not active stay zero
    free = torch.ones(out.shape[0], dtype=torch.bool)
    free[idx] = False
    assert bool((out[free] == 0).all())


def test_gaussian_filter_window(cpu_ash):
    """The window sums to one, so a constant field is unchanged wherever the
    whole window lies inside active blocks; the window is symmetric, so a
    linear ramp is unchanged there as well."""
    g, s = 4, 4
    grid, _, _ = _grid(cpu_ash, 2, torch.float32, seed=50, n_blocks=64)  # every block active
    keys, idx = grid.engine.items()
    with torch.no_grad():
        grid.embeddings[..., 0] = 3.5
        cells = grid.cell_coords.view(1, -1, 3).float()
        pos = keys.view(-1, 1, 3).float() * g + cells  # (n, M, 3)
        ramp = torch.zeros_like(grid.embeddings[..., 1])
        ramp[idx] = pos[..., 0] * 0.25 - pos[..., 1] * 0.5 + pos[..., 2]
        grid.embeddings[..., 1] = ramp
    before = grid.embeddings.detach().clone()
    grid.gaussian_filter_(5, 1.5)
    after = grid.embeddings.detach()
    interior = torch.zeros(before.shape[:2], dtype=torch.bool)
    interior[idx] = ((pos >= 2) & (pos <= s * g - 3)).all(-1)
    assert int(interior.sum()) == 12 ** 3
    assert torch.allclose(after[interior], before[interior], rtol=1e-5, atol=1e-5)
    # at the border mass leaks into the zero outside: values shrink
    assert bool((after[..., 0][~interior & (before[..., 0] > 0)] < 3.5).all())

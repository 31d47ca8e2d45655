"""Pins the trilinear half of the CPU oracle without the reference binary.

Each check is chosen so that a plausible slip (wrong corner bit order, a
transposed table, a dropped derivative factor, a sign) fails it:
  * closed form: embeddings := cell coordinates  =>  "linear" returns the query
    point (unittests/test_sparsedense_grid.py:139-181);
  * library routine: on a fully populated neighbourhood "linear" equals
    torch.nn.functional.grid_sample(mode="bilinear", align_corners=True);
  * an independent vectorised torch formula differentiated by autograd in
    float64 gives the first-order gradients and the two second-order products
    the reference returns (ash/src/grid.cu:177-255, 309-387);
  * special cases: masked-out and missing-neighbour queries give zero rows.
"""
import pytest
import torch
import torch.nn.functional as F

from helpers import torch_query, torch_term_sums


def _dense_grid(ash, grid_dim, embedding_dim, bound, dtype=torch.float32, seed=0):
    """Blocks -bound..bound in every axis, all active, random embeddings."""
    g = torch.Generator().manual_seed(seed)
    n_side = 2 * bound + 1
    grid = ash.SparseDenseGrid(3, n_side**3 + 3, embedding_dim, grid_dim, device="cpu")
    r = torch.arange(-bound, bound + 1, dtype=torch.int32)
    blocks = torch.stack(torch.meshgrid(r, r, r, indexing="ij"), dim=-1).view(-1, 3)
    grid.spatial_init_(blocks * grid_dim, dilation=0)
    with torch.no_grad():
        grid.embeddings.copy_(torch.rand(grid.embeddings.shape, generator=g) * 2 - 1)
    if dtype != torch.float32:
        grid.embeddings.data = grid.embeddings.data.to(dtype)
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    return grid


def _operands(grid, x):
    gi, ci, off, masks = grid.query(x)
    return (
        grid.embeddings.detach(), off, gi, ci, masks,
        grid.lut_grid_nb2grid_idx, grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb,
    )


def _queries(grid_dim, bound, n, seed):
    g = torch.Generator().manual_seed(seed)
    lo, hi = -grid_dim * bound, grid_dim * (bound + 1) - 1
    return torch.rand(n, 3, generator=g) * (hi - lo) + lo


@pytest.mark.parametrize("grid_dim", [1, 2, 4, 8])
def test_linear_reproduces_coordinates(cpu_ash, oracle, grid_dim):
    bound = 2
    grid = _dense_grid(cpu_ash, grid_dim, 3, bound)
    gc, cc, gi, ci = grid.items()
    coords = (gc * grid_dim + cc).float()
    with torch.no_grad():
        grid.embeddings[gi, ci] = coords
    x = _queries(grid_dim, bound, 2000, seed=1)
    y = oracle.query_forward(*_operands(grid, x), grid_dim, "linear")
    assert torch.allclose(y, x, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("grid_dim,embedding_dim", [(2, 1), (4, 5), (8, 16)])
def test_linear_equals_grid_sample(cpu_ash, oracle, grid_dim, embedding_dim):
    bound = 1
    grid = _dense_grid(cpu_ash, grid_dim, embedding_dim, bound, seed=3)
    side = (2 * bound + 1) * grid_dim
    # densify: volume[c, z, y, x] = embedding of integer cell (x, y, z)
    gc, cc, gi, ci = grid.items()
    cells = (gc * grid_dim + cc).view(-1, 3).long() + bound * grid_dim
    rows = grid.embeddings.detach()[gi.expand(-1, cc.shape[1]).reshape(-1), ci.expand(gc.shape[0], -1).reshape(-1)]
    volume = torch.zeros(embedding_dim, side, side, side)
    volume[:, cells[:, 2], cells[:, 1], cells[:, 0]] = rows.T
    x = _queries(grid_dim, bound, 3000, seed=4)
    y = oracle.query_forward(*_operands(grid, x), grid_dim, "linear")
    # align_corners=True maps -1 -> index 0 and +1 -> index side-1
    norm = (x + bound * grid_dim) / (side - 1) * 2 - 1
    ref = F.grid_sample(
        volume[None], norm.view(1, -1, 1, 1, 3), mode="bilinear", align_corners=True
    ).view(embedding_dim, -1).T
    assert torch.allclose(y, ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_forward_matches_independent_formula(cpu_ash, oracle, interpolation, dtype):
    grid = _dense_grid(cpu_ash, 4, 7, 1, dtype=dtype, seed=5)
    x = _queries(4, 1, 4000, seed=6)
    ops = _operands(grid, x)
    y = oracle.query_forward(*ops, 4, interpolation)
    ref = torch_query(*ops, interpolation)
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-12, atol=1e-13)
    assert torch.allclose(y, ref, **tol)


def test_constant_field_is_reproduced(cpu_ash, oracle):
    """Partition of unity: the weights of both bases sum to one."""
    grid = _dense_grid(cpu_ash, 4, 2, 1, seed=7)
    with torch.no_grad():
        grid.embeddings.fill_(1.25)
    x = _queries(4, 1, 1000, seed=8)
    for interpolation in ("linear", "smooth_step"):
        y = oracle.query_forward(*_operands(grid, x), 4, interpolation)
        assert torch.allclose(y, torch.full_like(y, 1.25), rtol=1e-6, atol=0)


def test_masked_and_incomplete_queries_are_zero(cpu_ash, oracle):
    """ash/src/grid.cu:84-86,109-111 and ash/grid.py:236: a query outside the
    active blocks is masked out; a query in an active block whose +1 neighbour
    block is missing keeps its mask but yields zeros."""
    grid_dim = 4
    grid = cpu_ash.SparseDenseGrid(3, 8, 3, grid_dim, device="cpu")
    grid.spatial_init_(torch.zeros(1, 3), dilation=0)  # single block (0,0,0)
    with torch.no_grad():
        grid.embeddings.fill_(1.0)
    grid.construct_grid_neighbor_lut_(1, False)
    x = torch.tensor([[1.5, 1.5, 1.5], [3.5, 1.0, 1.0], [9.0, 1.0, 1.0]])
    ops = _operands(grid, x)
    assert ops[4].tolist() == [True, True, False]
    for interpolation in ("linear", "smooth_step"):
        y = oracle.query_forward(*ops, grid_dim, interpolation)
        assert torch.allclose(y[0], torch.ones(3))
        assert torch.equal(y[1:], torch.zeros(2, 3))
        ge, go = oracle.query_backward_forward(torch.ones(3, 3), *ops, grid_dim, interpolation)
        assert torch.equal(go[1:], torch.zeros(2, 3))
        gz, ge2, _ = oracle.query_backward_backward(
            None, torch.ones(3, 3), torch.ones(3, 3), *ops, grid_dim, interpolation
        )
        assert torch.equal(gz[1:], torch.zeros(2, 3))


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
@pytest.mark.parametrize("grid_dim,embedding_dim", [(1, 2), (2, 1), (4, 4), (8, 8), (4, 16)])
def test_gradients_match_autograd(cpu_ash, oracle, interpolation, grid_dim, embedding_dim):
    """First order: (grad_embeddings, grad_offsets) = vjp of y with cotangent z.
    Second order: with u the cotangent of grad_offsets, the reference returns
    d(grad_offsets . u)/dz and d(grad_offsets . u)/dembeddings and nothing
    else (ash/src/grid.cu:417-426)."""
    grid = _dense_grid(cpu_ash, grid_dim, embedding_dim, 1, dtype=torch.float64, seed=9)
    x = _queries(grid_dim, 1, 1500, seed=10)
    ops = _operands(grid, x)
    n = x.shape[0]
    g = torch.Generator().manual_seed(11)
    z = torch.rand(n, embedding_dim, generator=g, dtype=torch.float64) - 0.5
    u = torch.rand(n, 3, generator=g, dtype=torch.float64) - 0.5

    emb = ops[0].clone().requires_grad_(True)
    # offsets are fp32 operands; differentiate through a float64 copy
    off64 = ops[1].double().requires_grad_(True)
    zz = z.clone().requires_grad_(True)

    def formula(e, o):
        dtype_ops = (e, o) + ops[2:]
        # torch_query evaluates "1 - o" in the offsets' own dtype
        return torch_query(*dtype_ops, interpolation)

    y = formula(emb, off64)
    ge_ref, go_ref = torch.autograd.grad(y, (emb, off64), zz, create_graph=True)
    gz_ref, ge2_ref = torch.autograd.grad((go_ref * u).sum(), (zz, emb))

    ge, go = oracle.query_backward_forward(z, *ops, grid_dim, interpolation)
    assert torch.allclose(ge, ge_ref.detach(), rtol=1e-9, atol=1e-10)
    assert torch.allclose(go, go_ref.detach(), rtol=1e-6, atol=1e-7)

    gz, ge2, goff2 = oracle.query_backward_backward(
        torch.zeros_like(ops[0]), u, z, *ops, grid_dim, interpolation
    )
    assert torch.allclose(gz, gz_ref, rtol=1e-6, atol=1e-7)
    assert torch.allclose(ge2, ge2_ref, rtol=1e-6, atol=1e-7)
    assert torch.equal(goff2, torch.zeros(n, 3, dtype=torch.float64))


def test_finite_differences_of_forward(cpu_ash, oracle):
    """Central differences of the oracle's own forward against its
    grad_offsets, float64, both bases."""
    grid = _dense_grid(cpu_ash, 4, 3, 1, dtype=torch.float64, seed=12)
    g = torch.Generator().manual_seed(13)
    cells = torch.randint(-4, 7, (400, 3), generator=g).float()
    frac = torch.rand(400, 3, generator=g).clamp(0.05, 0.95)
    x = cells + frac
    z = torch.rand(400, 3, generator=g, dtype=torch.float64)
    eps = 1e-3
    for interpolation in ("linear", "smooth_step"):
        ops = list(_operands(grid, x))
        _, go = oracle.query_backward_forward(z, *ops, 4, interpolation)
        for d in range(3):
            plus, minus = list(ops), list(ops)
            shift = torch.zeros(3)
            shift[d] = eps
            plus[1] = ops[1] + shift
            minus[1] = ops[1] - shift
            yp = oracle.query_forward(*plus, 4, interpolation)
            ym = oracle.query_forward(*minus, 4, interpolation)
            fd = ((yp - ym) * z).sum(dim=1) / (plus[1][:, d] - minus[1][:, d]).double()
            assert torch.allclose(go[:, d], fd, rtol=1e-3, atol=1e-4)


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
def test_term_sums_equal_an_independent_formula(cpu_ash, oracle, interpolation):
    """The magnitudes that the GPU tests scale their rounding bound with
    (sum of |terms| per output element) against a vectorised torch statement,
    with masked-out queries and missing neighbour blocks in the batch."""
    grid = _dense_grid(cpu_ash, 4, 3, 1, seed=9)
    x = _queries(4, 1, 1500, seed=10) + 2.5          # some queries leave the populated blocks
    ops = _operands(grid, x)
    g = torch.Generator().manual_seed(11)
    z = torch.rand(1500, 3, generator=g) - 0.5
    u = torch.rand(1500, 3, generator=g) - 0.5
    got = oracle.query_term_sums(u, z, *ops, 4, interpolation)
    ref = torch_term_sums(*ops, interpolation, z, u)
    assert set(got) == set(ref)
    for name in ref:
        assert torch.allclose(got[name], ref[name], rtol=1e-12, atol=1e-14), name
        assert float(ref[name].sum()) > 1.0
    assert 0.2 < float(ops[4].float().mean()) < 0.99

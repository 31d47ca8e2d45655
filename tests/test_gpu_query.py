"""GPU parity tests of the trilinear query kernels against the CPU oracle on
identical seeded inputs.  fp32 tolerance (north-star): 1e-5 relative / 1e-6
absolute, fp64 1e-12 / 1e-13.  Outputs that belong to one query (forward rows,
grad_offsets, grad_z) are compared at exactly that.  The dense embedding
gradients are sums over many queries that the GPU accumulates with atomics in
an order of its own; for them the bound also admits the rounding of such a sum,
K_ROUND * eps * (sum of |terms| of the element), with the sums of |terms| taken
from the oracle (helpers.assert_close_sums states K_ROUND)."""
import pytest
import torch

import workloads
from helpers import K_ROUND, assert_close_sums, torch_query

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
RTOL32, ATOL32 = 1e-5, 1e-6


def _tol(dtype):
    return dict(rtol=RTOL32, atol=ATOL32) if dtype == torch.float32 else dict(rtol=1e-12, atol=1e-13)


def _make_grid(ash, grid_dim, embedding_dim, bound, dtype=torch.float32, seed=0, holes=0):
    """Blocks -bound..bound in each axis (minus `holes` random ones) with
    uniform(-1,1) embeddings and the neighbour table built."""
    g = torch.Generator().manual_seed(seed)
    side = 2 * bound + 1
    grid = ash.SparseDenseGrid(3, side**3 + 5, embedding_dim, grid_dim, device=DEV)
    r = torch.arange(-bound, bound + 1, dtype=torch.int32)
    blocks = torch.stack(torch.meshgrid(r, r, r, indexing="ij"), dim=-1).view(-1, 3)
    if holes:
        blocks = blocks[torch.randperm(len(blocks), generator=g)[holes:]]
    grid.engine.insert_keys(blocks.to(DEV))
    with torch.no_grad():
        grid.embeddings.copy_((torch.rand(grid.embeddings.shape, generator=g) * 2 - 1).to(DEV))
    if dtype != torch.float32:
        grid.embeddings.data = grid.embeddings.data.to(dtype)
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    return grid


def _queries(grid_dim, bound, n, seed, margin=0.0):
    g = torch.Generator().manual_seed(seed)
    lo, hi = -grid_dim * bound - margin, grid_dim * (bound + 1) + margin
    return (torch.rand(n, 3, generator=g) * (hi - lo) + lo).to(DEV)


def _operands(grid, x):
    gi, ci, off, masks = grid.query(x)
    return (
        grid.embeddings.detach(), off, gi, ci, masks,
        grid.lut_grid_nb2grid_idx, grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb,
    )


def _to_cpu(ops):
    return tuple(o.cpu() for o in ops)


def _eps(dtype):
    return 2.0**-24 if dtype == torch.float32 else 2.0**-53


def _compare_all(ash, oracle, grid, x, interpolation, seed=0):
    ops = _operands(grid, x)
    cops = _to_cpu(ops)
    dtype = ops[0].dtype
    n, e, g_dim = x.shape[0], ops[0].shape[2], grid.grid_dim
    backend = ash.grid_query.backend
    gen = torch.Generator().manual_seed(seed)
    z = (torch.rand(n, e, generator=gen, dtype=torch.float64) - 0.5).to(dtype)
    u = (torch.rand(n, 3, generator=gen, dtype=torch.float64) - 0.5).to(dtype)
    tol = _tol(dtype)
    sums = oracle.query_term_sums(u, z, *cops, g_dim, interpolation)
    dense = dict(eps=_eps(dtype), **tol)

    y = backend.query_forward(*ops, g_dim, interpolation)
    y_ref = oracle.query_forward(*cops, g_dim, interpolation)
    assert torch.allclose(y.cpu(), y_ref, **tol), (y.cpu() - y_ref).abs().max()

    ge, go = backend.query_backward_forward(z.to(DEV), *ops, g_dim, interpolation)
    ge_ref, go_ref = oracle.query_backward_forward(z, *cops, g_dim, interpolation)
    assert torch.allclose(go.cpu(), go_ref, **tol), (go.cpu() - go_ref).abs().max()
    assert_close_sums(ge, ge_ref, sums["bf_embeddings"], what="grad_embeddings", **dense)

    gz, ge2, goff2 = backend.query_backward_backward(
        torch.zeros_like(ops[0]), u.to(DEV), z.to(DEV), *ops, g_dim, interpolation
    )
    gz_ref, ge2_ref, _ = oracle.query_backward_backward(None, u, z, *cops, g_dim, interpolation)
    assert torch.allclose(gz.cpu(), gz_ref, **tol), (gz.cpu() - gz_ref).abs().max()
    assert_close_sums(ge2, ge2_ref, sums["bb_embeddings"], what="grad_embeddings (2nd order)",
                      **dense)
    assert float(goff2.abs().sum()) == 0.0
    return ops, z, u, (ge, ge2)


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
@pytest.mark.parametrize("embedding_dim", [1, 2, 3, 4, 5, 6, 7, 8, 12, 16])
def test_all_embedding_dims_fp32(gpu_ash, oracle, interpolation, embedding_dim):
    grid = _make_grid(gpu_ash, 4, embedding_dim, 1, seed=embedding_dim, holes=3)
    x = _queries(4, 1, 6000, seed=100 + embedding_dim, margin=2.0)
    _compare_all(gpu_ash, oracle, grid, x, interpolation, seed=embedding_dim)


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
@pytest.mark.parametrize("grid_dim", [1, 2, 8, 16])
def test_all_grid_dims_fp32(gpu_ash, oracle, interpolation, grid_dim):
    """grid_dim 16 has 4096 cells per block: the per-cell tables no longer fit
    the LDS staging and are read through the caches."""
    grid = _make_grid(gpu_ash, grid_dim, 4, 1, seed=grid_dim, holes=2)
    x = _queries(grid_dim, 1, 5000, seed=200 + grid_dim, margin=1.0)
    _compare_all(gpu_ash, oracle, grid, x, interpolation, seed=grid_dim)


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
@pytest.mark.parametrize("embedding_dim", [1, 4, 7, 16])
def test_fp64(gpu_ash, oracle, interpolation, embedding_dim):
    grid = _make_grid(gpu_ash, 4, embedding_dim, 1, dtype=torch.float64, seed=7, holes=3)
    x = _queries(4, 1, 4000, seed=300 + embedding_dim, margin=2.0)
    _compare_all(gpu_ash, oracle, grid, x, interpolation, seed=3)


def test_repeated_cells_merge_path(gpu_ash, oracle):
    """Ray-like input: long runs of consecutive queries in one cell, the case
    the per-wavefront pre-reduction of atomics is for."""
    grid = _make_grid(gpu_ash, 8, 4, 1, seed=11)
    g = torch.Generator().manual_seed(12)
    starts = torch.rand(300, 1, 3, generator=g) * 20 - 6
    steps = torch.arange(64).view(1, -1, 1) * torch.rand(300, 1, 3, generator=g) * 0.05
    x = (starts + steps).view(-1, 3).to(DEV)
    for interpolation in ("linear", "smooth_step"):
        _compare_all(gpu_ash, oracle, grid, x, interpolation, seed=13)


def test_ordered_and_unordered_stretches_in_one_batch(gpu_ash, oracle):
    """The four-channel backward kernels gather gradient lines in a per-wavefront
    table, send rows past it when it is full and leave it aside for a few tiles
    when most rows went past it.  The batch makes every workgroup walk through
    all of that (a workgroup takes every n-th tile of its eighth of the batch,
    so each eighth holds the whole pattern): rays (few lines per tile), one
    query repeated over several tiles (a single line, runs that span rows of
    lanes), scattered queries (more lines per tile than the table holds: rows
    spill, then the table rests), rays again (the table comes back)."""
    grid = _make_grid(gpu_ash, 8, 4, 1, seed=21)
    g = torch.Generator().manual_seed(22)
    parts = []
    for _ in range(8):
        starts = torch.rand(1600, 1, 3, generator=g) * 20 - 6
        steps = torch.arange(128).view(1, -1, 1) * torch.rand(1600, 1, 3, generator=g) * 0.04
        rays = (starts + steps).view(-1, 3)
        same = (torch.rand(1, 3, generator=g) * 6 + 1).repeat(12800, 1)
        scattered = torch.rand(102400, 3, generator=g) * 20 - 6
        parts += [rays[:102400], same, scattered, rays[102400:]]
    x = torch.cat(parts).to(DEV)
    _compare_all(gpu_ash, oracle, grid, x, "smooth_step", seed=23)


def test_empty_batch_and_bad_arguments(gpu_ash):
    grid = _make_grid(gpu_ash, 2, 3, 1, seed=5)
    backend = gpu_ash.grid_query.backend
    x = _queries(2, 1, 10, seed=1)
    ops = _operands(grid, x)
    empty = (ops[0], ops[1][:0], ops[2][:0], ops[3][:0], ops[4][:0]) + ops[5:]
    y = backend.query_forward(*empty, 2, "linear")
    assert y.shape == (0, 3)
    ge, go = backend.query_backward_forward(torch.zeros((0, 3), device=DEV), *empty, 2, "linear")
    assert ge.shape == ops[0].shape and float(ge.abs().sum()) == 0 and go.shape == (0, 3)
    with pytest.raises(RuntimeError, match="Unknown interpolation"):
        backend.query_forward(*ops, 2, "cubic")
    with pytest.raises(RuntimeError):
        backend.query_forward(ops[0].cpu(), *ops[1:], 2, "linear")


@pytest.mark.parametrize("grid_dim", [1, 4, 8])
def test_reference_forward_closed_form(gpu_ash, grid_dim):
    """unittests/test_sparsedense_grid.py:139-181: embeddings := coordinates."""
    bound = 3
    grid = gpu_ash.SparseDenseGrid(3, 1000, 3, grid_dim, device=DEV)
    r = torch.arange(-bound, bound + 1, dtype=torch.int, device=DEV)
    blocks = grid_dim * torch.stack(torch.meshgrid(r, r, r, indexing="ij"), dim=-1).view(-1, 3)
    grid.spatial_init_(blocks, dilation=0)
    gc, cc, gi, ci = grid.items()
    coords = (gc * grid_dim + cc).view(-1, 3).float()
    with torch.no_grad():
        grid.embeddings[gi, ci, :3] = coords.view(gi.shape[0], ci.shape[1], 3)
    q = (2 * grid_dim * bound - 1) * torch.rand(1000, 3, device=DEV) - grid_dim * bound
    emb, masks = grid(q, interpolation="linear")
    assert torch.allclose(emb[..., :3], q, rtol=1e-5, atol=1e-4)
    assert bool(masks.all())
    feats, masks = grid(coords, interpolation="nearest")
    gi2, ci2, off, _ = grid.query(coords)
    assert torch.allclose(off, torch.zeros_like(off))
    assert torch.equal(feats, grid.embeddings[gi2, ci2])
    feats.sum().backward()
    assert grid.embeddings.grad is not None


class _SineMLP(torch.nn.Module):
    """Small sine network standing in for the reference tests' SirenNet."""

    def __init__(self, d_in, d_hidden=32):
        super().__init__()
        self.a = torch.nn.Linear(d_in, d_hidden)
        self.b = torch.nn.Linear(d_hidden, 1)

    def forward(self, x):
        return self.b(torch.sin(3.0 * self.a(x)))


@pytest.mark.parametrize("embedding_dim,grid_dim", [(2, 1), (1, 2), (4, 4), (8, 8)])
def test_reference_gradcheck(gpu_ash, embedding_dim, grid_dim):
    """unittests/test_sparsedense_grid.py:183-281: gradcheck w.r.t. positions
    and w.r.t. embeddings through a small network, fp32, eps 1e-3, tol 1e-2."""
    torch.manual_seed(15213)
    grid = gpu_ash.SparseDenseGrid(3, 8, embedding_dim, grid_dim, device=DEV)
    r = torch.arange(0, 2, dtype=torch.int, device=DEV)
    blocks = grid_dim * torch.stack(torch.meshgrid(r, r, r, indexing="ij"), dim=-1).view(-1, 3)
    grid.spatial_init_(blocks, dilation=0)
    torch.nn.init.uniform_(grid.embeddings, -1, 1)
    eps = 1e-3
    cells = torch.randint(high=grid_dim * 2 - 1, size=(200, 3), device=DEV)
    frac = torch.rand(200, 3, device=DEV).clamp(2 * eps, 1 - 2 * eps)
    positions = (cells + frac).requires_grad_(True)
    net = _SineMLP(embedding_dim + 3).to(DEV)
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)

    def run(embeddings, x_in, interpolation):
        gi, ci, off, masks = grid.query(grid.transform_world_to_cell(x_in))
        assert bool(masks.all())
        feats = gpu_ash.SparseDenseGridQuery.apply(
            embeddings, off, gi, ci, masks, grid.lut_grid_nb2grid_idx,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, grid.grid_dim, interpolation,
        )
        return net(torch.cat((feats, x_in), dim=-1))

    torch.autograd.gradcheck(
        lambda x: run(grid.embeddings, x, "linear"), (positions,), eps=eps, atol=1e-2, rtol=1e-2,
        nondet_tol=1e-4,
    )
    torch.autograd.gradcheck(
        lambda e: run(e, positions, "smooth_step"), (grid.embeddings,), eps=eps, atol=1e-2,
        rtol=1e-2, nondet_tol=1e-4,
    )


def test_double_backward_gradcheck_fp64(gpu_ash):
    """unittests/test_sparsedense_grid.py:283-347 (defined upstream, never
    called): fp64 gradcheck of SparseDenseGridQueryBackward w.r.t. embeddings
    and w.r.t. z."""
    torch.manual_seed(1)
    grid_dim, e = 4, 3
    grid = gpu_ash.SparseDenseGrid(3, 8, e, grid_dim, device=DEV)
    r = torch.arange(0, 2, dtype=torch.int, device=DEV)
    blocks = grid_dim * torch.stack(torch.meshgrid(r, r, r, indexing="ij"), dim=-1).view(-1, 3)
    grid.spatial_init_(blocks, dilation=0)
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    cells = torch.randint(high=grid_dim * 2 - 1, size=(60, 3), device=DEV)
    positions = cells + torch.rand(60, 3, device=DEV).clamp(0.01, 0.99)
    gi, ci, off, masks = grid.query(positions)
    emb64 = (torch.rand(grid.embeddings.shape, device=DEV, dtype=torch.float64) * 2 - 1).requires_grad_(True)
    z = torch.rand(60, e, device=DEV, dtype=torch.float64).requires_grad_(True)

    def grad_offsets(embeddings, zz):
        return gpu_ash.SparseDenseGridQueryBackward.apply(
            zz, embeddings, off, gi, ci, masks, grid.lut_grid_nb2grid_idx,
            grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb, grid.grid_dim, "smooth_step",
        )[1]

    torch.autograd.gradcheck(grad_offsets, (emb64, z), eps=1e-6, atol=1e-6, rtol=1e-6, nondet_tol=1e-9)


@pytest.mark.parametrize("interpolation", ["linear", "smooth_step"])
def test_eikonal_training_step_matches_autograd(gpu_ash, interpolation):
    """The flow of configuration 4 end to end through the module: value loss +
    gradient-norm loss, second-order backward to the embeddings; compared with
    float64 autograd of the independent torch formula.  The offsets-Hessian
    term the reference leaves out (ash/src/grid.cu:417-418) is removed from the
    comparison by detaching the positions inside the formula's gradient."""
    grid = _make_grid(gpu_ash, 4, 4, 1, seed=21)
    x = _queries(4, 1, 3000, seed=22).requires_grad_(True)

    feats, masks = grid(x, interpolation)
    sdf = feats[:, 0]
    (grad_x,) = torch.autograd.grad(sdf.sum(), x, create_graph=True)
    loss = (feats[:, 1:] ** 2).mean() + ((grad_x.norm(dim=-1) - 1) ** 2).mean()
    loss.backward()
    got = grid.embeddings.grad.detach().cpu().double()

    gi, ci, off, masks2 = grid.query(x.detach())
    ops = [o.cpu() for o in (gi, ci, masks2, grid.lut_grid_nb2grid_idx,
                             grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb)]
    emb = grid.embeddings.detach().cpu().double().requires_grad_(True)
    off_leaf = off.detach().cpu().requires_grad_(True)
    y = torch_query(emb, off_leaf, *ops, interpolation)
    (gx,) = torch.autograd.grad(y[:, 0].sum(), off_leaf, create_graph=True)
    ref_loss = (y[:, 1:] ** 2).mean() + ((gx.norm(dim=-1) - 1) ** 2).mean()
    (ref,) = torch.autograd.grad(ref_loss, emb)
    assert abs(loss.item() - ref_loss.item()) < 1e-5 * max(1.0, abs(ref_loss.item()))
    assert torch.allclose(got, ref, rtol=1e-4, atol=1e-6), (got - ref).abs().max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_accumulating_gradient_calls(gpu_ash, oracle, dtype):
    """ash_query_backward_forward_accumulate / _backward_accumulate add to the
    tensor they are given what the plain calls return (checked against the
    oracle's gradient on top of a random start), write the other output as
    usual, and refuse a tensor that is not like the embeddings."""
    grid = _make_grid(gpu_ash, 4, 3, 1, dtype=dtype, seed=51, holes=2)
    x = _queries(4, 1, 5000, seed=52, margin=1.0)
    ops = _operands(grid, x)
    backend = gpu_ash.grid_query.backend
    g = torch.Generator().manual_seed(53)
    n = x.shape[0]
    z = (torch.rand(n, 3, generator=g, dtype=dtype) - 0.5).to(DEV)
    u = (torch.rand(n, 3, generator=g, dtype=dtype) - 0.5).to(DEV)
    start = (torch.rand(ops[0].shape, generator=g, dtype=dtype) - 0.5).to(DEV)
    tol = _tol(dtype)
    sums = oracle.query_term_sums(u, z, *_to_cpu(ops), 4, "smooth_step")
    dense = dict(eps=_eps(dtype), **tol)
    began = start.cpu().double().abs()        # the start value is one more term of every sum

    ref_emb, ref_off = oracle.query_backward_forward(z.cpu(), *_to_cpu(ops), 4, "smooth_step")
    acc = start.clone()
    got_emb, got_off = backend.query_backward_forward(z, *ops, 4, "smooth_step", accumulate_into=acc)
    assert got_emb is acc
    assert_close_sums(acc, start.cpu() + ref_emb, sums["bf_embeddings"] + began, **dense)
    assert torch.allclose(got_off.cpu(), ref_off, **tol)
    acc = start.clone()
    _, none_off = backend.query_backward_forward(z, *ops, 4, "smooth_step", need_offsets=False,
                                                 accumulate_into=acc)
    assert none_off is None
    assert_close_sums(acc, start.cpu() + ref_emb, sums["bf_embeddings"] + began, **dense)

    ref_z, ref_emb2, _ = oracle.query_backward_backward(None, u.cpu(), z.cpu(), *_to_cpu(ops), 4, "smooth_step")
    acc = start.clone()
    got_z, got_emb2, _ = backend.query_backward_backward(None, u, z, *ops, 4, "smooth_step",
                                                         accumulate_into=acc)
    assert got_emb2 is acc
    assert_close_sums(acc, start.cpu() + ref_emb2, sums["bb_embeddings"] + began, **dense)
    assert torch.allclose(got_z.cpu(), ref_z, **tol)

    with pytest.raises(RuntimeError, match="accumulate_into"):
        backend.query_backward_forward(z, *ops, 4, "smooth_step", accumulate_into=start[:-1])
    with pytest.raises(RuntimeError, match="accumulate_into"):
        backend.query_backward_backward(None, u, z, *ops, 4, "smooth_step",
                                        accumulate_into=start.to(torch.float16))


def test_training_step_with_one_dense_gradient(gpu_ash, oracle):
    """In a pass that reaches the embeddings through the first- and the
    second-order backward every node fills a dense gradient of its own, as in
    the reference (ash/grid_query.py:86-129,209-283); inside
    `with ash.dense_grad(grid):` both nodes add to `embeddings.grad`
    (ash_query_backward_*_accumulate) and hand autograd nothing.  Same .grad as
    two separate passes, also on a second pass into an existing .grad and with
    a hook that keeps the query node's gradients while a weight-decay term
    contributes as well (the step of demo/train_scene_recon.py:326-341 with a
    regulariser).  Both sides add up the same terms in another order, so they
    may differ by the rounding of those sums: K_ROUND * eps * sum|terms|, the
    terms being those of the recorded calls."""
    grid = _make_grid(gpu_ash, 4, 4, 2, seed=41, holes=5)
    x = _queries(4, 2, 20_000, seed=42)
    backend = gpu_ash.grid_query.backend
    in_place_calls, recorded = [], []
    reals = {name: getattr(backend, name)
             for name in ("query_backward_forward", "query_backward_backward")}

    def spy(name):
        def call(*args, **kwargs):
            if kwargs.get("accumulate_into") is not None:
                in_place_calls.append(name)
            if kwargs.get("need_embeddings", True):
                recorded.append((name, [a.detach().clone() if torch.is_tensor(a) else a for a in args]))
            return reals[name](*args, **kwargs)
        return call

    def term_sums(calls):
        total = torch.zeros(grid.embeddings.shape, dtype=torch.float64)
        for name, args in calls:
            if name == "query_backward_forward":
                z, ops = args[0], args[1:9]
                total += oracle.query_term_sums(torch.zeros(z.shape[0], 3), z, *ops, 4,
                                                "smooth_step")["bf_embeddings"]
            else:
                u, z, ops = args[1], args[2], args[3:11]
                total += oracle.query_term_sums(u, z, *ops, 4, "smooth_step")["bb_embeddings"]
        return total

    def losses(hook=None):
        xq = x.clone().requires_grad_(True)
        feats, _ = grid(xq, "smooth_step")
        if hook is not None:
            feats.grad_fn.register_hook(hook)
        (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
        return (feats[:, 1:] ** 2).mean(), (gx.norm(dim=-1) - 1).abs().mean()

    for name in reals:
        setattr(backend, name, spy(name))
    try:
        expected = torch.zeros_like(grid.embeddings)
        for which in (0, 1):
            grid.embeddings.grad = None
            losses()[which].backward()
            expected += grid.embeddings.grad
        assert in_place_calls == []
        sums = term_sums(recorded)
        assert float(sums.sum()) > 0
        order = dict(rtol=0.0, atol=0.0, eps=2.0**-24)
        # as shipped, outside a block: every node fills a dense gradient of its own
        grid.embeddings.grad = None
        value, eikonal = losses()
        (value + eikonal).backward()
        assert in_place_calls == [] and gpu_ash.grid_query.LAST_GRADIENT_PATH == "own"
        assert_close_sums(grid.embeddings.grad, expected, sums, what="plain", **order)
        # inside the block: two in-place calls, one .grad tensor
        grid.embeddings.grad = None
        with gpu_ash.dense_grad(grid):
            value, eikonal = losses()
            (value + eikonal).backward()
            assert len(in_place_calls) == 2
            assert gpu_ash.grid_query.LAST_GRADIENT_PATH == "contract"
            assert_close_sums(grid.embeddings.grad, expected, sums, what="one pass", **order)
            held = grid.embeddings.grad
            value, eikonal = losses()
            (value + eikonal).backward()
            assert len(in_place_calls) == 4 and grid.embeddings.grad is held
            assert_close_sums(grid.embeddings.grad, 2 * expected, 2 * sums, what="two passes",
                              **order)
        # a hook that keeps the node's gradients + a weight-decay term, inside
        # the block and outside: the same total
        decay = grid.embeddings.detach().cpu().double()
        for inside in (False, True):
            kept = []
            grid.embeddings.grad = None
            value, eikonal = losses(hook=lambda gin, gout: kept.append(gin))
            loss = value + eikonal + 0.5 * (grid.embeddings ** 2).sum()
            if inside:
                with gpu_ash.dense_grad(grid):
                    loss.backward()
            else:
                loss.backward()
            assert len(kept) >= 1
            assert len(in_place_calls) == (6 if inside else 4)
            assert_close_sums(grid.embeddings.grad, expected.cpu().double() + decay,
                              sums + decay.abs(), what=f"hook + decay, inside={inside}", **order)
    finally:
        for name in reals:
            delattr(backend, name)


def test_gradient_paths_on_this_torch(gpu_ash):
    """Which gradients a backward node computes is decided with one private
    call of the autograd engine (torch._C._will_engine_execute_node); where it
    is missing or means something else both gradients are produced (right, but
    `autograd.grad(y, x, create_graph=True)` then fills and accumulates a dense
    gradient of the whole parameter that nobody reads).  This pins the
    behaviour on the torch that is installed."""
    assert hasattr(torch._C, "_will_engine_execute_node"), torch.__version__
    grid = _make_grid(gpu_ash, 4, 4, 1, seed=43)
    xq = _queries(4, 1, 2000, seed=44).requires_grad_(True)
    feats, _ = grid(xq, "smooth_step")
    gpu_ash.grid_query.LAST_GRADIENT_PATH = None
    (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
    assert gpu_ash.grid_query.LAST_GRADIENT_PATH == "skipped", torch.__version__
    grid.embeddings.grad = None
    ((feats[:, 1:] ** 2).mean() + (gx.norm(dim=-1) - 1).abs().mean()).backward()
    assert gpu_ash.grid_query.LAST_GRADIENT_PATH == "own", torch.__version__
    assert grid.embeddings.grad is not None and xq.grad is not None


def _config_grid(gpu_ash, embedding_dim, num_blocks=3000, sparse=64):
    return workloads.build_grid(
        gpu_ash, num_blocks, embedding_dim, grid_dim=8, sparse_grid_dim=sparse, device=DEV
    )


def test_config3_reduced_against_oracle(gpu_ash, oracle):
    """Configuration 3 at reduced size: bounded grid, 8^3 cells, E = 16,
    queries uniform in active blocks plus 10 % in empty space."""
    grid, _, _ = _config_grid(gpu_ash, 16)
    x = workloads.uniform_queries(grid, 60000)
    cells = grid.transform_world_to_cell(x)
    for interpolation in ("linear", "smooth_step"):
        ops = _operands(grid, cells)
        masks = ops[4]
        assert 0.85 < float(masks.float().mean()) < 0.95
        y = gpu_ash.grid_query.backend.query_forward(*ops, 8, interpolation)
        y_ref = oracle.query_forward(*_to_cpu(ops), 8, interpolation)
        assert torch.allclose(y.cpu(), y_ref, rtol=RTOL32, atol=ATOL32)
        assert float(y[~masks].abs().sum()) == 0.0
        feats, m2 = grid(x, interpolation)
        assert torch.equal(m2, masks) and torch.equal(feats.detach(), y)


def test_config4_reduced_against_oracle(gpu_ash, oracle):
    """Configuration 4 at reduced size: E = 4, ray-ordered stratified samples,
    forward + backward + double backward."""
    grid, radii, centres = _config_grid(gpu_ash, 4)
    x = workloads.ray_queries(grid, radii, centres, num_rays=512, samples_per_ray=128)
    cells = grid.transform_world_to_cell(x)
    ops, _, _, _ = _compare_all(gpu_ash, oracle, grid, cells, "smooth_step", seed=31)
    assert float(ops[4].float().mean()) > 0.5


def test_config4_full_size_against_oracle(gpu_ash, oracle):
    """Configuration 4 at its full size (200 k blocks of 8^3 cells, E = 4,
    32 768 rays x 128 samples = 2^22 queries): forward, backward and double
    backward against the oracle, which pins the launch geometry of the full
    shape (32-bit row numbers, the walk of the tiles over the XCDs).  Plus a
    check that needs no oracle: the eight weights of a query add up to one, so
    the embedding gradient summed over all rows is the sum of z over the
    queries that have all eight corners."""
    grid, radii, centres = workloads.build_grid(gpu_ash, embedding_dim=4, device=DEV)
    x = workloads.ray_queries(grid, radii, centres)
    assert x.shape[0] == 1 << 22 and grid.embeddings.shape == (200_000, 512, 4)
    cells = grid.transform_world_to_cell(x)
    ops, z, u, (ge, ge2) = _compare_all(gpu_ash, oracle, grid, cells, "smooth_step", seed=41)
    assert 0.3 < float(ops[4].float().mean()) < 1.0
    ones = (torch.ones_like(ops[0]),) + tuple(ops[1:])
    complete = gpu_ash.grid_query.backend.query_forward(*ones, 8, "smooth_step")[:, 0] != 0
    assert bool((complete <= ops[4]).all()) and int(complete.sum()) > 1_000_000
    zc = z.to(DEV).double() * complete.unsqueeze(1)
    total, magnitude = zc.sum(dim=0), zc.abs().sum(dim=0)
    got = ge.double().sum(dim=(0, 1))
    # each query's weights add up to 1 within a few eps; K_ROUND eps sum|z| covers
    # that and the accumulation
    assert bool(((got - total).abs() <= K_ROUND * 2.0**-24 * magnitude).all()), (got, total)
    # the module's forward (one kernel from positions to features) at this size
    y = gpu_ash.grid_query.backend.query_forward(*ops, 8, "smooth_step")
    feats, masks = grid(x, "smooth_step")
    assert torch.equal(masks, ops[4]) and torch.equal(feats, y)


def test_config3_full_size_against_oracle(gpu_ash, oracle):
    """Configuration 3 at full size (200 k blocks of 8^3 cells, E = 16: 1.64 G
    embedding values, 4.4 M queries of which a tenth in empty space): forward
    with both interpolations against the oracle (ash/src/grid.cu:68-132) at the
    fp32 tolerance -- 1.64 G elements, byte offsets beyond 32 bits -- the module's fused forward bit for bit against
    the two calls, and properties that need no oracle: linearity in the
    embeddings, constants reproduced where all 8 corners exist, masked rows
    zero."""
    grid, _, _ = workloads.build_grid(gpu_ash, device=DEV)
    x = workloads.uniform_queries(grid)
    assert grid.embeddings.shape == (200_000, 512, 16) and x.shape[0] == 4_400_000
    ops = list(_operands(grid, grid.transform_world_to_cell(x)))
    assert int(ops[2].max()) * 512 * 16 * 4 > 2**32     # byte offsets beyond 32 bits are addressed
    backend = gpu_ash.grid_query.backend
    cops = _to_cpu(ops)
    masks = ops[4]
    assert 0.85 < float(masks.float().mean()) < 0.95
    for interpolation in ("linear", "smooth_step"):
        y = backend.query_forward(*ops, 8, interpolation)
        y_ref = oracle.query_forward(*cops, 8, interpolation)
        assert torch.allclose(y.cpu(), y_ref, rtol=RTOL32, atol=ATOL32), (
            interpolation, float((y.cpu() - y_ref).abs().max()))
        assert float(y[~masks].abs().sum()) == 0.0
        feats, m2 = grid(x, interpolation)
        assert torch.equal(m2, masks) and torch.equal(feats, y), interpolation
        del y_ref, feats
    del cops
    y1 = backend.query_forward(*ops, 8, "smooth_step")
    emb = ops[0]
    ops[0] = emb * 3.0
    y3 = backend.query_forward(*ops, 8, "smooth_step")
    assert torch.allclose(y3, 3.0 * y1, rtol=1e-5, atol=1e-7)
    ops[0] = torch.ones_like(emb)
    yc = backend.query_forward(*ops, 8, "smooth_step")
    row_sum = yc.sum(dim=1)
    complete = row_sum != 0
    assert bool((complete <= masks).all())
    assert float(complete.float().mean()) > 0.7
    assert torch.allclose(yc[complete], torch.ones_like(yc[complete]), rtol=1e-5, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("grid_dim,embedding_dim", [(1, 3), (2, 1), (3, 5), (8, 4), (8, 8), (8, 16), (16, 2)])
def test_fused_forward_equals_query_then_interpolation(gpu_ash, oracle, monkeypatch, dtype,
                                                       grid_dim, embedding_dim):
    """`SparseDenseGrid.forward` through ash_grid_forward (positions -> features
    in one kernel) against `query` followed by `query_forward`
    (ash/grid.py:201-238), bit for bit: features, masks and -- when a backward
    pass will want them -- block indices, cell indices and offsets; positions
    inside, outside and right on block boundaries, run-ordered and shuffled;
    against the oracle at the stated tolerance; and the gradients that flow
    through either formulation."""
    grid = _make_grid(gpu_ash, grid_dim, embedding_dim, 2, dtype=dtype,
                      seed=7 * grid_dim + embedding_dim, holes=9)
    g = torch.Generator().manual_seed(70 + grid_dim)
    span = grid_dim * 3.5
    rand = (torch.rand(30_011, 3, generator=g) * 2 - 1) * span
    # runs of positions inside one block, as samples along a ray come
    walk = (torch.rand(300, 1, 3, generator=g) * 2 - 1) * span * 0.6 + \
        torch.linspace(0, 1, 40).view(1, 40, 1) * (torch.rand(300, 1, 3, generator=g) - 0.5) * grid_dim
    ints = torch.randint(-3 * grid_dim, 3 * grid_dim + 1, (1000, 3), generator=g).float()
    edge = torch.tensor([[-1e-9, 0.0, 0.0], [-1e-9, -1e-9, -1e-9], [grid_dim - 1e-7, 0.5, 0.5],
                         [-0.0, 0.0, -1e-30], [1e-7 - grid_dim, 0.25, 0.75]])
    x = torch.cat([rand, walk.reshape(-1, 3), ints, edge]).to(DEV)
    backend = gpu_ash.grid_query.backend
    tables = (grid.lut_grid_nb2grid_idx, grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb)
    emb = grid.embeddings.detach()
    gi, ci, off, masks = grid.query(x)
    for interpolation in ("linear", "smooth_step"):
        y = backend.query_forward(emb, off, gi, ci, masks, *tables, grid_dim, interpolation)
        y_ref = oracle.query_forward(emb.cpu(), off.cpu(), gi.cpu(), ci.cpu(), masks.cpu(),
                                     *[t.cpu() for t in tables], grid_dim, interpolation)
        assert torch.allclose(y.cpu(), y_ref, **_tol(dtype))
        # inference: nothing but features and masks is produced
        f0, m0, none_gi, none_ci, none_off = backend.grid_forward(
            grid.engine.backend, x, emb, *tables, grid_dim, interpolation, need_operands=False)
        assert none_gi is None and none_ci is None and none_off is None
        assert torch.equal(f0, y) and torch.equal(m0, masks)
        # with the operands of the backward pass
        f1, m1, gi1, ci1, off1 = backend.grid_forward(
            grid.engine.backend, x, emb, *tables, grid_dim, interpolation)
        assert torch.equal(f1, y) and torch.equal(m1, masks)
        assert torch.equal(gi1, gi) and torch.equal(ci1, ci) and torch.equal(off1, off)
        assert gi1.dtype == torch.int64 and off1.dtype == torch.float32 and m1.dtype == torch.bool
        # through the module, with and without gradients, both formulations
        results = {}
        for fused in (True, False):
            monkeypatch.setattr(gpu_ash.grid, "FUSED_FORWARD", fused)
            with torch.no_grad():
                f2, m2 = grid(x, interpolation)
            assert torch.equal(f2, y) and torch.equal(m2, masks)
            xq = x.clone().requires_grad_(True)
            grid.embeddings.grad = None
            feats, m3 = grid(xq, interpolation)
            assert torch.equal(feats.detach(), y) and torch.equal(m3, masks)
            assert not m3.requires_grad
            weights = torch.linspace(0.5, 1.5, embedding_dim, device=DEV, dtype=dtype)
            (gx,) = torch.autograd.grad((feats * weights).sum(), xq, create_graph=True)
            ((feats ** 2).sum() + (gx ** 2).sum()).backward()
            results[fused] = (gx.detach(), xq.grad.clone(), grid.embeddings.grad.clone())
        assert torch.equal(results[True][0], results[False][0])
        assert torch.equal(results[True][1], results[False][1])
        # the dense gradients are the same sums, accumulated in an order of the
        # device's own on either side
        scale = results[False][2].abs().max()
        assert torch.allclose(results[True][2], results[False][2], rtol=1e-4 if dtype == torch.float32 else 1e-10,
                              atol=float(scale) * (1e-5 if dtype == torch.float32 else 1e-12))
    with pytest.raises(RuntimeError, match="grid_dim"):
        backend.grid_forward(grid.engine.backend, x, emb, *tables, grid_dim + 1, "linear")
    with pytest.raises(RuntimeError, match="Unknown interpolation"):
        backend.grid_forward(grid.engine.backend, x, emb, *tables, grid_dim, "cubic")


@pytest.mark.parametrize("kind", ["bounded", "unbounded", "user transform"])
def test_fused_forward_applies_the_world_to_cell_transform(gpu_ash, monkeypatch, kind):
    """World positions go through `transform_world_to_cell` (ash/grid.py:753,852:
    `x / cell_size`, `(x - bbox_min) / cell_size`) before the query.  The fused
    forward applies the class's own transform inside its kernel, with torch's
    device arithmetic, and calls a transform that a user has assigned: features,
    masks and the gradients with respect to the world positions equal the
    formulation in separate calls bit for bit."""
    if kind == "unbounded":
        grid = gpu_ash.UnBoundedSparseDenseGrid(3, 4000, 4, 8, cell_size=0.0137, device=DEV)
        pts = (torch.rand(3000, 3, generator=torch.Generator().manual_seed(3)) * 2 - 1).to(DEV)
    else:
        grid = gpu_ash.BoundedSparseDenseGrid(
            3, 4000, 4, 8, sparse_grid_dim=24,
            bbox_min=torch.tensor([-0.9, -1.1, -0.7]), bbox_max=torch.tensor([1.3, 0.8, 1.0]),
            device=DEV)
        pts = (torch.rand(3000, 3, generator=torch.Generator().manual_seed(4)) * 1.4 - 0.6).to(DEV)
    if kind == "user transform":
        grid.transform_world_to_cell = lambda x: (x - grid.bbox_min) * (1.0 / grid.cell_size) + 0.25
    grid.spatial_init_(pts, dilation=1, bidirectional=True)
    with torch.no_grad():
        grid.embeddings.copy_(torch.rand(grid.embeddings.shape, device=DEV) * 2 - 1)
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    assert (grid._world_to_cell_affine(pts) is None) == (kind == "user transform")
    x = torch.cat([pts + 0.003, pts * 1.7, (torch.rand(5000, 3, device=DEV) * 2 - 1) * 1.2])
    results = {}
    for fused in (True, False):
        monkeypatch.setattr(gpu_ash.grid, "FUSED_FORWARD", fused)
        with torch.no_grad():
            f0, m0 = grid(x, "smooth_step")
        xq = x.clone().requires_grad_(True)
        grid.embeddings.grad = None
        feats, masks = grid(xq, "smooth_step")
        (gx,) = torch.autograd.grad(feats[:, 0].sum(), xq, create_graph=True)
        ((feats ** 2).sum() + (gx ** 2).sum()).backward()
        assert torch.equal(f0, feats.detach()) and torch.equal(m0, masks)
        results[fused] = (f0, m0, gx.detach(), xq.grad.clone())
    assert 0.1 < float(results[True][1].float().mean()) < 1.0
    for a, b in zip(results[True], results[False]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("grid_dim", [1, 3, 8, 16])
def test_fused_cell_query_equals_elementwise_chain(gpu_ash, grid_dim):
    """`SparseDenseGrid.query` through the fused kernel against the reference's
    chain of elementwise torch operations (ash/grid.py:183-199), bit for bit:
    random positions, integers, block boundaries and the fp32 rounding edge of
    tiny negative coordinates; gradients flow to the positions."""
    grid = _make_grid(gpu_ash, grid_dim, 2, 2, seed=grid_dim, holes=5)
    g = torch.Generator().manual_seed(50 + grid_dim)
    span = grid_dim * 4.0
    rand = (torch.rand(20000, 3, generator=g) * 2 - 1) * span
    ints = torch.randint(-3 * grid_dim, 3 * grid_dim + 1, (2000, 3), generator=g).float()
    edge = torch.tensor(
        [[-1e-9, 0.0, 0.0], [-1e-9, -1e-9, -1e-9], [grid_dim - 1e-7, 0.5, 0.5], [-0.0, 0.0, -1e-30],
         [grid_dim * 1.0, grid_dim * 2.0, -grid_dim * 1.0], [1e-7 - grid_dim, 0.25, 0.75]]
    )
    below = torch.nextafter(ints[:500], torch.full_like(ints[:500], -1e9))
    x = torch.cat([rand, ints, edge, below]).to(DEV)
    fused = grid.query(x)
    chain = grid._query_elementwise(x)
    names = ("grid_indices", "cell_indices", "offsets", "masks")
    for name, a, b in zip(names, fused, chain):
        assert a.dtype == b.dtype and a.shape == b.shape, name
        assert torch.equal(a, b), name
    assert int(fused[1].max()) < grid_dim**3 and int(fused[1].min()) >= 0
    assert float(fused[2].min()) >= 0 and float(fused[2].max()) < 1
    xg = x.clone().requires_grad_(True)
    off = grid.query(xg)[2]
    (off * torch.arange(3, device=DEV)).sum().backward()
    assert torch.equal(xg.grad, torch.arange(3, device=DEV).float().expand_as(xg))


def test_optional_gradient_outputs(gpu_ash, oracle, monkeypatch):
    """Each backward entry point may skip one of its outputs; what it still
    returns must equal the full call, and autograd asks only for what it needs
    (autograd.grad w.r.t. positions alone never builds the dense embedding
    gradient)."""
    grid = _make_grid(gpu_ash, 4, 4, 1, seed=61)
    x = _queries(4, 1, 5000, seed=62)
    ops = _operands(grid, x)
    backend = gpu_ash.grid_query.backend
    gen = torch.Generator().manual_seed(63)
    z = (torch.rand(5000, 4, generator=gen) - 0.5).to(DEV)
    u = (torch.rand(5000, 3, generator=gen) - 0.5).to(DEV)
    sums = oracle.query_term_sums(u, z, *_to_cpu(ops), 4, "smooth_step")
    order = dict(rtol=0.0, atol=0.0, eps=2.0**-24)    # same terms, another order of the atomics
    ge, go = backend.query_backward_forward(z, *ops, 4, "smooth_step")
    ge1, none1 = backend.query_backward_forward(z, *ops, 4, "smooth_step", need_offsets=False)
    none2, go2 = backend.query_backward_forward(z, *ops, 4, "smooth_step", need_embeddings=False)
    assert none1 is None and none2 is None
    assert_close_sums(ge1, ge, sums["bf_embeddings"], what="without offsets", **order)
    assert torch.equal(go2, go)
    gz, ge_b, _ = backend.query_backward_backward(None, u, z, *ops, 4, "smooth_step")
    gz1, n1, _ = backend.query_backward_backward(None, u, z, *ops, 4, "smooth_step", need_embeddings=False)
    n2, ge_b2, _ = backend.query_backward_backward(None, u, z, *ops, 4, "smooth_step", need_z=False)
    assert n1 is None and n2 is None
    assert torch.equal(gz1, gz)
    assert_close_sums(ge_b2, ge_b, sums["bb_embeddings"], what="without grad_z", **order)
    with pytest.raises(RuntimeError, match="at least one"):
        backend.query_backward_forward(
            z, *ops, 4, "smooth_step", need_embeddings=False, need_offsets=False
        )

    calls = []
    real = backend.query_backward_forward

    def spy(*args, **kwargs):
        calls.append(kwargs)
        return real(*args, **kwargs)

    backend.query_backward_forward = spy
    try:
        xq = x.clone().requires_grad_(True)
        feats, _ = grid(xq, "smooth_step")
        (gx,) = torch.autograd.grad(feats.sum(), xq, create_graph=True)
        # which branch ran: with torch._C._will_engine_execute_node the dense
        # gradient is skipped, without it the call asks for both (same numbers)
        assert hasattr(torch._C, "_will_engine_execute_node")
        assert calls == [{"need_embeddings": False, "need_offsets": True}]
        assert gpu_ash.grid_query.LAST_GRADIENT_PATH == "skipped"
        (gx.norm(dim=-1) - 1).abs().mean().backward()
        assert grid.embeddings.grad is not None
        skipping = grid.embeddings.grad.clone()
        # the conservative branch (the private call unavailable): both gradients
        # are produced, the numbers are the same
        calls.clear()
        grid.embeddings.grad = None
        with monkeypatch.context() as m:
            m.delattr(torch._C, "_will_engine_execute_node")
            xq = x.clone().requires_grad_(True)
            feats, _ = grid(xq, "smooth_step")
            (gx2,) = torch.autograd.grad(feats.sum(), xq, create_graph=True)
            assert calls == [{}] and gpu_ash.grid_query.LAST_GRADIENT_PATH == "own"
            (gx2.norm(dim=-1) - 1).abs().mean().backward()
        assert torch.equal(gx2, gx)
        # the same kernel on the same operands: only the order of the atomics differs
        assert torch.allclose(grid.embeddings.grad, skipping, rtol=RTOL32, atol=ATOL32)
    finally:
        del backend.query_backward_forward


def test_query_and_find_replay_in_a_hip_graph(gpu_ash, oracle):
    """The library allocates nothing, synchronises nowhere on these paths and
    clears its outputs with kernels, so the query kernels and the table look-up
    can be captured once and replayed; every replay is checked against the
    eager result on the inputs of that replay."""
    grid = _make_grid(gpu_ash, 4, 4, 2, seed=31, holes=6)
    backend = gpu_ash.grid_query.backend
    g = torch.Generator().manual_seed(32)
    x = _queries(4, 2, 20_000, 33)
    gi, ci, off, mk = grid.query(x.to(DEV))
    emb = grid.embeddings.detach().clone()
    z = torch.rand(x.shape[0], 4, generator=g).to(DEV) - 0.5
    tables = (grid.lut_grid_nb2grid_idx, grid.lut_cell_nb2cell_idx, grid.lut_cell_nb2grid_nb)
    keys = (torch.randint(-3, 4, (5000, 3), generator=g) ).int().to(DEV)

    def run():
        out = backend.query_forward(emb, off, gi, ci, mk, *tables, 4, "smooth_step")
        g_emb, g_off = backend.query_backward_forward(z, emb, off, gi, ci, mk, *tables, 4,
                                                      "smooth_step")
        idx, found = grid.engine.find(keys)
        return out, g_emb, g_off, idx, found

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                   # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for trial in range(3):
        emb.copy_((torch.rand(emb.shape, generator=g) * 2 - 1).to(DEV))
        z.copy_((torch.rand(z.shape, generator=g) - 0.5).to(DEV))
        keys.copy_(torch.randint(-3, 4, (5000, 3), generator=g).int().to(DEV))
        graph.replay()
        torch.cuda.synchronize()
        eager = run()
        torch.cuda.synchronize()
        assert torch.equal(captured[0], eager[0])
        sums = oracle.query_term_sums(torch.zeros(x.shape[0], 3), z, emb, off, gi, ci, mk, *tables,
                                      4, "smooth_step")
        assert_close_sums(captured[1], eager[1], sums["bf_embeddings"], rtol=0.0, atol=0.0,
                          eps=2.0**-24, what="replayed vs eager, another order of the atomics")
        assert torch.allclose(captured[2], eager[2], rtol=1e-5, atol=1e-6)
        assert torch.equal(captured[3], eager[3]) and torch.equal(captured[4], eager[4])
        assert int(eager[4].sum()) > 100 and float(eager[1].abs().sum()) > 1.0


def test_module_forward_replays_in_a_hip_graph(gpu_ash):
    """SparseDenseGrid.forward on world positions is one launch that allocates
    nothing of its own (ash_grid_forward): captured once under no_grad, every
    replay equals the eager call on the positions and embeddings of that
    replay, bit for bit, masks included."""
    grid = gpu_ash.UnBoundedSparseDenseGrid(3, 400, 4, 4, cell_size=0.25, device=DEV)
    g = torch.Generator().manual_seed(71)
    r = torch.arange(-3, 4, dtype=torch.int32)
    blocks = torch.stack(torch.meshgrid(r, r, r, indexing="ij"), dim=-1).view(-1, 3)
    grid.engine.insert_keys(blocks[torch.randperm(len(blocks), generator=g)[5:]].to(DEV))
    grid.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
    x = torch.zeros(30_000, 3, device=DEV)

    def fill():
        x.copy_(((torch.rand(x.shape, generator=g) * 9.0 - 4.0)).to(DEV))
        with torch.no_grad():
            grid.embeddings.copy_((torch.rand(grid.embeddings.shape, generator=g) * 2 - 1).to(DEV))

    fill()
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            grid(x, "smooth_step")                   # warm-up outside the capture
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = grid(x, "smooth_step")
        for _ in range(3):
            fill()
            graph.replay()
            torch.cuda.synchronize()
            features, masks = grid(x, "smooth_step")
            torch.cuda.synchronize()
            assert torch.equal(captured[0], features) and torch.equal(captured[1], masks)
            assert 1000 < int(masks.sum()) < x.shape[0] and float(features.abs().sum()) > 100.0

"""Autograd wiring of the trilinear query: forward, backward, backward of the
backward.  Two chained Functions with the same operands and return
conventions as the reference (ash/grid_query.py:10-283); each one is a single
call into the HIP library.
"""
import weakref
from typing import Literal

import torch

from .common import _get_c_extension

backend = _get_c_extension()

_N_TABLE_ARGS = 8  # grid_indices .. interpolation: operands without gradients

# One backward pass can reach the same embeddings through several nodes: a
# training step with a value loss and a gradient-norm loss runs both the first-
# and the second-order backward, and each zero-fills a dense gradient of the
# whole parameter and leaves the sum of the two to autograd (two fills and an
# add over the parameter: about a third of such a step), as in the reference.
# `dense_grad` below is the way around that.
#
# which way the embedding gradient of the latest backward node went: "own"
# (a dense tensor of its own, handed to autograd), "contract" (added to the
# parameter's .grad inside a dense_grad block), "skipped" (nobody asked for it)
LAST_GRADIENT_PATH = None


# ---------------------------------------------------------------------------
# One dense gradient per step, by contract.
#
#     optimizer.zero_grad()
#     with ash.dense_grad(grid):          # or a Parameter, or several of either
#         loss.backward()
#     optimizer.step()
#
# Inside the block every backward node of the query adds its contribution for
# a registered parameter straight into `parameter.grad` (the library's
# `_accumulate` entries) and hands autograd no gradient for it: one zero fill
# per step instead of one per node plus autograd's additions over the whole
# parameter.  On entry a parameter whose `.grad` is None gets a zero-filled
# one (filled once); an existing `.grad` is accumulated onto, as
# `loss.backward()` would.  Nothing is handed to the engine and nothing is
# learnt from it: `.grad` is looked up when a node runs, other contributions to
# the parameter (a weight-decay term, say) reach the same tensor through
# autograd's own in-place accumulation, and hooks on other nodes may keep
# whatever they like.  What differs from plain `backward()`: hooks registered
# on the parameter itself do not see the query's contributions (they bypass
# its accumulation node), and under `create_graph=True` the block has no
# effect (an in-place addition would be invisible to the recorded graph).
# The block is for `loss.backward()`: a `torch.autograd.grad(..)` *with respect
# to a registered parameter* inside it would find the query's share in `.grad`
# and not in what it returns (gradients with respect to anything else, the
# positions for instance, are not affected).
_DENSE_TARGETS = {}   # id(parameter) -> (weak reference, nesting depth)


class dense_grad:
    """Context manager: see the comment above.  `targets` are Parameters or
    modules (every parameter of a module that is an `embeddings` operand of a
    query is simply one of its parameters).  `buffers` maps a parameter to the
    tensor to install as its `.grad` when it has none (default: a new one per
    entry)."""

    def __init__(self, *targets, buffers=None):
        self.parameters = []
        for t in targets:
            if isinstance(t, torch.nn.Module):
                self.parameters.extend(p for p in t.parameters() if p.requires_grad)
            elif isinstance(t, torch.Tensor):
                self.parameters.append(t)
            else:
                raise TypeError(f"dense_grad takes parameters or modules, got {type(t)}")
        self.buffers = buffers or {}

    def __enter__(self):
        for p in self.parameters:
            if p.grad is None:
                given = self.buffers.get(p)
                if given is not None:
                    if given.shape != p.shape or given.dtype != p.dtype or given.device != p.device:
                        raise RuntimeError("dense_grad: a buffer must be like its parameter")
                    p.grad = given.zero_()
                else:
                    p.grad = torch.zeros_like(p, memory_format=torch.contiguous_format)
            ref, depth = _DENSE_TARGETS.get(id(p), (weakref.ref(p), 0))
            _DENSE_TARGETS[id(p)] = (ref, depth + 1)
        return self

    def __exit__(self, *exc):
        for p in self.parameters:
            ref, depth = _DENSE_TARGETS[id(p)]
            if depth <= 1:
                del _DENSE_TARGETS[id(p)]
            else:
                _DENSE_TARGETS[id(p)] = (ref, depth - 1)
        return False


def _dense_target(embeddings):
    """The `.grad` tensor the running node is to add to, if `embeddings` is a
    parameter registered by a `dense_grad` block that applies, else None."""
    if not _DENSE_TARGETS or torch.is_grad_enabled():
        return None
    entry = _DENSE_TARGETS.get(id(embeddings))
    if entry is None or entry[0]() is not embeddings:
        return None
    grad = embeddings.grad
    if grad is None:
        # somebody dropped it inside the block: start a new one
        grad = embeddings.grad = torch.zeros_like(embeddings, memory_format=torch.contiguous_format)
    if (grad.shape != embeddings.shape or grad.dtype != embeddings.dtype
            or grad.device != embeddings.device or not grad.is_contiguous()):
        return None
    return grad


def _record_path(path: str) -> None:
    global LAST_GRADIENT_PATH
    LAST_GRADIENT_PATH = path


def _grad_requested(ctx, index: int) -> bool:
    """Whether the running backward pass will consume the gradient of input
    `index`.  `ctx.needs_input_grad` only says that the input requires grad;
    in `autograd.grad(y, x)` the engine additionally knows which graph nodes it
    is going to execute, and the node behind an input it will not execute (the
    dense embeddings parameter, typically) needs no gradient from us."""
    if not ctx.needs_input_grad[index]:
        return False
    try:
        node = ctx.next_functions[index][0]
        return node is not None and torch._C._will_engine_execute_node(node)
    except Exception:  # outside an engine pass, or an older torch: be conservative
        return True


class SparseDenseGridQuery(torch.autograd.Function):
    """y[i] = sum over the 8 cell corners c of w_c(offsets[i]) * embeddings[row_c(i)].

    Differentiable with respect to `embeddings` and `offsets`; the indices,
    masks and neighbour tables only address memory.
    """

    @staticmethod
    def forward(
        ctx,
        embeddings: torch.Tensor,
        offsets: torch.Tensor,
        grid_indices: torch.Tensor,
        cell_indices: torch.Tensor,
        masks: torch.Tensor,
        lut_grid_nb2grid_idx: torch.Tensor,
        lut_cell_nb2cell_idx: torch.Tensor,
        lut_cell_nb2grid_nb: torch.Tensor,
        grid_dim: int,
        interpolation: Literal["linear", "smooth_step"] = "smooth_step",
    ) -> torch.Tensor:
        """embeddings (B, M, E), offsets (N, 3) in [0, 1), grid/cell indices and
        masks (N,), tables (B, 8), (M, 8), (M, 8); returns (N, E)."""
        operands = (
            embeddings,
            offsets,
            grid_indices,
            cell_indices,
            masks,
            lut_grid_nb2grid_idx,
            lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb,
        )
        ctx.save_for_backward(*operands)
        ctx.grid_dim = grid_dim
        ctx.interpolation = interpolation
        return backend.query_forward(*operands, grid_dim, interpolation)

    @staticmethod
    def backward(ctx, z: torch.Tensor):
        """Delegates to SparseDenseGridQueryBackward so that this step is itself
        differentiable (needed for gradient-norm losses)."""
        return first_order_backward(ctx, z, ctx.saved_tensors) + (None,) * _N_TABLE_ARGS


def first_order_backward(ctx, z, operands, embeddings_input: int = 0, offsets_input: int = 1):
    """(grad_embeddings, grad_offsets) of a forward node whose inputs number
    `embeddings_input` / `offsets_input` are the embeddings and (what the
    offsets depend on with unit Jacobian:) the offsets or positions; `operands`
    = (embeddings, offsets, grid_indices, cell_indices, masks, three tables)."""
    need_embeddings = _grad_requested(ctx, embeddings_input)
    need_offsets = _grad_requested(ctx, offsets_input)
    if not (need_embeddings or need_offsets):
        return None, None
    # The reference always produces both gradients (ash/grid_query.py:104-116);
    # the dense embedding gradient (zero fill + atomics over the whole
    # parameter) is skipped when nobody asked for it, e.g. in
    # autograd.grad(y, x, create_graph=True).
    target = _dense_target(operands[0]) if need_embeddings else None
    _record_path("contract" if target is not None else "own" if need_embeddings else "skipped")
    if target is not None:
        # no graph is being recorded: the library is called directly
        _, grad_offsets = backend.query_backward_forward(
            z.contiguous(),
            *operands,
            ctx.grid_dim,
            ctx.interpolation,
            need_embeddings=True,
            need_offsets=need_offsets,
            accumulate_into=target,
        )
        return None, grad_offsets
    grad_embeddings, grad_offsets = SparseDenseGridQueryBackward.apply(
        z.contiguous(),
        *operands,
        ctx.grid_dim,
        ctx.interpolation,
        need_embeddings,
        need_offsets,
    )
    return grad_embeddings, grad_offsets


class SparseDenseGridQueryBackward(torch.autograd.Function):
    """(z, embeddings, offsets) -> (grad_embeddings, grad_offsets) with

        grad_embeddings[row_c(i)] += w_c(offsets[i]) * z[i]
        grad_offsets[i] = sum_c (embeddings[row_c(i)] . z[i]) * dw_c/doffsets

    `z` may carry a graph itself (autograd.grad(..., create_graph=True)).
    """

    @staticmethod
    def forward(
        ctx,
        z,
        embeddings,
        offsets,
        grid_indices,
        cell_indices,
        masks,
        lut_grid_nb2grid_idx,
        lut_cell_nb2cell_idx,
        lut_cell_nb2grid_nb,
        grid_dim,
        interpolation,
        need_grad_embeddings: bool = True,
        need_grad_offsets: bool = True,
    ):
        """With both `need_*` flags at their default this is the reference's
        signature and result; an output that is not needed is returned as None
        and its work is skipped."""
        operands = (
            z,
            embeddings,
            offsets,
            grid_indices,
            cell_indices,
            masks,
            lut_grid_nb2grid_idx,
            lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb,
        )
        ctx.save_for_backward(*operands)
        ctx.grid_dim = grid_dim
        ctx.interpolation = interpolation
        if need_grad_embeddings and need_grad_offsets:
            return backend.query_backward_forward(*operands, grid_dim, interpolation)
        return backend.query_backward_forward(
            *operands,
            grid_dim,
            interpolation,
            need_embeddings=need_grad_embeddings,
            need_offsets=need_grad_offsets,
        )

    @staticmethod
    def backward(ctx, grad_grad_embeddings: torch.Tensor, grad_grad_offsets: torch.Tensor):
        """Given u = d loss / d grad_offsets, returns

            grad_z[i]                = sum_c (dw_c/doffsets . u[i]) * embeddings[row_c(i)]
            grad_embeddings[row_c(i)] += (dw_c/doffsets . u[i]) * z[i]

        Exactly like the reference (ash/grid_query.py:209-283,
        ash/src/grid.cu:417-426) the incoming `grad_grad_embeddings` is not used
        and no gradient flows to `offsets` at second order.
        """
        need_z, need_embeddings = _grad_requested(ctx, 0), _grad_requested(ctx, 1)
        n_rest = _N_TABLE_ARGS + 3  # offsets, tables, grid_dim, interpolation, 2 flags
        if grad_grad_offsets is None or not (need_z or need_embeddings):
            return (None, None) + (None,) * n_rest
        target = _dense_target(ctx.saved_tensors[1]) if need_embeddings else None
        _record_path("contract" if target is not None else "own" if need_embeddings else "skipped")
        if target is not None:
            grad_z, _, _ = backend.query_backward_backward(
                grad_grad_embeddings,
                grad_grad_offsets,
                *ctx.saved_tensors,
                ctx.grid_dim,
                ctx.interpolation,
                need_z=need_z,
                need_embeddings=True,
                accumulate_into=target,
            )
            return (grad_z, None) + (None,) * n_rest
        if need_z and need_embeddings:
            grad_z, grad_embeddings, _ = backend.query_backward_backward(
                grad_grad_embeddings,
                grad_grad_offsets,
                *ctx.saved_tensors,
                ctx.grid_dim,
                ctx.interpolation,
            )
        else:
            grad_z, grad_embeddings, _ = backend.query_backward_backward(
                grad_grad_embeddings,
                grad_grad_offsets,
                *ctx.saved_tensors,
                ctx.grid_dim,
                ctx.interpolation,
                need_z=need_z,
                need_embeddings=need_embeddings,
            )
        return (grad_z, grad_embeddings) + (None,) * n_rest

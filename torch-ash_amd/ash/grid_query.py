"""Autograd wiring of the trilinear query: forward, backward, backward of the
backward.  Two chained Functions with the same operands and return
conventions as the reference (ash/grid_query.py:10-283); each one is a single
call into the HIP library.
"""
import os
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
#
# SHARE_DENSE_GRADIENT (off unless the caller switches it on, here or with
# ASH_SHARE_DENSE_GRADIENT=1) saves the second fill and the add: the first node
# of a pass that produces the gradient for a leaf parameter leaves a note with
# the parameter's accumulation node -- the graph task, the stream and a weak
# reference to the tensor, in the node's own metadata dictionary, so that the
# note lives and dies with the node -- and a later node of the same pass adds its
# contribution to that tensor in place and returns no gradient of its own.
#
# Why it is a switch: the in-place addition is only right while the tensor the
# first node returned still is what the autograd engine holds for the
# parameter.  The engine replaces it by a new tensor when a further gradient
# for the same parameter arrives (a weight-decay term, say) while something
# else still refers to the first one -- a hook on this function's grad_fn that
# keeps its grad_inputs is enough -- and this code cannot see that; the later
# contribution would then be lost.  Without such references the engine adds
# in place (or autograd drops the tensor and the weak reference dies, and the
# node falls back to a gradient of its own).  So: switch it on for training
# loops that keep no references to intermediate gradients.
#
# Shared only: with the switch on, without create_graph (an in-place change
# would be invisible to a graph recorded over the first gradient), towards the
# accumulation node of a leaf, by nodes that run on the same stream.
_NOTE = "ash_shared_gradient"
SHARE_DENSE_GRADIENT = os.environ.get("ASH_SHARE_DENSE_GRADIENT", "0") not in ("", "0")
# which way the embedding gradient of the latest backward node went: "own"
# (a dense tensor of its own), "shared" (added to another node's), "skipped"
LAST_GRADIENT_PATH = None


def _pass_id() -> int:
    if not SHARE_DENSE_GRADIENT or torch.is_grad_enabled():
        return -1
    try:
        return torch._C._current_graph_task_id()
    except Exception:  # older torch
        return -1


def _notes(consumer):
    """(graph task, dictionary of the consumer node, key) or None."""
    task = _pass_id()
    if task < 0 or consumer is None or consumer[0] is None:
        return None
    node = consumer[0]
    # only the accumulation node of a leaf: what it receives is added to .grad
    # and goes nowhere else
    if type(node).__name__ != "AccumulateGrad":
        return None
    try:
        return task, node.metadata, (_NOTE, consumer[1])
    except Exception:  # a node without metadata
        return None


def _stream_id(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream if t.is_cuda else 0


def _shared_gradient(consumer):
    """The gradient another node of the running pass already produced for
    `consumer`, or None."""
    notes = _notes(consumer)
    if notes is None:
        return None
    task, where, key = notes
    entry = where.get(key)
    if entry is None or entry[0] != task:
        return None
    gradient = entry[2]()
    if gradient is None or entry[1] != _stream_id(gradient):
        return None
    return gradient


def _share_gradient(consumer, gradient) -> None:
    notes = _notes(consumer)
    if notes is None or gradient is None:
        return
    task, where, key = notes
    where[key] = (task, _stream_id(gradient), weakref.ref(gradient))


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
        need_embeddings, need_offsets = _grad_requested(ctx, 0), _grad_requested(ctx, 1)
        if not (need_embeddings or need_offsets):
            return (None,) * (2 + _N_TABLE_ARGS)
        # The reference always produces both gradients (ash/grid_query.py:104-116);
        # the dense embedding gradient (zero fill + atomics over the whole
        # parameter) is skipped when nobody asked for it, e.g. in
        # autograd.grad(y, x, create_graph=True).
        consumer = ctx.next_functions[0] if need_embeddings else None
        shared = _shared_gradient(consumer)
        _record_path("shared" if shared is not None else "own" if need_embeddings else "skipped")
        if shared is not None:
            # no graph is being recorded: the library is called directly
            _, grad_offsets = backend.query_backward_forward(
                z.contiguous(),
                *ctx.saved_tensors,
                ctx.grid_dim,
                ctx.interpolation,
                need_embeddings=True,
                need_offsets=need_offsets,
                accumulate_into=shared,
            )
            return (None, grad_offsets) + (None,) * _N_TABLE_ARGS
        grad_embeddings, grad_offsets = SparseDenseGridQueryBackward.apply(
            z.contiguous(),
            *ctx.saved_tensors,
            ctx.grid_dim,
            ctx.interpolation,
            need_embeddings,
            need_offsets,
        )
        _share_gradient(consumer, grad_embeddings)
        return (grad_embeddings, grad_offsets) + (None,) * _N_TABLE_ARGS


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
        consumer = ctx.next_functions[1] if need_embeddings else None
        shared = _shared_gradient(consumer)
        _record_path("shared" if shared is not None else "own" if need_embeddings else "skipped")
        if shared is not None:
            grad_z, _, _ = backend.query_backward_backward(
                grad_grad_embeddings,
                grad_grad_offsets,
                *ctx.saved_tensors,
                ctx.grid_dim,
                ctx.interpolation,
                need_z=need_z,
                need_embeddings=True,
                accumulate_into=shared,
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
        _share_gradient(consumer, grad_embeddings)
        return (grad_z, grad_embeddings) + (None,) * n_rest

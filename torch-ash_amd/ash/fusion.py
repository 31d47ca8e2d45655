"""TSDF fusion of depth frames into a sparse-dense grid: the per-frame step of
the reference's demo (demo/rgbd_fusion.py:200-254) on two fused library calls.

The reference activates blocks with `spatial_init_` and then updates
`embeddings[grid_indices, cell_indices]` through torch expressions
(`project_points_to_rgbd`, demo/rgbd_fusion.py:76-110, and the running weighted
mean, :232-254).  Here the activation is one kernel (positions in, blocks
inserted, their rows flagged) and the projection + update another that rewrites
the embedding rows of the flagged blocks in place.  Row layout as in the demo: channel 0 signed distance, channels 1..3
colour (only when a colour image is given), last channel weight.
"""
from typing import Optional

import torch

from .common import COLLECT_MAX_BLOCKS, _get_c_extension
from .grid import SparseDenseGrid

backend = _get_c_extension()


@torch.no_grad()
def integrate_depth(
    grid: SparseDenseGrid,
    grid_coords: torch.Tensor,
    grid_indices: torch.Tensor,
    depth: torch.Tensor,
    intrinsic: torch.Tensor,
    extrinsic: torch.Tensor,
    trunc: float,
    depth_max: float,
    color: Optional[torch.Tensor] = None,
    counted_by=None,
    flagged_by=None,
) -> None:
    """Projects every cell of the listed blocks into `depth` (H, W; metres, 0 =
    no reading) with the pinhole `intrinsic` (3, 3) and the world-to-camera
    `extrinsic` (4, 4) and folds the truncated signed distance (and `color`
    (H, W, 3), if given) into the grid's embedding rows.  `counted_by`: the
    table whose deferred activation made the listing (its length is then read
    on the device); `flagged_by`: the table whose `activate_positions` flagged
    the blocks (no listing at all: pass None for the first two)."""
    scale, origin = grid._cell_to_world_affine()
    backend.integrate_depth(
        grid.embeddings.data,
        grid_indices,
        grid_coords,
        grid.grid_dim,
        scale,
        origin,
        intrinsic,
        extrinsic,
        depth,
        color,
        trunc,
        depth_max,
        counted_by=counted_by,
        flagged_by=flagged_by,
    )


@torch.no_grad()
def fuse_frame(
    grid: SparseDenseGrid,
    points: torch.Tensor,
    depth: torch.Tensor,
    intrinsic: torch.Tensor,
    extrinsic: torch.Tensor,
    trunc: float,
    depth_max: float,
    color: Optional[torch.Tensor] = None,
    dilation: int = 1,
    count_blocks: bool = True,
) -> Optional[int]:
    """One fusion step: activate the blocks around the unprojected `points`
    (world coordinates) with a two-sided dilation, then integrate the frame
    into them.  Returns the number of touched blocks -- or, with
    `count_blocks=False`, nothing: the frame then runs without a single
    read-back from the device (the reference's loop needs the number to size
    its tensors, demo/rgbd_fusion.py:216-254; the kernels here read it where it
    is), the host only queues launches, and the reference's capacity warning
    comes with the next call that reads the table's counters."""
    if not count_blocks and points.shape[0] > 0 and points.dtype == torch.float32:
        affine = grid._world_to_cell_affine(points)
        if affine is not None:
            # three launches: the transform is applied inside the activation
            # kernels, which flag the touched rows; the integration goes by the
            # flags and takes them down
            lo, hi = grid._block_bounds()
            table = grid.engine.backend
            table.activate_positions(points, affine[0], affine[1], grid.grid_dim, dilation, True,
                                     lo, hi)
            integrate_depth(grid, None, None, depth, intrinsic, extrinsic, trunc, depth_max,
                            color, flagged_by=table)
            return None
    if not count_blocks and points.shape[0] > 0 and grid.engine.capacity <= COLLECT_MAX_BLOCKS:
        cells = grid.transform_world_to_cell(points)
        if cells.dtype == torch.float32:
            lo, hi = grid._block_bounds()
            table = grid.engine.backend
            grid_coords, grid_indices = table.activate_blocks_deferred(
                cells, grid.grid_dim, dilation, True, lo, hi
            )
            integrate_depth(
                grid, grid_coords, grid_indices, depth, intrinsic, extrinsic, trunc, depth_max,
                color, counted_by=table,
            )
            return None
    if (count_blocks and points.shape[0] > 0 and points.dtype == torch.float32
            and grid.engine.capacity <= COLLECT_MAX_BLOCKS):
        # the same launches as without the count (activation, listing on the
        # device, integration over the listing), and one look at the table's
        # counters behind them all -- not between activation and integration
        engine = grid.engine
        table = engine.backend
        cells = grid.transform_world_to_cell(points)
        lo, hi = grid._block_bounds()
        dropped_before = engine._dropped()
        grid_coords, grid_indices = table.activate_blocks_deferred(
            cells, grid.grid_dim, dilation, True, lo, hi
        )
        integrate_depth(
            grid, grid_coords, grid_indices, depth, intrinsic, extrinsic, trunc, depth_max,
            color, counted_by=table,
        )
        touched = table.counters()["touched"]
        engine._warn_if_overfull(points.shape[0], dropped_before)
        return int(touched)
    grid_coords, _, grid_indices, _ = grid.spatial_init_(
        points, dilation=dilation, bidirectional=True
    )
    if grid_indices.numel() == 0:
        return 0
    integrate_depth(
        grid, grid_coords, grid_indices, depth, intrinsic, extrinsic, trunc, depth_max, color
    )
    return int(grid_indices.shape[0])

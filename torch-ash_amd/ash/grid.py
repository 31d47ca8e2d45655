"""Sparse-dense grids: a hash map of active blocks, each a dense G^3 array of
cells carrying an embedding row.

Public names, shapes and semantics follow ash/grid.py:29-863: allocation,
query, interpolation, enumeration, neighbour tables and coordinate transforms
on the query path, and around it ray sampling, filtering / convolution and
surface extraction, each on the library's kernel for it.
"""
from typing import Literal, Optional, Tuple, Union

import torch
import torch.nn as nn

from .common import _get_c_extension
from .core import ASHEngine, ASHModule
from .grid_nns import enumerate_neighbor_coord_offsets
from .grid_query import SparseDenseGridQuery, first_order_backward
from .hashmap import HashSet

backend = _get_c_extension()

# spatial_init_ through the library's activation kernels (one pass over the
# positions); False = the reference's formulation: candidate expansion, scratch
# hash set, insert, find.  Both leave the same map and return the same blocks.
FUSED_ACTIVATION = True

# From this many active blocks on, the functions that walk all blocks list them
# along a Z-order curve (see SparseDenseGrid._blocks_in_spatial_order).
SPATIAL_ORDER_MIN_BLOCKS = 4096

Interpolation = Literal["nearest", "linear", "smooth_step"]


class _FusedCellQuery(torch.autograd.Function):
    """x (cell units) -> (grid_indices, cell_indices, offsets, masks) through the
    table's fused kernel.  Only `offsets` depends differentiably on x, with unit
    Jacobian (offsets = x - floor(x) up to block shifts)."""

    @staticmethod
    def forward(ctx, x, table, grid_dim):
        grid_indices, cell_indices, offsets, masks = table.query_cells(x, grid_dim)
        ctx.mark_non_differentiable(grid_indices, cell_indices, masks)
        return grid_indices, cell_indices, offsets, masks

    @staticmethod
    def backward(ctx, _grad_grid, _grad_cell, grad_offsets, _grad_masks):
        return grad_offsets, None, None


# `SparseDenseGrid.forward` through the library's fused kernel (positions ->
# features in one launch, the intermediate index / offset arrays written only
# when a backward pass will read them); False = `query` and the interpolation
# as two calls, as the reference has them.  Same numbers either way.
FUSED_FORWARD = True


class _FusedGridForward(torch.autograd.Function):
    """(embeddings, x in cell units) -> (features, masks) in one kernel; the
    operands of the backward pass (block / cell indices, offsets) come out of
    the same kernel.  Differentiable like `query` followed by
    `SparseDenseGridQuery`: with respect to the embeddings and, through the
    offsets (unit Jacobian), to x; the backward is itself differentiable."""

    @staticmethod
    def forward(ctx, embeddings, x, table, lut_grid_nb2grid_idx, lut_cell_nb2cell_idx,
                lut_cell_nb2grid_nb, grid_dim, interpolation, origin, cell_size):
        features, masks, grid_indices, cell_indices, offsets = backend.grid_forward(
            table, x, embeddings, lut_grid_nb2grid_idx, lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb, grid_dim, interpolation, need_operands=True,
            origin=origin, cell_size=cell_size,
        )
        ctx.save_for_backward(embeddings, offsets, grid_indices, cell_indices, masks,
                              lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb)
        ctx.grid_dim = grid_dim
        ctx.interpolation = interpolation
        ctx.cell_size = cell_size
        ctx.mark_non_differentiable(masks)
        return features, masks

    @staticmethod
    def backward(ctx, z, _grad_masks):
        grad_embeddings, grad_x = first_order_backward(ctx, z, ctx.saved_tensors, 0, 1)
        if grad_x is not None and ctx.cell_size != 1.0:
            # d cell / d x of x -> (x - origin) / cell_size, as autograd has it
            grad_x = grad_x / ctx.cell_size
        return (grad_embeddings, grad_x) + (None,) * 8


class SparseDenseGrid(ASHModule):
    """Grid addressed in cell units: position x lies in block floor(x / G) and,
    inside it, in cell floor(x - G * block).

    `embeddings` has shape (num_embeddings, G**3, embedding_dim); the row of a
    cell is `embeddings[grid_index, cell_index]` with
    cell_index = cx + G * cy + G**2 * cz.
    """

    def __init__(
        self,
        in_dim: int,
        num_embeddings: int,
        embedding_dim: int,
        grid_dim: int,
        device: Optional[Union[str, torch.device]] = torch.device("cpu"),
    ):
        assert in_dim == 3, "Only 3D sparse-dense grid is supported for now."
        assert embedding_dim <= 16, "Embedding dim must be <= 16 for now."
        super().__init__()

        self.transform_world_to_cell = lambda x: x
        self.transform_cell_to_world = lambda x: x
        self._remember_world_to_cell(lambda: (None, 1.0))

        self.in_dim = in_dim
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.grid_dim = grid_dim
        self.device = torch.device(device) if isinstance(device, str) else device

        self.engine = ASHEngine(in_dim, num_embeddings, device)
        self.num_cells_per_grid = grid_dim**in_dim
        self.embeddings = nn.Parameter(
            torch.zeros(num_embeddings, self.num_cells_per_grid, embedding_dim, device=device)
        )

        # Per-cell constants: the dense part has the same structure in every block.
        self.cell_indices = torch.arange(
            self.num_cells_per_grid, dtype=torch.long, device=self.device
        )
        self.cell_coords = self._delinearize_cell_indices(self.cell_indices)
        assert self.cell_coords.shape == (self.num_cells_per_grid, in_dim)
        self.lut_cell_nb2grid_nb, self.lut_cell_nb2cell_idx = self.construct_cell_neighbor_lut(
            radius=1, bidirectional=False
        )

        # Per-block tables exist only once blocks have been activated.
        self.grid_indices = None
        self.grid_coords = None
        self.lut_grid_nb2grid_idx = None

    # ------------------------------------------------------------ activation
    def spatial_init_(
        self, points: torch.Tensor, dilation: int = 1, bidirectional: bool = False
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Activates the blocks containing `points` (world coordinates) and their
        neighbours within `dilation` blocks (ash/grid.py:121-159).

        Returns the touched blocks in broadcastable form:
        grid_coords (n, 1, 3), cell_coords (1, M, 3), grid_indices (n, 1),
        cell_indices (1, M).
        """
        cells = self.transform_world_to_cell(points)
        table = self.engine.backend
        if (
            FUSED_ACTIVATION
            and hasattr(table, "activate_blocks")
            and self.in_dim == 3
            and cells.dtype == torch.float32
            and len(cells) > 0
        ):
            # one pass over the positions instead of candidate expansion +
            # scratch set + insert + find; same set of touched blocks
            lo, hi = self._block_bounds()
            dropped_before = self.engine._dropped()
            unique_coords, grid_indices = table.activate_blocks(
                cells, self.grid_dim, dilation, bidirectional, lo, hi
            )
            self.engine._warn_if_overfull(len(cells), dropped_before)
            return (
                unique_coords.view(-1, 1, self.in_dim),
                self.cell_coords.view(1, -1, self.in_dim),
                grid_indices.view(-1, 1),
                self.cell_indices.view(1, -1),
            )
        block_coords = self.grids_in_bound(torch.floor(cells / self.grid_dim).int())

        nb_offsets, _ = enumerate_neighbor_coord_offsets(
            self.in_dim, dilation, bidirectional=bidirectional, device=self.device
        )
        candidates = (block_coords.view(-1, 1, 3) + nb_offsets).view(-1, 3)

        unique_coords = self.grids_in_bound(self._unique_keys(candidates, len(block_coords)))

        self.engine.insert_keys(unique_coords)
        grid_indices, masks = self.engine.find(unique_coords)
        assert masks.all()

        return (
            unique_coords.view(-1, 1, self.in_dim),
            self.cell_coords.view(1, -1, self.in_dim),
            grid_indices.view(-1, 1),
            self.cell_indices.view(1, -1),
        )

    def _unique_keys(self, candidates: torch.Tensor, num_sources: int) -> torch.Tensor:
        """Distinct rows of `candidates` through a scratch hash set.  The
        reference sizes that set by the number of source points
        (ash/grid.py:145), which is too small when few points are dilated
        widely; here a set that turns out too small is retried at the size that
        cannot fail."""
        if len(candidates) == 0:
            return candidates
        first_try = min(len(candidates), max(num_sources, 1024))
        for capacity in (first_try, len(candidates)):
            scratch = HashSet(key_dim=3, capacity=capacity, device=self.device)
            scratch.engine.backend.insert_keys(candidates.int().contiguous())
            if capacity == len(candidates) or scratch.engine.backend.status()["dropped"] == 0:
                return scratch.keys()
        raise AssertionError("unreachable")

    def ray_init_(self, ray_o, rays_d, rays_near, rays_far, dilation: int = 3) -> None:
        raise NotImplementedError("Ray-tracing initialization not implemented yet")

    # ----------------------------------------------------------------- query
    def query(
        self, x: torch.Tensor
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Splits positions (cell units) into block / cell / fractional parts
        (ash/grid.py:183-199).

        Returns grid_indices (N,), cell_indices (N,), offsets (N, 3) in [0, 1),
        masks (N,) = block is active.
        """
        table = self.engine.backend
        if hasattr(table, "query_cells") and x.dtype == torch.float32 and len(x) > 0:
            # one kernel instead of the elementwise chain; same numbers
            return _FusedCellQuery.apply(x, table, self.grid_dim)
        return self._query_elementwise(x)

    def _query_elementwise(self, x: torch.Tensor):
        """`query` as a chain of elementwise torch operations around one find,
        as the reference writes it; used for inputs the fused kernel does not
        take (non-fp32 positions, empty batches)."""
        g = self.grid_dim
        x_sparse = (x / g).floor()
        x_dense = x - x_sparse * g
        # Two fp32 rounding cases right at a block boundary, where the plain
        # formula leaves [0, g): x / g rounds up to an integer although x lies
        # just below the boundary (x_dense < 0), and x - x_sparse * g rounds to
        # exactly g for tiny negative x.  Both are moved back into range.
        under = (x_dense < 0).to(x_dense.dtype)
        x_sparse = x_sparse - under
        x_dense = x_dense + under * g
        spill = (x_dense >= g).to(x_dense.dtype)
        x_sparse = x_sparse + spill
        x_dense = x_dense - spill * g
        offsets = x_dense - x_dense.floor()

        grid_indices, masks = self.engine.find(x_sparse.int())
        cell_indices = self._linearize_cell_coords(x_dense.int())
        return grid_indices, cell_indices, offsets, masks

    def forward(
        self, x: torch.Tensor, interpolation: Interpolation = "smooth_step"
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Embeddings at world positions x (N, 3): features (N, E) and the mask
        of positions that fall into an active block (ash/grid.py:201-238)."""
        if interpolation not in ("nearest", "linear", "smooth_step"):
            raise ValueError(f"Unknown interpolation: {interpolation}")
        table = self.engine.backend
        if (
            FUSED_FORWARD
            and interpolation != "nearest"
            and hasattr(backend, "grid_forward")
            and hasattr(table, "query_cells")
            and x.dtype == torch.float32
            and x.dim() == 2
            and len(x) > 0
            and self.embeddings.is_contiguous()
        ):
            if self.grid_coords is None or self.lut_grid_nb2grid_idx is None:
                self.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
            tables = (self.lut_grid_nb2grid_idx, self.lut_cell_nb2cell_idx,
                      self.lut_cell_nb2grid_nb)
            # world -> cell units inside the kernel when the transform is the
            # class's own affine one, else by calling it
            affine = self._world_to_cell_affine(x)
            if affine is None:
                x = self.transform_world_to_cell(x)
                affine = (None, 1.0)
            if (
                x.dtype == torch.float32 and torch.is_grad_enabled()
                and (x.requires_grad or self.embeddings.requires_grad)
            ):
                return _FusedGridForward.apply(self.embeddings, x, table, *tables,
                                               self.grid_dim, interpolation, *affine)
            if x.dtype == torch.float32:
                # nobody will ask for a gradient: the intermediate arrays are
                # not even written
                features, masks, _, _, _ = backend.grid_forward(
                    table, x.detach(), self.embeddings.detach(), *tables, self.grid_dim,
                    interpolation, need_operands=False, origin=affine[0], cell_size=affine[1])
                return features, masks
        else:
            x = self.transform_world_to_cell(x)

        grid_indices, cell_indices, offsets, masks = self.query(x)

        if interpolation == "nearest":
            return self.embeddings[grid_indices, cell_indices], masks

        if self.grid_coords is None or self.lut_grid_nb2grid_idx is None:
            self.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
        features = SparseDenseGridQuery.apply(
            self.embeddings,
            offsets,
            grid_indices,
            cell_indices,
            masks,
            self.lut_grid_nb2grid_idx,
            self.lut_cell_nb2cell_idx,
            self.lut_cell_nb2grid_nb,
            self.grid_dim,
            interpolation,
        )
        return features, masks

    @torch.no_grad()
    def _blocks_in_spatial_order(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """(grid_coords (n, 3), grid_indices (n,)) of the active blocks along a
        Z-order curve instead of in table order.  Kernels that walk the listing
        and read across block faces (surface extraction, convolution) then find
        the cells of neighbouring blocks in cache; their results do not depend
        on the order of the listing."""
        # kept while the table holds the same keys (its shim counts the calls
        # that may change them)
        table = self.engine.backend
        stamp = (id(table), getattr(table, "version", None))
        cached = getattr(self, "_spatial_order_cache", None)
        if stamp[1] is not None and cached is not None and cached[0] == stamp:
            return cached[1], cached[2]
        keys, indices = self.engine.items()
        if len(indices) < SPATIAL_ORDER_MIN_BLOCKS:
            return keys, indices

        def spread(v):  # bit i of v -> bit 3 i
            v = v & 0x1FFFFF
            v = (v | (v << 32)) & 0x1F00000000FFFF
            v = (v | (v << 16)) & 0x1F0000FF0000FF
            v = (v | (v << 8)) & 0x100F00F00F00F00F
            v = (v | (v << 4)) & 0x10C30C30C30C30C3
            v = (v | (v << 2)) & 0x1249249249249249
            return v

        k = (keys - keys.min(dim=0)[0]).long()
        code = spread(k[:, 0]) | (spread(k[:, 1]) << 1) | (spread(k[:, 2]) << 2)
        order = torch.argsort(code)
        keys, indices = keys[order], indices[order]
        self._spatial_order_cache = (stamp, keys, indices)
        return keys, indices

    def items(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Active blocks in broadcastable form (ash/grid.py:240-266):
        grid_coords (n, 1, 3), cell_coords (1, M, 3), grid_indices (n, 1),
        cell_indices (1, M); integer cell positions are
        grid_coords * G + cell_coords and their rows
        embeddings[grid_indices, cell_indices]."""
        grid_coords, grid_indices = self.engine.items()
        return (
            grid_coords.view(-1, 1, self.in_dim),
            self.cell_coords.view(1, -1, self.in_dim),
            grid_indices.view(-1, 1),
            self.cell_indices.view(1, -1),
        )

    # ------------------------------------------------------------ transforms
    @torch.no_grad()
    def get_bbox(self):
        return self.bbox_min, self.bbox_max

    def cell_to_world(self, grid_coords: torch.Tensor, cell_coords: torch.Tensor) -> torch.Tensor:
        """(n,1,3) block coords x (1,M,3) cell coords -> (n*M, 3) world positions."""
        cells = grid_coords.view(-1, 1, self.in_dim) * self.grid_dim + cell_coords.view(
            1, -1, self.in_dim
        )
        return self.transform_cell_to_world(cells).view(-1, self.in_dim)

    def grids_in_bound(self, grid_coords: torch.Tensor) -> torch.Tensor:
        """Unbounded by default; the bounded grid filters here."""
        return grid_coords

    def _block_bounds(self) -> Tuple[int, int]:
        """Inclusive range of block coordinates `grids_in_bound` lets through
        (all of int32 short of the dilation range when unbounded)."""
        return -(2**31) + 64, 2**31 - 65

    def _remember_world_to_cell(self, affine) -> None:
        """Notes that `transform_world_to_cell`, as it stands now, is
        x -> (x - origin) / cell_size with (origin, cell_size) = affine(); while
        the attribute still holds that function the fused forward applies the
        transform inside its kernel.  A transform assigned later by a user is
        simply called."""
        self._world_to_cell_known = (self.transform_world_to_cell, affine)

    def _world_to_cell_affine(self, like: torch.Tensor):
        """(origin float32[3] on the device or None, cell_size) if the fused
        kernel can apply `transform_world_to_cell` to `like` itself, else None."""
        fn, affine = self._world_to_cell_known
        if self.transform_world_to_cell is not fn:
            return None
        origin, cell_size = affine()
        if origin is not None and (
            not torch.is_tensor(origin) or origin.dtype != torch.float32
            or origin.device != like.device or origin.numel() != 3 or origin.requires_grad
        ):
            return None
        if torch.is_tensor(cell_size) or not (0.0 < float(cell_size) < float("inf")):
            return None
        return origin, float(cell_size)

    def _cell_to_world_affine(self) -> Tuple[float, Optional[torch.Tensor]]:
        """`transform_cell_to_world` as (scale, origin): world = cell * scale
        [+ origin]."""
        return 1.0, None

    @torch.no_grad()
    def _linearize_cell_coords(self, cell_coords: torch.Tensor) -> torch.Tensor:
        """(N, 3) cell coordinates -> int64 cell index cx + G*cy + G^2*cz."""
        assert cell_coords.dim() == 2 and cell_coords.shape[1] == self.in_dim
        index = torch.zeros(cell_coords.shape[0], dtype=torch.long, device=cell_coords.device)
        for d in range(self.in_dim):
            index += cell_coords[:, d].long() * self.grid_dim**d
        return index

    @torch.no_grad()
    def _delinearize_cell_indices(self, cell_indices: torch.Tensor) -> torch.Tensor:
        """Inverse of `_linearize_cell_coords`; int32 coordinates, last dim 3."""
        rest = cell_indices.clone()
        coords = []
        for _ in range(self.in_dim):
            coords.append(rest % self.grid_dim)
            rest = torch.div(rest, self.grid_dim, rounding_mode="floor")
        return torch.stack(coords, dim=-1).int()

    # -------------------------------------------------------------- sampling
    def uniform_sample(
        self, num_samples: int, space: Literal["occupied", "empty"] = "occupied"
    ) -> torch.Tensor:
        """World positions drawn uniformly inside randomly chosen active blocks
        (ash/grid.py:405-430)."""
        if space != "occupied":
            raise NotImplementedError("empty space sampling not implemented")
        active_coords, _ = self.engine.items()
        pick = torch.randint(len(active_coords), (num_samples,), device=self.device)
        inside = torch.rand(num_samples, self.in_dim, device=self.device)
        return self.transform_cell_to_world((active_coords[pick].float() + inside) * self.grid_dim)

    # Native kernels of the reference that are not part of the query path.
    @torch.no_grad()
    def ray_sample(
        self,
        rays_o: torch.Tensor,
        rays_d: torch.Tensor,
        rays_near,
        rays_far,
        max_samples_per_ray: int,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Samples along rays inside active blocks (ash/grid.py:322-377).

        rays_o, rays_d (N, 3) world coordinates; rays_near / rays_far per-ray
        ranges (tensors as returned by `ray_find_near_far`, or numbers).
        Returns ray_indices (M,), t_near (M,), t_far (M,) in world units and
        the inclusive prefix sum of the per-ray sample counts (N,).  Sample
        positions are rays_o[ray_indices] + (t_near + t_far) / 2 *
        rays_d[ray_indices]."""
        bbox_min, bbox_max = self.get_bbox()
        ray_indices, t_nears, t_fars, ray_prefix_sum = backend.ray_sample(
            self.engine.backend,
            self.transform_world_to_cell(rays_o),
            rays_d,
            rays_near / self.cell_size,
            rays_far / self.cell_size,
            self.transform_world_to_cell(bbox_min),
            self.transform_world_to_cell(bbox_max),
            max_samples_per_ray,
            float(self.grid_dim),
        )
        return (ray_indices, t_nears * self.cell_size, t_fars * self.cell_size, ray_prefix_sum)

    @torch.no_grad()
    def ray_find_near_far(
        self, rays_o: torch.Tensor, rays_d: torch.Tensor, t_min: float, t_max: float, t_step: float
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Per-ray range that contains active blocks (ash/grid.py:379-403), in
        world units; near is negative where a ray meets no active block."""
        bbox_min, bbox_max = self.get_bbox()
        ray_nears, ray_fars = backend.ray_find_near_far(
            self.engine.backend,
            self.transform_world_to_cell(rays_o),
            rays_d,
            self.transform_world_to_cell(bbox_min),
            self.transform_world_to_cell(bbox_max),
            t_min / self.cell_size,
            t_max / self.cell_size,
            t_step / self.cell_size,
            float(self.grid_dim),
        )
        return (ray_nears * self.cell_size, ray_fars * self.cell_size)

    @torch.no_grad()
    def gaussian_filter_(self, size: int, sigma: float) -> None:
        """Smooths the embeddings in place with a size^3 Gaussian window
        (ash/grid.py:435-476): per-axis weights are the normal probability mass
        of `size` equal bins over [-sigma, sigma], normalised, and the window is
        their outer product, the same for every channel."""
        assert size % 2 == 1, "size must be odd"
        import numpy as np
        import scipy.stats as st

        edges = np.linspace(-sigma, sigma, size + 1)
        axis = np.diff(st.norm.cdf(edges))
        window = np.outer(axis, np.outer(axis, axis)).reshape((size, size, size))
        window = torch.from_numpy(window / window.sum()).float()
        channels = self.embeddings.shape[-1]
        weights = window.view(size, size, size, 1).repeat(1, 1, 1, channels)
        weights = weights.to(self.embeddings.device)
        self.embeddings.copy_(self.convolution(self.embeddings, weights))

    def convolution(self, inputs: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        """Per-channel sparse convolution over the active cells
        (ash/grid.py:478-520).  inputs (num_embeddings, cells_per_grid, C) laid
        out like the embeddings; weights (2R+1, 2R+1, 2R+1, C), first axis =
        slowest neighbour offset; neighbours in missing blocks count as zero.
        Forward only, like the reference."""
        assert inputs.is_contiguous()
        assert inputs.shape[:2] == self.embeddings.shape[:2]
        assert weights.is_contiguous()
        assert len(weights.shape) == 4
        assert weights.shape[0] % 2 == 1
        radius = weights.shape[0] // 2
        for d in range(3):
            assert weights.shape[d] == 2 * radius + 1
        assert weights.shape[3] == inputs.shape[-1]
        assert weights.device == inputs.device

        lut_cell_nb2grid_nb, lut_cell_nb2cell_idx, lut_grid_nb2grid_idx = self._window_tables(radius)
        _, grid_indices = self._blocks_in_spatial_order()
        cell_indices = self.cell_indices
        num_cell_nbs = lut_cell_nb2grid_nb.shape[1]
        return backend.convolution_forward(
            inputs,
            weights.view(num_cell_nbs, weights.shape[-1]),
            torch.ones(inputs.shape[:2], dtype=torch.bool, device=inputs.device),
            grid_indices,
            cell_indices,
            lut_grid_nb2grid_idx,
            lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb,
            self.grid_dim,
        )

    def _window_tables(self, radius: int):
        """The three tables of a (2 radius + 1)^3 window: the per-cell pair
        depends on the block size alone and is built once per radius, the
        per-block one is kept while the table holds the same keys (as the
        Z-order listing)."""
        cell_tables = getattr(self, "_window_cell_tables", None)
        if cell_tables is None:
            cell_tables = self._window_cell_tables = {}
        if radius not in cell_tables:
            cell_tables[radius] = self.construct_cell_neighbor_lut(radius, bidirectional=True)
        lut_cell_nb2grid_nb, lut_cell_nb2cell_idx = cell_tables[radius]
        grid_radius = (radius + self.grid_dim - 1) // self.grid_dim
        table = self.engine.backend
        stamp = (id(table), getattr(table, "version", None), grid_radius)
        cached = getattr(self, "_window_block_table", None)
        if stamp[1] is not None and cached is not None and cached[0] == stamp:
            lut_grid_nb2grid_idx = cached[1]
        else:
            _, lut_grid_nb2grid_idx = self.construct_grid_neighbor_lut(grid_radius, bidirectional=True)
            self._window_block_table = (stamp, lut_grid_nb2grid_idx)
        return lut_cell_nb2grid_nb, lut_cell_nb2cell_idx, lut_grid_nb2grid_idx

    @torch.no_grad()
    def isosurface_points(
        self, tsdfs: torch.Tensor, weights: torch.Tensor, iso_value: float = 0.0,
        weight_thr: float = 1.0,
    ) -> torch.Tensor:
        """World positions (P, 3) where `tsdfs` crosses `iso_value` on the cell
        edges of the active blocks, both end points weighing at least
        `weight_thr`: the `vertices_only` branch of the reference's
        `marching_cubes` (ash/grid.py:628-678) without its open3d packaging.
        tsdfs, weights: (num_embeddings, cells_per_grid[, 1])."""
        if self.grid_coords is None or self.lut_grid_nb2grid_idx is None:
            self.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
        _, grid_indices = self._blocks_in_spatial_order()
        vertices = backend.isosurface_extraction(
            tsdfs,
            weights,
            grid_indices,
            self.grid_coords,
            self.lut_grid_nb2grid_idx,
            self.cell_coords,
            self.lut_cell_nb2cell_idx,
            self.lut_cell_nb2grid_nb,
            self.grid_dim,
            iso_value,
            weight_thr,
        )
        return self.transform_cell_to_world(vertices)

    def surface_mesh(
        self, tsdfs: torch.Tensor, weights: torch.Tensor, iso_value: float = 0.0,
        weight_thr: float = 1.0,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Marching cubes over the active blocks: (triangles int32 (T, 3), world
        positions (V, 3)) -- the mesh branch of the reference's `marching_cubes`
        (ash/grid.py:680-711) without its open3d packaging.  A cell contributes
        when all eight of its corners exist and weigh at least `weight_thr`;
        triangle normals point towards larger `tsdfs`."""
        if self.grid_coords is None or self.lut_grid_nb2grid_idx is None:
            self.construct_grid_neighbor_lut_(radius=1, bidirectional=False)
        _, grid_indices = self._blocks_in_spatial_order()
        triangles, vertices = backend.marching_cubes(
            tsdfs,
            weights,
            grid_indices,
            self.grid_coords,
            self.lut_grid_nb2grid_idx,
            self.cell_coords,
            self.lut_cell_nb2cell_idx,
            self.lut_cell_nb2grid_nb,
            self.grid_dim,
            iso_value,
            weight_thr,
        )
        return triangles, self.transform_cell_to_world(vertices)

    def marching_cubes(
        self, tsdfs, weights, color_fn=None, normal_fn=None, iso_value: float = 0.0,
        weight_thr: float = 1.0, vertices_only: bool = False,
    ):
        """Surface extraction (ash/grid.py:628-711): a point cloud of the edge
        crossings (`vertices_only=True`) or a triangle mesh.  Returns the open3d
        geometry of the reference when open3d is importable, otherwise a dict of
        tensors with the same fields (positions, [triangles,] colors, normals);
        None when there are no points."""
        triangles = None
        if vertices_only:
            positions = self.isosurface_points(tsdfs, weights, iso_value, weight_thr)
        else:
            triangles, positions = self.surface_mesh(tsdfs, weights, iso_value, weight_thr)
        if len(positions) == 0:
            return None
        fields = {"positions": positions}
        if triangles is not None:
            fields["triangles"] = triangles
        if color_fn is not None:
            fields["colors"] = color_fn(positions)
        if normal_fn is not None:
            fields["normals"] = normal_fn(positions)
        try:
            import open3d as o3d
        except ImportError:
            return fields
        if triangles is None:
            geometry = o3d.t.geometry.PointCloud(positions.detach().cpu().numpy())
            attributes = geometry.point
        else:
            geometry = o3d.t.geometry.TriangleMesh(
                positions.detach().cpu().numpy(), triangles.detach().cpu().numpy()
            )
            attributes = geometry.vertex
        for name in ("colors", "normals"):
            if name in fields:
                attributes[name] = fields[name].detach().cpu().numpy()
        return geometry

    # ------------------------------------------------------ neighbour tables
    @torch.no_grad()
    def construct_cell_neighbor_lut(
        self, radius: int, bidirectional: bool
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Per-cell tables (ash/grid.py:525-564).  For cell p and window offset
        o_k: the neighbour lies in block offset floor((p + o_k) / G), reported
        as its row in the block-offset window, at cell (p + o_k) mod G.

        Returns (lut_cell_nb2grid_nb, lut_cell_nb2cell_idx), both int64 (M, K).
        """
        cell_offsets, _ = enumerate_neighbor_coord_offsets(
            self.in_dim, radius, bidirectional, self.device
        )
        block_radius = (radius + self.grid_dim - 1) // self.grid_dim
        _, block_offset2idx = enumerate_neighbor_coord_offsets(
            self.in_dim, block_radius, bidirectional, self.device
        )
        assert self.cell_coords is not None
        shifted = (
            self.cell_coords.view(-1, 1, self.in_dim) + cell_offsets.view(1, -1, self.in_dim)
        ).view(-1, self.in_dim)
        block_shift = torch.div(shifted, self.grid_dim, rounding_mode="floor").long()
        wrapped = torch.remainder(shifted, self.grid_dim)

        lut_cell_nb2grid_nb = block_offset2idx(block_shift).view(self.num_cells_per_grid, -1)
        lut_cell_nb2cell_idx = self._linearize_cell_coords(wrapped).view(
            self.num_cells_per_grid, -1
        )
        return lut_cell_nb2grid_nb, lut_cell_nb2cell_idx

    @torch.no_grad()
    def construct_grid_neighbor_lut(
        self, radius: int, bidirectional: bool
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Per-block tables over all `num_embeddings` rows (ash/grid.py:566-617):
        grid_coords int32 (B, 3) and lut_grid_nb2grid_idx int64 (B, K), both -1
        in rows of inactive blocks and for missing neighbours."""
        active_coords, active_indices = self.engine.items()
        nb_offsets, _ = enumerate_neighbor_coord_offsets(
            self.in_dim, radius, bidirectional, self.device
        )
        num_nbs = len(nb_offsets)

        grid_coords = torch.full(
            (self.num_embeddings, self.in_dim), -1, dtype=torch.int32, device=self.device
        )
        lut = torch.full(
            (self.num_embeddings, num_nbs), -1, dtype=torch.int64, device=self.device
        )
        if len(active_coords) == 0:
            return grid_coords, lut

        nb_coords = (
            active_coords.view(-1, 1, self.in_dim).int() + nb_offsets.view(1, -1, self.in_dim).int()
        ).view(-1, self.in_dim)
        nb_indices, nb_found = self.engine.find(nb_coords)
        nb_indices[~nb_found] = -1

        grid_coords[active_indices] = active_coords
        lut[active_indices] = nb_indices.view(-1, num_nbs)
        return grid_coords, lut

    @torch.no_grad()
    def construct_grid_neighbor_lut_(self, radius: int, bidirectional: bool) -> None:
        """Caches the per-block tables; callers rebuild them after activating or
        erasing blocks (they are not invalidated automatically, as in the
        reference, ash/grid.py:221-222)."""
        self.grid_coords, self.lut_grid_nb2grid_idx = self.construct_grid_neighbor_lut(
            radius, bidirectional
        )


class UnBoundedSparseDenseGrid(SparseDenseGrid):
    """Grid with a fixed metric cell size and no fixed extent
    (ash/grid.py:714-775): world = cell * cell_size."""

    def __init__(
        self,
        in_dim: int,
        num_embeddings: int,
        embedding_dim: int,
        grid_dim: int,
        cell_size: float = 0.01,
        device: Optional[Union[str, torch.device]] = torch.device("cpu"),
    ):
        super().__init__(in_dim, num_embeddings, embedding_dim, grid_dim, device)
        self.cell_size = cell_size
        self.transform_world_to_cell = lambda x: x / self.cell_size
        self.transform_cell_to_world = lambda x: x * self.cell_size
        self._remember_world_to_cell(lambda: (None, self.cell_size))
        self._cell_to_world_affine = lambda: (self.cell_size, None)
        self.bbox_min = None
        self.bbox_max = None

    @torch.no_grad()
    def compute_bbox_(self):
        """World-space box spanned by the active blocks."""
        active_coords, _ = self.engine.items()
        lo = active_coords.min(dim=0)[0]
        hi = active_coords.max(dim=0)[0] + 1
        self.bbox_min = self.transform_cell_to_world(lo * self.grid_dim)
        self.bbox_max = self.transform_cell_to_world(hi * self.grid_dim)

    @torch.no_grad()
    def get_bbox(self, force_recompute: bool = False):
        if self.bbox_min is None or self.bbox_max is None or force_recompute:
            self.compute_bbox_()
        return self.bbox_min, self.bbox_max


class BoundedSparseDenseGrid(SparseDenseGrid):
    """Grid covering a fixed box with sparse_grid_dim^3 potential blocks
    (ash/grid.py:778-863).  The cell size is chosen so that
    sparse_grid_dim * grid_dim cell *corners* span the box:
    cell_size = min((bbox_max - bbox_min) / (sparse_grid_dim * grid_dim - 1))."""

    def __init__(
        self,
        in_dim: int,
        num_embeddings: int,
        embedding_dim: int,
        grid_dim: int = 8,
        sparse_grid_dim: int = 128,
        bbox_min: torch.Tensor = None,
        bbox_max: torch.Tensor = None,
        device: Optional[Union[str, torch.device]] = None,
    ):
        assert in_dim == 3, "Only 3D is supported now"
        super().__init__(in_dim, num_embeddings, embedding_dim, grid_dim, device)
        self.sparse_grid_dim = sparse_grid_dim
        self.bbox_min = (
            bbox_min.to(self.device)
            if bbox_min is not None
            else -torch.ones(self.in_dim, device=self.device)
        )
        self.bbox_max = (
            bbox_max.to(self.device)
            if bbox_max is not None
            else torch.ones(self.in_dim, device=self.device)
        )
        extent = self.bbox_max - self.bbox_min
        self.cell_size = (extent / (sparse_grid_dim * grid_dim - 1)).min().item()
        self.transform_world_to_cell = lambda x: (x - self.bbox_min) / self.cell_size
        self.transform_cell_to_world = lambda x: x * self.cell_size + self.bbox_min
        self._remember_world_to_cell(lambda: (self.bbox_min, self.cell_size))
        self._cell_to_world_affine = lambda: (self.cell_size, self.bbox_min)

    def grids_in_bound(self, grid_coords: torch.Tensor) -> torch.Tensor:
        inside = ((grid_coords >= 0) & (grid_coords < self.sparse_grid_dim)).all(dim=-1)
        return grid_coords[inside]

    def _block_bounds(self) -> Tuple[int, int]:
        return 0, self.sparse_grid_dim - 1

    def dense_init_(self):
        """Activates every block of the box."""
        axis = torch.arange(self.sparse_grid_dim)
        all_blocks = (
            torch.stack(torch.meshgrid(*[axis] * self.in_dim, indexing="ij"))
            .reshape(self.in_dim, -1)
            .T.to(self.device)
        )
        self.engine.insert_keys(all_blocks)

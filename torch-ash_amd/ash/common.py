"""Loader and thin Python face of libash_hip.so.

The reference binds its native code with pybind11 (`import __ash`,
ash/common.py:4-15 and ash/src/pybind.cpp:8-38).  Here the native side is a
plain C-ABI shared library (include/ash_hip.h) loaded with ctypes; this module
rebuilds the exact surface the rest of the package expects from the extension
module: a `HashMap` class and the three `query_*` functions.

There is no CPU or PyTorch fallback: if the library is missing, or a tensor is
not on a HIP device, the calls raise.
"""
import ctypes
import itertools
import os
import threading
import warnings
from typing import Dict, Optional, Tuple

import torch

_LIB_NAME = "libash_hip.so"
_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")

_I64 = ctypes.c_int64
_PTR = ctypes.c_void_p


class DotDict(dict):
    """dict whose items are also attributes (ash/common.py:19-22)."""

    __getattr__ = dict.__getitem__
    __setattr__ = dict.__setitem__
    __delattr__ = dict.__delitem__


class _QueryArgs(ctypes.Structure):
    _fields_ = [
        ("embeddings", _PTR),
        ("offsets", _PTR),
        ("grid_indices", _PTR),
        ("cell_indices", _PTR),
        ("masks", _PTR),
        ("lut_grid_nb2grid_idx", _PTR),
        ("lut_cell_nb2cell_idx", _PTR),
        ("lut_cell_nb2grid_nb", _PTR),
        ("num_queries", _I64),
        ("num_embeddings", _I64),
        ("cells_per_grid", _I64),
        ("embedding_dim", _I64),
        ("interpolation", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
    ]


# name -> (restype, argtypes); mirrors include/ash_hip.h
_SIGNATURES = {
    "ash_last_error": (ctypes.c_char_p, []),
    "ash_abi_version": (ctypes.c_int, []),
    "ash_source_fingerprint": (ctypes.c_char_p, []),
    "ash_map_workspace_bytes": (
        ctypes.c_int,
        [ctypes.c_int, _I64, ctypes.POINTER(_I64), ctypes.POINTER(_I64)],
    ),
    "ash_map_create": (
        ctypes.c_int,
        [ctypes.c_int, _I64, _PTR, _PTR, _I64, ctypes.c_int, _PTR, ctypes.POINTER(_PTR)],
    ),
    "ash_map_attach_general": (ctypes.c_int, [_PTR, _PTR, _I64, _PTR]),
    "ash_map_destroy": (ctypes.c_int, [_PTR]),
    "ash_map_find": (ctypes.c_int, [_PTR, _PTR, _I64, _PTR, _PTR, _PTR]),
    "ash_grid_query": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, ctypes.c_int, _PTR, _PTR, _PTR, _PTR, _PTR],
    ),
    "ash_grid_forward": (
        ctypes.c_int,
        [_PTR, _PTR, _PTR, ctypes.c_float, ctypes.c_int, ctypes.POINTER(_QueryArgs), _PTR, _PTR, _PTR,
         _PTR, _PTR, _PTR],
    ),
    "ash_grid_activate": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         _PTR, _PTR, _PTR, _PTR],
    ),
    "ash_grid_activate_static": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         _PTR, _PTR, _PTR],
    ),
    "ash_grid_activate_positions": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, _PTR, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_int,
         ctypes.c_int, ctypes.c_int, _PTR, _PTR, _PTR],
    ),
    "ash_grid_integrate_depth_flagged": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, ctypes.c_int, ctypes.c_int, _PTR, _PTR, ctypes.c_float,
         ctypes.POINTER(ctypes.c_float), _PTR, _PTR, _PTR, _PTR, ctypes.c_int, ctypes.c_int,
         ctypes.c_float, ctypes.c_float, _PTR],
    ),
    "ash_grid_integrate_depth": (
        ctypes.c_int,
        [_PTR, _I64, ctypes.c_int, ctypes.c_int, _PTR, _PTR, _I64, ctypes.c_float,
         ctypes.POINTER(ctypes.c_float), _PTR, _PTR, _PTR, _PTR, ctypes.c_int, ctypes.c_int,
         ctypes.c_float, ctypes.c_float, _PTR],
    ),
    "ash_grid_integrate_depth_touched": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, ctypes.c_int, ctypes.c_int, _PTR, _PTR, ctypes.c_float,
         ctypes.POINTER(ctypes.c_float), _PTR, _PTR, _PTR, _PTR, ctypes.c_int, ctypes.c_int,
         ctypes.c_float, ctypes.c_float, _PTR],
    ),
    "ash_ray_find_near_far": (
        ctypes.c_int,
        [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, ctypes.c_float, ctypes.c_float, ctypes.c_float,
         ctypes.c_float, _PTR, _PTR, _PTR],
    ),
    "ash_ray_sample": (
        ctypes.c_int,
        [_PTR, _PTR, _PTR, _PTR, _PTR, _I64, _I64, ctypes.c_float, _PTR, _PTR, _PTR, _PTR, _PTR,
         _PTR],
    ),
    "ash_ray_sample_staged": (
        ctypes.c_int,
        [_PTR] * 5 + [_I64, _I64, ctypes.c_float, _PTR, _PTR, _I64, _PTR],
    ),
    "ash_ray_sample_compact": (ctypes.c_int, [_PTR] * 3 + [_I64, _I64] + [_PTR] * 4),
    "ash_map_insert_keys": (ctypes.c_int, [_PTR, _PTR, _I64, _PTR]),
    "ash_map_insert_needs_scratch": (ctypes.c_int, [ctypes.c_int, ctypes.POINTER(_I64)]),
    "ash_map_insert": (
        ctypes.c_int,
        [
            _PTR,
            _PTR,
            _I64,
            ctypes.c_int,
            ctypes.POINTER(_PTR),
            ctypes.POINTER(_PTR),
            ctypes.POINTER(_I64),
            _PTR,
            _PTR,
        ],
    ),
    "ash_map_bulk_workspace_bytes": (
        ctypes.c_int,
        [_PTR, _I64, ctypes.c_int, ctypes.POINTER(_I64), ctypes.POINTER(_I64),
         ctypes.POINTER(ctypes.c_int)],
    ),
    "ash_map_insert_bulk": (
        ctypes.c_int,
        [
            _PTR,
            _PTR,
            _I64,
            ctypes.c_int,
            ctypes.POINTER(_PTR),
            ctypes.POINTER(_PTR),
            ctypes.POINTER(_I64),
            _PTR,
            _I64,
            _PTR,
        ],
    ),
    "ash_map_items_in_index_order": (ctypes.c_int, [_PTR, ctypes.POINTER(ctypes.c_int)]),
    "ash_map_erase": (ctypes.c_int, [_PTR, _PTR, _I64, _PTR]),
    "ash_map_erase_bulk_query": (
        ctypes.c_int, [_PTR, _I64, ctypes.POINTER(_I64), ctypes.POINTER(ctypes.c_int)]
    ),
    "ash_map_erase_bulk": (ctypes.c_int, [_PTR, _PTR, _I64, _PTR, _I64, _PTR]),
    "ash_map_clear": (ctypes.c_int, [_PTR, _PTR]),
    "ash_map_status": (ctypes.c_int, [_PTR, ctypes.POINTER(_I64), _PTR]),
    "ash_map_counters": (ctypes.c_int, [_PTR, _PTR, ctypes.POINTER(_I64), _PTR]),
    "ash_map_counters_pending": (ctypes.c_int, [_PTR]),
    "ash_map_known_size": (ctypes.c_int, [_PTR, ctypes.POINTER(_I64)]),
    "ash_map_set_staging": (ctypes.c_int, [_PTR, _PTR]),
    "ash_map_insert_scratch_bytes": (
        ctypes.c_int,
        [_PTR, _I64, ctypes.c_int, ctypes.POINTER(_I64), ctypes.c_int, ctypes.POINTER(_I64)],
    ),
    "ash_map_insert_auto": (
        ctypes.c_int,
        [_PTR, _PTR, _I64, ctypes.c_int, ctypes.POINTER(_PTR), ctypes.POINTER(_PTR),
         ctypes.POINTER(_I64), _PTR, _I64, ctypes.c_int, _PTR, _PTR],
    ),
    "ash_map_erase_scratch_bytes": (
        ctypes.c_int, [_PTR, _I64, ctypes.c_int, ctypes.POINTER(_I64)]
    ),
    "ash_map_erase_auto": (ctypes.c_int, [_PTR, _PTR, _I64, _PTR, _I64, ctypes.c_int, _PTR]),
    "ash_map_upkeep": (ctypes.c_int, [_PTR, _I64, _PTR, _I64, _PTR, _PTR]),
    "ash_grid_collect_touched": (ctypes.c_int, [_PTR] * 6),
    "ash_map_size": (ctypes.c_int, [_PTR, ctypes.POINTER(_I64), _PTR]),
    "ash_map_items": (ctypes.c_int, [_PTR, _PTR, _PTR, _I64, _PTR]),
    "ash_map_load": (ctypes.c_int, [_PTR, _PTR, _PTR, _I64, _PTR, _PTR]),
    "ash_map_should_rebuild": (ctypes.c_int, [_PTR, _I64, _I64, _I64]),
    "ash_map_rebuild": (ctypes.c_int, [_PTR, _PTR, _PTR, _I64, _PTR]),
    "ash_scatter_rows": (ctypes.c_int, [_PTR, _PTR, _PTR, _I64, _I64, _PTR]),
    "ash_gather_rows": (
        ctypes.c_int,
        [ctypes.c_int, ctypes.POINTER(_PTR), ctypes.POINTER(_PTR), ctypes.POINTER(_I64),
         ctypes.POINTER(_I64), _PTR, _I64, _PTR],
    ),
    "ash_isosurface_workspace_ints": (ctypes.c_int64, [_I64, _I64]),
    "ash_isosurface_classify": (
        ctypes.c_int,
        [_PTR] * 7 + [_I64] * 3
        + [ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int32] + [_PTR] * 3,
    ),
    "ash_isosurface_points": (
        ctypes.c_int,
        [_PTR] * 7 + [_I64] * 3 + [ctypes.c_int, ctypes.c_float, ctypes.c_int32]
        + [_PTR] * 2 + [_I64] + [_PTR] * 2,
    ),
    "ash_convolution_forward": (
        ctypes.c_int,
        [_PTR] * 9 + [_I64] * 6 + [ctypes.c_int32, _PTR],
    ),
    "ash_convolution_forward_listed": (
        ctypes.c_int,
        [_PTR] * 9 + [_I64] * 6 + [ctypes.c_int32, _PTR, _PTR],
    ),
    "ash_marching_cubes_workspace_ints": (ctypes.c_int64, [_I64, _I64]),
    "ash_marching_cubes_classify": (
        ctypes.c_int,
        [_PTR] * 7 + [_I64] * 3
        + [ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int32] + [_PTR] * 4,
    ),
    "ash_marching_cubes_extract": (
        ctypes.c_int,
        [_PTR] * 7 + [_I64] * 3 + [ctypes.c_int, ctypes.c_float, ctypes.c_int32]
        + [_PTR] * 3 + [_I64] * 2 + [_PTR] * 3,
    ),
    "ash_query_forward": (ctypes.c_int, [ctypes.POINTER(_QueryArgs), _PTR, _PTR]),
    "ash_query_backward_forward": (
        ctypes.c_int,
        [ctypes.POINTER(_QueryArgs), _PTR, _PTR, _PTR, _PTR],
    ),
    "ash_query_backward_backward": (
        ctypes.c_int,
        [ctypes.POINTER(_QueryArgs), _PTR, _PTR, _PTR, _PTR, _PTR],
    ),
    "ash_query_backward_forward_accumulate": (
        ctypes.c_int,
        [ctypes.POINTER(_QueryArgs), _PTR, _PTR, _PTR, _PTR],
    ),
    "ash_query_backward_backward_accumulate": (
        ctypes.c_int,
        [ctypes.POINTER(_QueryArgs), _PTR, _PTR, _PTR, _PTR, _PTR],
    ),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_INTERPOLATION = {"linear": 0, "smooth_step": 1}

# Stamps of the tables' contents: a table takes a new one whenever its keys may
# have changed, and no two tables ever share one (a table made by `resize` may
# sit at the address of the one it replaces), so that what callers derive from
# the keys can be kept under the stamp alone.
_VERSIONS = itertools.count(1)

# Largest number of staged sample slots (rays x stride, 8 bytes each) for which
# ray_sample keeps the samples of its allocation pass; beyond it the march is
# run twice as in the reference.
RAY_STAGE_LIMIT = 1 << 30
# Staged slots per ray beyond max_samples_per_ray.
RAY_STAGE_EXTRA = 2
# Largest table whose touched rows ash_grid_collect_touched lists (the header's
# ASH_COLLECT_MAX_BLOCKS).
COLLECT_MAX_BLOCKS = 1 << 20
# Size of a second region that is attached before any key has asked for it
# (2^16 slots of 20 bytes).
GENERAL_JUST_IN_CASE_BYTES = 20 << 16
# Which inserts (and erases) take the streaming path of the library (batch split
# by bucket range, ranges handled in LDS) instead of the per-key kernel:
# "auto" = when the library says the batch is large enough relative to the
# table, "always" = whenever the path applies, "never".
BULK_INSERT = os.environ.get("ASH_BULK_INSERT", "auto")
BULK_ERASE = os.environ.get("ASH_BULK_ERASE", "auto")
_POLICY = {"auto": 0, "always": 1, "never": 2}   # the header's ASH_STREAMING_*
NEEDS_GENERAL = 2                                # the header's ASH_NEEDS_GENERAL
_DTYPE = {torch.float32: 0, torch.float64: 1}


def library_path() -> str:
    return os.environ.get("ASH_HIP_LIBRARY", os.path.join(_LIB_DIR, _LIB_NAME))


def load_library(path: Optional[str] = None) -> ctypes.CDLL:
    """dlopen the C-ABI library and attach the prototypes."""
    lib = ctypes.CDLL(path or library_path())
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    return lib


def _stream_of(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_hip(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what} must live on a HIP device, got {t.device}")


class _Backend:
    """Stands where the reference's `__ash` extension module stands."""

    def __init__(self, lib: ctypes.CDLL):
        self.lib = lib
        backend = self

        class HashMap(_HashMap):
            _backend = backend

        self.HashMap = HashMap

    # -- error plumbing -------------------------------------------------
    def check(self, status: int) -> None:
        if status != 0:
            msg = self.lib.ash_last_error()
            raise RuntimeError(msg.decode() if msg else "libash_hip call failed")

    # -- iso-surface points (ash/src/pybind.cpp:30) --------------------------
    def isosurface_extraction(
        self, sdfs, weights, grid_indices, grid_coords_table, lut_grid_nb2grid_idx,
        cell_coords_table, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, grid_dim, iso_value,
        weight_thr,
    ) -> torch.Tensor:
        """Zero crossings of `sdfs - iso_value` on the +x/+y/+z edges of the
        listed blocks' cells, (P, 3) float32 in cell units, in the order of the
        listing."""
        _require_hip(sdfs, "sdfs")
        dev = sdfs.device
        if sdfs.dtype not in _DTYPE:
            raise RuntimeError("sdfs must be float32 or float64")
        b, m = sdfs.shape[0], sdfs.shape[1]
        sdfs = sdfs.reshape(b, m).contiguous()
        weights = weights.to(dev, sdfs.dtype).reshape(b, m).contiguous()
        gi = grid_indices.reshape(-1).to(dev, torch.int64).contiguous()
        gc = grid_coords_table.to(dev, torch.int32).contiguous()
        cc = cell_coords_table.to(dev, torch.int32).contiguous()
        lut_g = lut_grid_nb2grid_idx.to(dev, torch.int64).contiguous()
        lut_c2c = lut_cell_nb2cell_idx.to(dev, torch.int64).contiguous()
        lut_c2g = lut_cell_nb2grid_nb.to(dev, torch.int64).contiguous()
        if gc.shape != (b, 3) or cc.shape != (m, 3) or lut_g.shape != (b, 8):
            raise RuntimeError("coordinate / neighbour tables do not match the grid")
        if lut_c2c.shape != (m, 8) or lut_c2g.shape != (m, 8):
            raise RuntimeError("cell neighbour tables must be (cells_per_grid, 8)")
        flags = torch.empty(b * m, dtype=torch.uint8, device=dev)
        workspace = torch.empty(
            self.lib.ash_isosurface_workspace_ints(gi.numel(), m), dtype=torch.int32, device=dev
        )
        with torch.cuda.device(dev):
            self.check(
                self.lib.ash_isosurface_classify(
                    sdfs.data_ptr(), weights.data_ptr(), gi.data_ptr(), lut_g.data_ptr(),
                    cc.data_ptr(), lut_c2c.data_ptr(), lut_c2g.data_ptr(), gi.numel(), b, m,
                    int(grid_dim), float(iso_value), float(weight_thr), _DTYPE[sdfs.dtype],
                    flags.data_ptr(), workspace.data_ptr(), _stream_of(dev),
                )
            )
            n_points = int(workspace[0].item())
            positions = torch.empty((n_points, 3), dtype=torch.float32, device=dev)
            if n_points:
                self.check(
                    self.lib.ash_isosurface_points(
                        sdfs.data_ptr(), gi.data_ptr(), gc.data_ptr(), lut_g.data_ptr(),
                        cc.data_ptr(), lut_c2c.data_ptr(), lut_c2g.data_ptr(), gi.numel(), b, m,
                        int(grid_dim), float(iso_value), _DTYPE[sdfs.dtype], flags.data_ptr(),
                        workspace.data_ptr(), n_points, positions.data_ptr(), _stream_of(dev),
                    )
                )
        return positions

    # -- marching cubes (ash/src/pybind.cpp:31) ------------------------------
    def marching_cubes(
        self, sdfs, weights, grid_indices, grid_coords_table, lut_grid_nb2grid_idx,
        cell_coords_table, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, grid_dim, iso_value,
        weight_thr,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Triangle mesh of the surface `sdfs == iso_value` over the listed
        blocks: (triangles int32 (T, 3), vertices float32 (V, 3) in cell units).
        A cell contributes when its eight corners exist and weigh at least
        `weight_thr`.  Vertices and triangles follow the order of `grid_indices`."""
        _require_hip(sdfs, "sdfs")
        dev = sdfs.device
        if sdfs.dtype not in _DTYPE:
            raise RuntimeError("sdfs must be float32 or float64")
        b, m = sdfs.shape[0], sdfs.shape[1]
        sdfs = sdfs.reshape(b, m).contiguous()
        weights = weights.to(dev, sdfs.dtype).reshape(b, m).contiguous()
        gi = grid_indices.reshape(-1).to(dev, torch.int64).contiguous()
        gc = grid_coords_table.to(dev, torch.int32).contiguous()
        cc = cell_coords_table.to(dev, torch.int32).contiguous()
        lut_g = lut_grid_nb2grid_idx.to(dev, torch.int64).contiguous()
        lut_c2c = lut_cell_nb2cell_idx.to(dev, torch.int64).contiguous()
        lut_c2g = lut_cell_nb2grid_nb.to(dev, torch.int64).contiguous()
        if gc.shape != (b, 3) or cc.shape != (m, 3) or lut_g.shape != (b, 8):
            raise RuntimeError("coordinate / neighbour tables do not match the grid")
        if lut_c2c.shape != (m, 8) or lut_c2g.shape != (m, 8):
            raise RuntimeError("cell neighbour tables must be (cells_per_grid, 8)")
        cases = torch.empty(b * m, dtype=torch.uint8, device=dev)
        slots = torch.empty(b * m, dtype=torch.int32, device=dev)
        counters = torch.empty(
            self.lib.ash_marching_cubes_workspace_ints(gi.numel(), m), dtype=torch.int32, device=dev
        )
        with torch.cuda.device(dev):
            self.check(
                self.lib.ash_marching_cubes_classify(
                    sdfs.data_ptr(), weights.data_ptr(), gi.data_ptr(), lut_g.data_ptr(),
                    cc.data_ptr(), lut_c2c.data_ptr(), lut_c2g.data_ptr(), gi.numel(), b, m,
                    int(grid_dim), float(iso_value), float(weight_thr), _DTYPE[sdfs.dtype],
                    cases.data_ptr(), slots.data_ptr(), counters.data_ptr(), _stream_of(dev),
                )
            )
            n_triangles, n_vertices = counters[:2].tolist()
            triangles = torch.empty((n_triangles, 3), dtype=torch.int32, device=dev)
            vertices = torch.empty((n_vertices, 3), dtype=torch.float32, device=dev)
            if n_vertices:
                self.check(
                    self.lib.ash_marching_cubes_extract(
                        sdfs.data_ptr(), gi.data_ptr(), gc.data_ptr(), lut_g.data_ptr(),
                        cc.data_ptr(), lut_c2c.data_ptr(), lut_c2g.data_ptr(), gi.numel(), b, m,
                        int(grid_dim), float(iso_value), _DTYPE[sdfs.dtype], cases.data_ptr(),
                        slots.data_ptr(), counters.data_ptr(), n_vertices, n_triangles,
                        vertices.data_ptr(), triangles.data_ptr() if n_triangles else None,
                        _stream_of(dev),
                    )
                )
        return triangles, vertices

    # -- sparse convolution (ash/src/pybind.cpp:33) -------------------------
    def convolution_forward(
        self, inputs, weights, masks, grid_indices, cell_indices, lut_grid_nb2grid_idx,
        lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, grid_dim,
    ) -> torch.Tensor:
        """outputs[row] = sum over window taps k of inputs[row of neighbour k] *
        weights[k], per channel; same shape as `inputs`, zero rows for blocks
        that are not listed."""
        _require_hip(inputs, "inputs")
        dev = inputs.device
        if inputs.dtype not in _DTYPE or inputs.dim() != 3 or not inputs.is_contiguous():
            raise RuntimeError("inputs must be contiguous float32/float64 (B, M, E)")
        b, m, e = inputs.shape
        weights = weights.to(dev, inputs.dtype).contiguous()
        lut_g = lut_grid_nb2grid_idx.to(dev, torch.int64).contiguous()
        lut_c2c = lut_cell_nb2cell_idx.to(dev, torch.int64).contiguous()
        lut_c2g = lut_cell_nb2grid_nb.to(dev, torch.int64).contiguous()
        k = lut_c2c.shape[1]
        if weights.shape != (k, e):
            raise RuntimeError(f"weights must be ({k}, {e}), got {tuple(weights.shape)}")
        if lut_c2c.shape != (m, k) or lut_c2g.shape != (m, k) or lut_g.shape[0] != b:
            raise RuntimeError("neighbour tables do not match the inputs")
        gi = grid_indices.reshape(-1).to(dev, torch.int64).contiguous()
        ci = cell_indices.reshape(-1).to(dev, torch.int64).contiguous()
        if ci.numel() != m:
            raise RuntimeError("cell_indices must list every cell of a block")
        masks = masks.to(dev, torch.bool).contiguous()
        if masks.numel() < gi.numel() * m:
            raise RuntimeError("masks must cover every listed cell")
        outputs = torch.empty_like(inputs)
        # one scratch byte per block: the library then clears only the rows of
        # the blocks that are not listed
        listed = torch.empty(b, dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            self.check(
                self.lib.ash_convolution_forward_listed(
                    inputs.data_ptr(), weights.data_ptr(), masks.data_ptr(), gi.data_ptr(),
                    ci.data_ptr(), lut_g.data_ptr(), lut_c2c.data_ptr(), lut_c2g.data_ptr(),
                    outputs.data_ptr(), gi.numel(), b, m, e, k, lut_g.shape[1],
                    _DTYPE[inputs.dtype], listed.data_ptr(), _stream_of(dev),
                )
            )
        return outputs

    # -- rays (ash/src/pybind.cpp:35-37) ----------------------------------
    @staticmethod
    def _rays(hashmap, ray_origins, ray_directions):
        dev = hashmap.device()
        o = ray_origins.to(dev, torch.float32).contiguous()
        d = ray_directions.to(dev, torch.float32).contiguous()
        if o.dim() != 2 or o.shape[1] != 3 or d.shape != o.shape:
            raise RuntimeError("ray origins and directions must both be (N, 3)")
        return dev, o, d

    def ray_find_near_far(
        self, hashmap, ray_origins, ray_directions, bbox_min, bbox_max, t_min, t_max, t_step,
        grid2cell_multiplier,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Per ray, the parameter range that contains active blocks (cell
        units); near = -1 where the ray meets none."""
        dev, o, d = self._rays(hashmap, ray_origins, ray_directions)
        lo = bbox_min.to(dev, torch.float32).contiguous()
        hi = bbox_max.to(dev, torch.float32).contiguous()
        n = o.shape[0]
        nears = torch.zeros(n, dtype=torch.float32, device=dev)
        fars = torch.zeros(n, dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            self.check(
                self.lib.ash_ray_find_near_far(
                    hashmap._handle, o.data_ptr(), d.data_ptr(), lo.data_ptr(), hi.data_ptr(), n,
                    float(t_min), float(t_max), float(t_step), float(grid2cell_multiplier),
                    nears.data_ptr(), fars.data_ptr(), _stream_of(dev),
                )
            )
        return nears, fars

    def ray_sample(
        self, hashmap, ray_origins, ray_directions, ray_nears, ray_fars, bbox_min, bbox_max,
        max_samples_per_ray, grid2cell_multiplier,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """(ray_indices int64[M], t_nears fp32[M], t_fars fp32[M], inclusive
        prefix sum of the per-ray sample counts int64[N])."""
        dev, o, d = self._rays(hashmap, ray_origins, ray_directions)
        n = o.shape[0]

        def per_ray(t):
            if not torch.is_tensor(t):
                return torch.full((n,), float(t), dtype=torch.float32, device=dev)
            return t.to(dev, torch.float32).expand(n).contiguous()

        nears, fars = per_ray(ray_nears), per_ray(ray_fars)
        counts = torch.zeros(n, dtype=torch.int64, device=dev)
        fixed = (hashmap._handle, o.data_ptr(), d.data_ptr(), nears.data_ptr(), fars.data_ptr(), n,
                 int(max_samples_per_ray), float(grid2cell_multiplier))
        # One march: the allocation pass keeps its samples, the assignment pass
        # copies them.  A ray takes at most max_samples steps of its own size
        # (+ rounding), so the staging stride below is never exceeded; the
        # two-march path of the reference remains for the case that it is.
        stride = max(1, int(max_samples_per_ray) + RAY_STAGE_EXTRA)
        staged = n * stride <= RAY_STAGE_LIMIT
        if staged:
            stage = torch.empty((n, stride, 2), dtype=torch.float32, device=dev)
            with torch.cuda.device(dev):
                self.check(
                    self.lib.ash_ray_sample_staged(*fixed, counts.data_ptr(), stage.data_ptr(),
                                                   stride, _stream_of(dev))
                )
        else:
            with torch.cuda.device(dev):
                self.check(
                    self.lib.ash_ray_sample(*fixed, counts.data_ptr(), None, None, None, None,
                                            _stream_of(dev))
                )
        prefix = torch.cumsum(counts, 0)
        if n:
            total, most = torch.stack([prefix[-1], counts.max()]).tolist()
        else:
            total, most = 0, 0
        ray_indices = torch.empty(total, dtype=torch.int64, device=dev)
        t_nears = torch.empty(total, dtype=torch.float32, device=dev)
        t_fars = torch.empty(total, dtype=torch.float32, device=dev)
        if total:
            with torch.cuda.device(dev):
                if staged and most <= stride:
                    self.check(
                        self.lib.ash_ray_sample_compact(
                            counts.data_ptr(), prefix.data_ptr(), stage.data_ptr(), stride, n,
                            ray_indices.data_ptr(), t_nears.data_ptr(), t_fars.data_ptr(),
                            _stream_of(dev),
                        )
                    )
                else:
                    self.check(
                        self.lib.ash_ray_sample(
                            *fixed, None, prefix.data_ptr(), ray_indices.data_ptr(),
                            t_nears.data_ptr(), t_fars.data_ptr(), _stream_of(dev),
                        )
                    )
        return ray_indices, t_nears, t_fars, prefix

    # -- depth integration (no pybind counterpart: the reference's demo does
    #    this with torch expressions, demo/rgbd_fusion.py:76-110,216-254) -----
    def integrate_depth(
        self,
        embeddings: torch.Tensor,
        grid_indices: torch.Tensor,
        grid_coords: torch.Tensor,
        grid_dim: int,
        cell_size: float,
        origin: Optional[torch.Tensor],
        intrinsic: torch.Tensor,
        extrinsic: torch.Tensor,
        depth: torch.Tensor,
        color: Optional[torch.Tensor],
        trunc: float,
        depth_max: float,
        counted_by=None,
        flagged_by=None,
    ) -> None:
        """In-place TSDF update of the cells of the listed blocks.  With
        `counted_by` (a map whose latest deferred activation made the listing)
        the number of listed blocks is read on the device; with `flagged_by` (a
        map whose latest `activate_positions` left flags) there is no listing
        and the kernel goes by the map's flags, which it takes down."""
        _require_hip(embeddings, "embeddings")
        dev = embeddings.device
        if embeddings.dtype != torch.float32 or not embeddings.is_contiguous():
            raise RuntimeError("embeddings must be contiguous float32")
        if embeddings.dim() != 3 or embeddings.shape[1] != grid_dim**3:
            raise RuntimeError("embeddings must be (num_embeddings, grid_dim^3, embedding_dim)")
        if flagged_by is not None:
            if flagged_by._device != dev or getattr(flagged_by, "_touched", None) is None:
                raise RuntimeError("no activation has flagged rows of this map on this device")
            if embeddings.shape[0] < flagged_by.capacity:
                raise RuntimeError("one embedding row per index of the map is needed")
        else:
            grid_indices = grid_indices.reshape(-1).to(dev, torch.int64).contiguous()
            grid_coords = grid_coords.reshape(-1, 3).to(dev, torch.int32).contiguous()
            if grid_coords.shape[0] != grid_indices.shape[0]:
                raise RuntimeError("one coordinate row per block index is needed")
        if counted_by is not None and grid_indices.shape[0] != counted_by.capacity:
            raise RuntimeError("a listing counted on the device has one row per block of the map")
        intrinsic = intrinsic.to(dev, torch.float32).contiguous()
        extrinsic = extrinsic.to(dev, torch.float32).contiguous()
        if intrinsic.shape != (3, 3) or extrinsic.shape != (4, 4):
            raise RuntimeError("intrinsic must be 3x3 and extrinsic 4x4")
        depth = depth.to(dev, torch.float32).contiguous()
        if depth.dim() != 2:
            raise RuntimeError("depth must be (H, W)")
        if color is not None:
            color = color.to(dev, torch.float32).contiguous()
            if color.shape != (*depth.shape, 3):
                raise RuntimeError("color must be (H, W, 3)")
        c_origin = None
        if origin is not None:
            c_origin = (ctypes.c_float * 3)(*[float(v) for v in origin.reshape(-1).tolist()])
        tail = (float(cell_size), c_origin, intrinsic.data_ptr(), extrinsic.data_ptr(),
                depth.data_ptr(), color.data_ptr() if color is not None else None,
                depth.shape[0], depth.shape[1], float(trunc), float(depth_max), _stream_of(dev))
        with torch.cuda.device(dev):
            if flagged_by is not None:
                self.check(
                    self.lib.ash_grid_integrate_depth_flagged(
                        flagged_by._handle, embeddings.data_ptr(), embeddings.shape[0],
                        int(grid_dim), embeddings.shape[2], flagged_by._touched.data_ptr(),
                        flagged_by._block_coords.data_ptr(), *tail,
                    )
                )
            elif counted_by is not None:
                self.check(
                    self.lib.ash_grid_integrate_depth_touched(
                        counted_by._handle, embeddings.data_ptr(), embeddings.shape[0],
                        int(grid_dim), embeddings.shape[2], grid_indices.data_ptr(),
                        grid_coords.data_ptr(), *tail,
                    )
                )
            else:
                self.check(
                    self.lib.ash_grid_integrate_depth(
                        embeddings.data_ptr(), embeddings.shape[0], int(grid_dim),
                        embeddings.shape[2], grid_indices.data_ptr(), grid_coords.data_ptr(),
                        grid_indices.shape[0], *tail,
                    )
                )

    # -- value rows by index (ash/hashmap.py:87-95,138-146) -------------------
    def gather_rows(self, tables: Dict[str, torch.Tensor], indices: Optional[torch.Tensor],
                    first: int = 0) -> Dict[str, torch.Tensor]:
        """{name: table[indices]} for value tables on a HIP device, four tables
        per launch; with indices None, {name: copy of table[:first]}.  Tables
        the kernel does not take (rows that are not a multiple of 4 bytes,
        non-contiguous storage) are indexed by torch."""
        out: Dict[str, torch.Tensor] = {}
        batch = []
        if indices is not None:
            indices = indices.reshape(-1)
        n = indices.shape[0] if indices is not None else int(first)
        for name, table in tables.items():
            row_bytes = (table.numel() // max(table.shape[0], 1)) * table.element_size()
            fits = (table.is_cuda and table.is_contiguous() and table.shape[0] > 0
                    and row_bytes % 4 == 0 and row_bytes > 0 and not table.requires_grad
                    and (indices is None
                         or (indices.device == table.device and indices.dtype == torch.int64)))
            if not fits:
                out[name] = table[indices] if indices is not None else table[:n].clone()
                continue
            out[name] = torch.empty((n,) + tuple(table.shape[1:]), dtype=table.dtype,
                                    device=table.device)
            batch.append((table, out[name], row_bytes))
        if indices is not None:
            indices = indices.contiguous()
        for start in range(0, len(batch), 4):
            part = batch[start:start + 4]
            if n == 0:
                break
            k = len(part)
            c_src = (_PTR * k)(*[t.data_ptr() for t, _, _ in part])
            c_dst = (_PTR * k)(*[d.data_ptr() for _, d, _ in part])
            c_rows = (_I64 * k)(*[rb for _, _, rb in part])
            c_count = (_I64 * k)(*[t.shape[0] for t, _, _ in part])
            dev = part[0][0].device
            with torch.cuda.device(dev):
                self.check(self.lib.ash_gather_rows(
                    k, c_src, c_dst, c_rows, c_count,
                    indices.data_ptr() if indices is not None else None, n, _stream_of(dev)))
        return {name: out[name] for name in tables}

    # -- trilinear queries (ash/src/pybind.cpp:25-29) ---------------------
    def _query_args(
        self,
        embeddings,
        offsets,
        grid_indices,
        cell_indices,
        masks,
        lut_grid_nb2grid_idx,
        lut_cell_nb2cell_idx,
        lut_cell_nb2grid_nb,
        interpolation,
    ):
        if interpolation not in _INTERPOLATION:
            raise RuntimeError(f"Unknown interpolation functor: {interpolation}")
        if embeddings.dtype not in _DTYPE:
            raise RuntimeError(f"embeddings must be float32 or float64, got {embeddings.dtype}")
        if embeddings.dim() != 3:
            raise RuntimeError("embeddings must be (num_embeddings, cells_per_grid, dim)")
        _require_hip(embeddings, "embeddings")
        dev = embeddings.device
        n = grid_indices.shape[0]

        def prep(t, dtype, shape, name):
            if t.device != dev:
                raise RuntimeError(f"{name} is on {t.device}, embeddings on {dev}")
            if t.dtype != dtype:
                raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")
            if tuple(t.shape) != shape and t.numel() != _numel(shape):
                raise RuntimeError(f"{name} has shape {tuple(t.shape)}, expected {shape}")
            return t.contiguous()

        b, m, e = embeddings.shape
        held = [
            prep(embeddings, embeddings.dtype, (b, m, e), "embeddings"),
            prep(offsets, torch.float32, (n, 3), "offsets"),
            prep(grid_indices, torch.int64, (n,), "grid_indices"),
            prep(cell_indices, torch.int64, (n,), "cell_indices"),
            prep(masks, torch.bool, (n,), "masks"),
            prep(lut_grid_nb2grid_idx, torch.int64, (b, 8), "lut_grid_nb2grid_idx"),
            prep(lut_cell_nb2cell_idx, torch.int64, (m, 8), "lut_cell_nb2cell_idx"),
            prep(lut_cell_nb2grid_nb, torch.int64, (m, 8), "lut_cell_nb2grid_nb"),
        ]
        args = _QueryArgs(
            *[t.data_ptr() for t in held],
            n,
            b,
            m,
            e,
            _INTERPOLATION[interpolation],
            _DTYPE[embeddings.dtype],
        )
        return args, held, dev

    def query_forward(
        self,
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
    ) -> torch.Tensor:
        args, held, dev = self._query_args(
            embeddings,
            offsets,
            grid_indices,
            cell_indices,
            masks,
            lut_grid_nb2grid_idx,
            lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb,
            interpolation,
        )
        out = torch.empty(
            (args.num_queries, args.embedding_dim), dtype=embeddings.dtype, device=dev
        )
        with torch.cuda.device(dev):
            self.check(
                self.lib.ash_query_forward(ctypes.byref(args), out.data_ptr(), _stream_of(dev))
            )
        return out

    def grid_forward(
        self,
        hashmap,
        x,
        embeddings,
        lut_grid_nb2grid_idx,
        lut_cell_nb2cell_idx,
        lut_cell_nb2grid_nb,
        grid_dim,
        interpolation,
        need_operands: bool = True,
        origin: Optional[torch.Tensor] = None,
        cell_size: float = 1.0,
    ):
        """`SparseDenseGrid.query` and `query_forward` in one kernel: positions x
        (float32 (N, 3); cell units = (x - origin) / cell_size, evaluated as
        torch does on the device) -> (features (N, E), masks (N,),
        grid_indices, cell_indices, offsets).  The last three are what a
        backward pass needs; with need_operands False they are not produced
        (None)."""
        if interpolation not in _INTERPOLATION:
            raise RuntimeError(f"Unknown interpolation functor: {interpolation}")
        if embeddings.dtype not in _DTYPE:
            raise RuntimeError(f"embeddings must be float32 or float64, got {embeddings.dtype}")
        if embeddings.dim() != 3 or not embeddings.is_contiguous():
            raise RuntimeError("embeddings must be contiguous (num_embeddings, cells_per_grid, dim)")
        _require_hip(embeddings, "embeddings")
        dev = embeddings.device
        if hashmap.device() != dev:
            raise RuntimeError(f"the map is on {hashmap.device()}, embeddings on {dev}")
        if x.dim() != 2 or x.shape[1] != 3 or x.dtype != torch.float32 or x.device != dev:
            raise RuntimeError("positions must be float32 (N, 3) on the device of the embeddings")
        x = x.contiguous()
        if origin is not None:
            if origin.device != dev or origin.dtype != torch.float32 or origin.numel() != 3:
                raise RuntimeError("origin must be three float32 on the device of the embeddings")
            origin = origin.contiguous()
        b, m, e = embeddings.shape
        n = x.shape[0]

        def table(t, shape, name):
            if t.device != dev or t.dtype != torch.int64 or tuple(t.shape) != shape:
                raise RuntimeError(f"{name} must be int64 {shape} on {dev}")
            return t.contiguous()

        held = [table(lut_grid_nb2grid_idx, (b, 8), "lut_grid_nb2grid_idx"),
                table(lut_cell_nb2cell_idx, (m, 8), "lut_cell_nb2cell_idx"),
                table(lut_cell_nb2grid_nb, (m, 8), "lut_cell_nb2grid_nb")]
        args = _QueryArgs(embeddings.data_ptr(), None, None, None, None,
                          *[t.data_ptr() for t in held], n, b, m, e,
                          _INTERPOLATION[interpolation], _DTYPE[embeddings.dtype])
        out = torch.empty((n, e), dtype=embeddings.dtype, device=dev)
        masks = torch.empty(n, dtype=torch.bool, device=dev)
        grid_indices = cell_indices = offsets = None
        if need_operands:
            grid_indices = torch.empty(n, dtype=torch.int64, device=dev)
            cell_indices = torch.empty(n, dtype=torch.int64, device=dev)
            offsets = torch.empty((n, 3), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            self.check(
                self.lib.ash_grid_forward(
                    hashmap._handle, x.data_ptr(),
                    origin.data_ptr() if origin is not None else None, float(cell_size),
                    int(grid_dim), ctypes.byref(args),
                    out.data_ptr(), masks.data_ptr(),
                    grid_indices.data_ptr() if need_operands else None,
                    cell_indices.data_ptr() if need_operands else None,
                    offsets.data_ptr() if need_operands else None, _stream_of(dev),
                )
            )
        return out, masks, grid_indices, cell_indices, offsets

    def query_backward_forward(
        self,
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
        need_embeddings: bool = True,
        need_offsets: bool = True,
        accumulate_into: Optional[torch.Tensor] = None,
    ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        """(grad_embeddings, grad_offsets); an output that is not needed is
        None and its work (for grad_embeddings: dense zero fill + atomics) is
        skipped.  With `accumulate_into` (a gradient of the embeddings' shape
        that already holds other contributions) the embedding gradient is added
        to that tensor, which is also what is returned."""
        args, held, dev = self._query_args(
            embeddings,
            offsets,
            grid_indices,
            cell_indices,
            masks,
            lut_grid_nb2grid_idx,
            lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb,
            interpolation,
        )
        z = _as_like(z, embeddings, (args.num_queries, args.embedding_dim), "z")
        entry = self.lib.ash_query_backward_forward
        if accumulate_into is not None:
            need_embeddings = True
            grad_embeddings = _accumulator(accumulate_into, held[0])
            entry = self.lib.ash_query_backward_forward_accumulate
        else:
            grad_embeddings = torch.empty_like(held[0]) if need_embeddings else None
        grad_offsets = (
            torch.empty((args.num_queries, 3), dtype=embeddings.dtype, device=dev)
            if need_offsets
            else None
        )
        with torch.cuda.device(dev):
            self.check(
                entry(
                    ctypes.byref(args),
                    z.data_ptr(),
                    grad_embeddings.data_ptr() if need_embeddings else None,
                    grad_offsets.data_ptr() if need_offsets else None,
                    _stream_of(dev),
                )
            )
        return grad_embeddings, grad_offsets

    def query_backward_backward(
        self,
        grad_grad_embeddings,
        grad_grad_offsets,
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
        need_z: bool = True,
        need_embeddings: bool = True,
        accumulate_into: Optional[torch.Tensor] = None,
    ) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], torch.Tensor]:
        """(grad_z, grad_embeddings, zero grad_offsets); outputs that are not
        needed are None and their work is skipped.  `accumulate_into` as for
        query_backward_forward."""
        args, held, dev = self._query_args(
            embeddings,
            offsets,
            grid_indices,
            cell_indices,
            masks,
            lut_grid_nb2grid_idx,
            lut_cell_nb2cell_idx,
            lut_cell_nb2grid_nb,
            interpolation,
        )
        n, e = args.num_queries, args.embedding_dim
        z = _as_like(z, embeddings, (n, e), "z")
        gg_off = _as_like(grad_grad_offsets, embeddings, (n, 3), "grad_grad_offsets")
        grad_z = torch.empty((n, e), dtype=embeddings.dtype, device=dev) if need_z else None
        entry = self.lib.ash_query_backward_backward
        if accumulate_into is not None:
            need_embeddings = True
            grad_embeddings = _accumulator(accumulate_into, held[0])
            entry = self.lib.ash_query_backward_backward_accumulate
        else:
            grad_embeddings = torch.empty_like(held[0]) if need_embeddings else None
        with torch.cuda.device(dev):
            self.check(
                entry(
                    ctypes.byref(args),
                    gg_off.data_ptr(),
                    z.data_ptr(),
                    grad_z.data_ptr() if need_z else None,
                    grad_embeddings.data_ptr() if need_embeddings else None,
                    _stream_of(dev),
                )
            )
        # the offsets second-order term is not produced (ash/src/grid.cu:417-418)
        grad_offsets = torch.zeros((n, 3), dtype=embeddings.dtype, device=dev)
        return grad_z, grad_embeddings, grad_offsets


_STAGING: Dict[int, torch.Tensor] = {}


def _status_staging() -> torch.Tensor:
    """Page-locked landing place for a copy of a map's counters that the caller
    waits for: one per host thread for all maps (such a copy is complete when
    the call returns, and short-lived scratch sets would otherwise each allocate
    their own)."""
    key = threading.get_ident()
    staging = _STAGING.get(key)
    if staging is None:
        staging = _STAGING[key] = torch.zeros(8, dtype=torch.int32, pin_memory=True)
    return staging


def _accumulator(t: torch.Tensor, embeddings: torch.Tensor) -> torch.Tensor:
    """Checks that `t` can take a gradient of `embeddings` in place."""
    if (
        t.shape != embeddings.shape
        or t.dtype != embeddings.dtype
        or t.device != embeddings.device
        or not t.is_contiguous()
    ):
        raise RuntimeError("accumulate_into must be a contiguous tensor like the embeddings")
    return t


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


def _as_like(t: torch.Tensor, ref: torch.Tensor, shape, name: str) -> torch.Tensor:
    if t.device != ref.device:
        raise RuntimeError(f"{name} is on {t.device}, embeddings on {ref.device}")
    if t.dtype != ref.dtype:
        raise RuntimeError(f"{name} must be {ref.dtype}, got {t.dtype}")
    if t.numel() != _numel(shape):
        raise RuntimeError(f"{name} has shape {tuple(t.shape)}, expected {shape}")
    return t.contiguous()


class _HashMap:
    """Same surface as the pybind class `HashMap` (ash/src/pybind.cpp:9-23).

    Owns the table workspace as torch tensors and a native handle.  `heap` is
    the caller's int32[capacity] buffer and is mutated in place by the kernels.
    Which insert path a batch takes, the upkeep of the table and what is known
    of its counters on the host are the library's business (ash_map_insert_auto,
    ash_map_counters); this class allocates what the calls ask for.
    """

    _backend: "_Backend" = None
    _COUNTERS = ("size", "dropped", "tombstones", "exotic_pending", "load_duplicates", "touched",
                 "general_live")

    def __init__(self, key_dim: int, capacity: int, heap: torch.Tensor, device):
        device = torch.device(device)
        if device.type != "cuda":
            # the reference has no CPU map either (ash/src/hashmap_cpu.cpp:8)
            raise RuntimeError("Not implemented: ash hash maps exist on HIP devices only")
        if heap.dtype != torch.int32 or heap.numel() != capacity or not heap.is_contiguous():
            raise RuntimeError("heap must be a contiguous int32 tensor of `capacity` elements")
        _require_hip(heap, "heap")
        lib = self._backend.lib
        self._lib = lib
        self._handle = None
        self._device = heap.device
        self.key_dim = int(key_dim)
        self.capacity = int(capacity)
        self._heap = heap
        table_bytes, general_bytes = _I64(0), _I64(0)
        self._check(
            lib.ash_map_workspace_bytes(
                self.key_dim, self.capacity, ctypes.byref(table_bytes), ctypes.byref(general_bytes)
            )
        )
        self._general_bytes = general_bytes.value
        self._table = torch.empty(table_bytes.value, dtype=torch.uint8, device=self._device)
        self._general = None
        self._landing = None   # page-locked int32[16] of this map's own, made on first use
        # counts the calls that may have changed the stored keys; lets callers
        # keep results derived from the key set (orderings, tables) while it stands
        self.version = next(_VERSIONS)
        handle = _PTR()
        with torch.cuda.device(self._device):
            self._check(
                lib.ash_map_create(
                    self.key_dim,
                    self.capacity,
                    heap.data_ptr(),
                    self._table.data_ptr(),
                    table_bytes.value,
                    self._device.index,
                    self._stream(),
                    ctypes.byref(handle),
                )
            )
        self._handle = handle

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            # (waits for a copy that is still on its way into `_landing`)
            self._lib.ash_map_destroy(handle)

    # -- helpers ---------------------------------------------------------
    def _check(self, status: int) -> None:
        self._backend.check(status)

    def _stream(self) -> int:
        return _stream_of(self._device)

    def _keys(self, keys: torch.Tensor) -> torch.Tensor:
        if keys.dim() != 2 or keys.shape[1] != self.key_dim:
            raise RuntimeError(f"keys must be (N, {self.key_dim}), got {tuple(keys.shape)}")
        if keys.device != self._device:
            raise RuntimeError(f"keys are on {keys.device}, the map on {self._device}")
        if keys.dtype != torch.int32:
            keys = keys.to(torch.int32)
        return keys.contiguous()

    def _scratch(self, nbytes: int) -> Optional[torch.Tensor]:
        return torch.empty(nbytes, dtype=torch.uint8, device=self._device) if nbytes else None

    def _attach_general(self, just_in_case: bool = False) -> None:
        """Hands the table its second region (keys that do not fit the packed
        code live there): sized for the capacity once such a key has shown up,
        or -- `just_in_case`, ahead of time by a path that cannot come back for
        it -- for a few thousand of them."""
        if self._general is not None:
            raise RuntimeError("internal error: unpackable keys pending with region attached")
        nbytes = min(self._general_bytes, GENERAL_JUST_IN_CASE_BYTES) if just_in_case \
            else self._general_bytes
        self._general = torch.empty(nbytes, dtype=torch.uint8, device=self._device)
        with torch.cuda.device(self._device):
            self._check(
                self._lib.ash_map_attach_general(
                    self._handle, self._general.data_ptr(), nbytes, self._stream()
                )
            )

    def _upkeep(self, incoming: int) -> None:
        """Before the entry points that insert without ash_map_insert_auto."""
        nbytes = _I64(0)
        self._check(self._lib.ash_map_insert_scratch_bytes(
            self._handle, 0, 0, None, _POLICY["never"], ctypes.byref(nbytes)))
        scratch = self._scratch(nbytes.value)
        with torch.cuda.device(self._device):
            self._check(self._lib.ash_map_upkeep(
                self._handle, incoming, scratch.data_ptr() if scratch is not None else None,
                nbytes.value, _status_staging().data_ptr(), self._stream()))

    # -- pybind surface --------------------------------------------------
    def device(self) -> torch.device:
        return self._device

    def counters(self) -> Dict[str, int]:
        """The table's counters as the handle knows them; copied from the
        device only when no earlier call has left them on the host."""
        out = (_I64 * 7)()
        with torch.cuda.device(self._device):
            self._check(self._lib.ash_map_counters(
                self._handle, _status_staging().data_ptr(), out, self._stream()))
        return dict(zip(self._COUNTERS, out))

    def status(self) -> Dict[str, int]:
        """The counters by a copy from the device, whatever the handle knows."""
        out = (_I64 * 5)()
        with torch.cuda.device(self._device):
            self._check(self._lib.ash_map_status(self._handle, out, self._stream()))
        fresh = dict(zip(self._COUNTERS[:5], out))
        fresh.update({k: v for k, v in self.counters().items() if k not in fresh})
        return fresh

    def status_after_insert(self) -> Dict[str, int]:
        """The counters after the latest insert: every insert reads them (or
        queues their read-back), which saves the caller a read-back of its own."""
        return self.counters()

    @property
    def counters_queued(self) -> bool:
        """Whether the latest insert returned with the read-back of the
        counters still queued behind it."""
        return bool(self._lib.ash_map_counters_pending(self._handle))

    def known_size(self) -> Optional[int]:
        """The size if it is known on the host (from the latest read-back, or
        zero after a clear), else None; never asks the device for it."""
        n = _I64(0)
        rc = self._lib.ash_map_known_size(self._handle, ctypes.byref(n))
        if rc < 0:
            self._check(1)
        return n.value if rc == 1 else None

    def size(self) -> int:
        return self.counters()["size"]

    def find(self, keys: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        keys = self._keys(keys)
        n = keys.shape[0]
        indices = torch.empty(n, dtype=torch.int64, device=self._device)
        masks = torch.empty(n, dtype=torch.bool, device=self._device)
        with torch.cuda.device(self._device):
            self._check(
                self._lib.ash_map_find(
                    self._handle, keys.data_ptr(), n, indices.data_ptr(), masks.data_ptr(),
                    self._stream(),
                )
            )
        return indices, masks

    def query_cells(
        self, x: torch.Tensor, grid_dim: int
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """Fused front end of `SparseDenseGrid.query`: positions in cell units ->
        (grid_indices, cell_indices, offsets, masks) in one kernel."""
        if x.dim() != 2 or x.shape[1] != 3 or x.dtype != torch.float32:
            raise RuntimeError("positions must be float32 (N, 3)")
        if x.device != self._device:
            raise RuntimeError(f"positions are on {x.device}, the map on {self._device}")
        x = x.contiguous()
        n = x.shape[0]
        grid_indices = torch.empty(n, dtype=torch.int64, device=self._device)
        cell_indices = torch.empty(n, dtype=torch.int64, device=self._device)
        offsets = torch.empty((n, 3), dtype=torch.float32, device=self._device)
        masks = torch.empty(n, dtype=torch.bool, device=self._device)
        with torch.cuda.device(self._device):
            self._check(
                self._lib.ash_grid_query(
                    self._handle, x.data_ptr(), n, int(grid_dim), grid_indices.data_ptr(),
                    cell_indices.data_ptr(), offsets.data_ptr(), masks.data_ptr(), self._stream(),
                )
            )
        return grid_indices, cell_indices, offsets, masks

    def _activation_buffers(self, cells: torch.Tensor) -> torch.Tensor:
        if self.key_dim != 3:
            raise RuntimeError("block activation needs 3-d keys")
        if cells.dim() != 2 or cells.shape[1] != 3 or cells.dtype != torch.float32:
            raise RuntimeError("positions must be float32 (N, 3)")
        if cells.device != self._device:
            raise RuntimeError(f"positions are on {cells.device}, the map on {self._device}")
        if getattr(self, "_touched", None) is None:
            self._touched = torch.zeros(self.capacity, dtype=torch.uint8, device=self._device)
            self._block_coords = torch.zeros(
                (self.capacity, 3), dtype=torch.int32, device=self._device
            )
        return cells.contiguous()

    def activate_blocks(
        self,
        cells: torch.Tensor,
        grid_dim: int,
        dilation: int,
        bidirectional: bool,
        bound_lo: int,
        bound_hi: int,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """Fused body of `SparseDenseGrid.spatial_init_`: inserts the blocks
        around the positions `cells` (fp32, cell units) and returns the touched
        blocks as (grid_coords int32[n,3], grid_indices int64[n])."""
        cells = self._activation_buffers(cells)
        self._upkeep(cells.shape[0])
        # the touched rows are listed on the device and their count travels with
        # the read-back that ends the activation (tables beyond the listing
        # kernel's limit take torch's nonzero and a second read-back)
        listing = self.capacity <= COLLECT_MAX_BLOCKS
        if listing:
            rows = torch.empty(self.capacity, dtype=torch.int64, device=self._device)
            coords = torch.empty((self.capacity, 3), dtype=torch.int32, device=self._device)
        for _ in range(2):
            with torch.cuda.device(self._device):
                # (positions in cell units: no origin, cell size 1)
                self._check(
                    self._lib.ash_grid_activate_positions(
                        self._handle, cells.data_ptr(), cells.shape[0], None, 1.0,
                        int(grid_dim), int(dilation), int(bool(bidirectional)), int(bound_lo),
                        int(bound_hi), self._touched.data_ptr(), self._block_coords.data_ptr(),
                        self._stream(),
                    )
                )
                if listing:
                    self._check(
                        self._lib.ash_grid_collect_touched(
                            self._handle, self._touched.data_ptr(), self._block_coords.data_ptr(),
                            rows.data_ptr(), coords.data_ptr(), self._stream(),
                        )
                    )
            self.version = next(_VERSIONS)
            counters = self.counters()
            if counters["exotic_pending"] == 0:
                break
            # blocks beyond the packed range: they need the second region
            self._attach_general()
        if listing:
            n = counters["touched"]
            return coords[:n], rows[:n]
        grid_indices = self._touched.nonzero().view(-1)
        grid_coords = self._block_coords[grid_indices]
        self._touched[grid_indices] = 0
        return grid_coords, grid_indices

    def activate_blocks_deferred(
        self,
        cells: torch.Tensor,
        grid_dim: int,
        dilation: int,
        bidirectional: bool,
        bound_lo: int,
        bound_hi: int,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        """activate_blocks without its read-back: the blocks are inserted and
        the touched ones listed on the device, and (grid_coords int32[capacity,3],
        grid_indices int64[capacity]) are returned whole -- how many of their
        rows the listing filled stays in the table's counters, where
        ash_grid_integrate_depth_touched reads it.  Nothing here waits for the
        device (every 64th call in a row looks at the counters for the table's
        upkeep), so the launches can be captured into a graph; keys refused for
        lack of capacity show in the counters at the next call that reads them
        (`counters`, `size`, any insert).  Both tensors are reused by the next
        deferred activation of this map."""
        if self.capacity > COLLECT_MAX_BLOCKS:
            raise RuntimeError("deferred activation lists at most 2^20 blocks")
        cells = self._activation_buffers(cells)
        n = cells.shape[0]
        if getattr(self, "_listing", None) is None:
            self._listing = (
                torch.empty((self.capacity, 3), dtype=torch.int32, device=self._device),
                torch.empty(self.capacity, dtype=torch.int64, device=self._device),
            )
        if self._general is None:
            # a key beyond the packed range would otherwise wait for a read-back
            # that this path does not make
            self._attach_general(just_in_case=True)
        self._upkeep(n)
        coords, rows = self._listing
        with torch.cuda.device(self._device):
            # (positions in cell units: no origin, cell size 1; no scratch)
            self._check(
                self._lib.ash_grid_activate_positions(
                    self._handle, cells.data_ptr(), n, None, 1.0, int(grid_dim), int(dilation),
                    int(bool(bidirectional)), int(bound_lo), int(bound_hi),
                    self._touched.data_ptr(), self._block_coords.data_ptr(), self._stream(),
                )
            )
            self._check(
                self._lib.ash_grid_collect_touched(
                    self._handle, self._touched.data_ptr(), self._block_coords.data_ptr(),
                    rows.data_ptr(), coords.data_ptr(), self._stream(),
                )
            )
        self.version = next(_VERSIONS)
        return coords, rows

    def activate_positions(
        self,
        positions: torch.Tensor,
        origin: Optional[torch.Tensor],
        cell_size: float,
        grid_dim: int,
        dilation: int,
        bidirectional: bool,
        bound_lo: int,
        bound_hi: int,
    ) -> None:
        """The activation of `activate_blocks` from world positions (cell units
        = (positions - origin) / cell_size), two launches and nothing else: the
        touched rows stay flagged in the map's own arrays for
        `integrate_depth(flagged_by=map)`, which takes the flags down again.
        Nothing waits for the device and nothing is allocated once the map's
        arrays exist, so the launches can be captured into a graph; keys
        refused for lack of capacity show in the counters at the next call that
        reads them."""
        positions = self._activation_buffers(positions)
        n = positions.shape[0]
        if self._general is None:
            # a key beyond the packed range would otherwise wait for a read-back
            # that this path does not make
            self._attach_general(just_in_case=True)
        self._upkeep(n)
        with torch.cuda.device(self._device):
            self._check(self._lib.ash_grid_activate_positions(
                self._handle, positions.data_ptr(), n,
                origin.data_ptr() if origin is not None else None, float(cell_size),
                int(grid_dim), int(dilation), int(bool(bidirectional)), int(bound_lo),
                int(bound_hi), self._touched.data_ptr(), self._block_coords.data_ptr(),
                self._stream()))
        self.version = next(_VERSIONS)

    def insert_keys(self, keys: torch.Tensor) -> None:
        self._insert(self._keys(keys), 0, None, None, None)

    def insert(
        self,
        keys: torch.Tensor,
        values: Dict[str, torch.Tensor],
        external_values: Dict[str, torch.Tensor],
    ) -> None:
        keys = self._keys(keys)
        n = keys.shape[0]
        names = list(values.keys())
        if not names:
            return self.insert_keys(keys)
        src, dst, row_bytes = [], [], []
        for name in names:
            v, ext = values[name], external_values[name]
            if v.shape[0] != n:
                raise RuntimeError(f"value '{name}' has {v.shape[0]} rows for {n} keys")
            if v.dtype != ext.dtype or v.shape[1:] != ext.shape[1:]:
                raise RuntimeError(f"value '{name}' does not match its destination buffer")
            if v.device != self._device or ext.device != self._device:
                raise RuntimeError(f"value '{name}' is not on {self._device}")
            if not ext.is_contiguous():
                raise RuntimeError(f"destination buffer '{name}' must be contiguous")
            if ext.shape[0] != self.capacity:
                raise RuntimeError(f"destination buffer '{name}' must have `capacity` rows")
            v = v.contiguous()
            src.append(v)
            dst.append(ext)
            row_bytes.append((v.numel() // max(n, 1)) * v.element_size() if n else 0)
        k = len(names)
        self._insert(keys, k, (_PTR * k)(*[t.data_ptr() for t in src]),
                     (_PTR * k)(*[t.data_ptr() for t in dst]), (_I64 * k)(*row_bytes), held=src)

    def _insert(self, keys, k, c_src, c_dst, c_rows, held=None) -> None:
        """One ash_map_insert_auto (a second one after the second region has
        been attached, the first time a key does not fit the packed code)."""
        n = keys.shape[0]
        if n == 0:
            return
        policy = _POLICY[BULK_INSERT]
        if self._landing is None and n >= (1 << 12):
            # a batch that may take the streaming path: the map gets a landing
            # place of its own for the read-back queued behind such an insert
            self._landing = torch.zeros(16, dtype=torch.int32, pin_memory=True)
            self._check(self._lib.ash_map_set_staging(self._handle, self._landing.data_ptr()))
        for _ in range(2):
            nbytes = _I64(0)
            self._check(self._lib.ash_map_insert_scratch_bytes(
                self._handle, n, k, c_rows, policy, ctypes.byref(nbytes)))
            scratch = self._scratch(nbytes.value)
            with torch.cuda.device(self._device):
                rc = self._lib.ash_map_insert_auto(
                    self._handle, keys.data_ptr(), n, k, c_src, c_dst, c_rows,
                    scratch.data_ptr() if scratch is not None else None, nbytes.value, policy,
                    _status_staging().data_ptr(), self._stream())
            self.version = next(_VERSIONS)
            if rc != NEEDS_GENERAL:
                return self._check(rc)
            self._attach_general()
        raise RuntimeError("internal error: unpackable keys pending with region attached")

    def erase(self, keys: torch.Tensor) -> None:
        keys = self._keys(keys)
        n = keys.shape[0]
        policy = _POLICY[BULK_ERASE]
        nbytes = _I64(0)
        self._check(self._lib.ash_map_erase_scratch_bytes(
            self._handle, n, policy, ctypes.byref(nbytes)))
        scratch = self._scratch(nbytes.value)
        self.last_erase_path = "per-key" if scratch is None else "streaming"
        self.version = next(_VERSIONS)
        with torch.cuda.device(self._device):
            self._check(self._lib.ash_map_erase_auto(
                self._handle, keys.data_ptr(), n,
                scratch.data_ptr() if scratch is not None else None, nbytes.value, policy,
                self._stream()))

    def clear(self) -> None:
        with torch.cuda.device(self._device):
            self._check(self._lib.ash_map_clear(self._handle, self._stream()))
        self.version = next(_VERSIONS)

    def items(self) -> Tuple[torch.Tensor, torch.Tensor]:
        n = self.size()
        keys = torch.empty((n, self.key_dim), dtype=torch.int32, device=self._device)
        indices = torch.empty(n, dtype=torch.int64, device=self._device)
        # whether entry i is listed under index i: the value rows of the listing
        # are then the first n rows of every value tensor (HashMap.items)
        dense = ctypes.c_int(0)
        self._check(self._lib.ash_map_items_in_index_order(self._handle, ctypes.byref(dense)))
        self.last_items_in_index_order = bool(dense.value)
        if n > 0:
            with torch.cuda.device(self._device):
                self._check(
                    self._lib.ash_map_items(
                        self._handle, keys.data_ptr(), indices.data_ptr(), n, self._stream()
                    )
                )
        return keys, indices

    def load_states(self, states: Dict[str, torch.Tensor]) -> None:
        keys = self._keys(states["active_keys"])
        indices = states["active_indices"].to(self._device, torch.int64).contiguous()
        heap = states["heap"].to(self._device, torch.int32).contiguous()
        n = keys.shape[0]
        if indices.numel() != n:
            raise RuntimeError("active_keys and active_indices differ in length")
        if heap.numel() != self.capacity:
            raise RuntimeError("heap length differs from the capacity")
        for _ in range(2):
            with torch.cuda.device(self._device):
                self._check(
                    self._lib.ash_map_load(
                        self._handle,
                        keys.data_ptr() if n else None,
                        indices.data_ptr() if n else None,
                        n,
                        heap.data_ptr(),
                        self._stream(),
                    )
                )
            self.version = next(_VERSIONS)
            counters = self.counters()
            if counters["exotic_pending"] == 0:
                break
            self._attach_general()
        refused = counters["load_duplicates"]
        if refused:
            # The reference prints "Error loading, should never reach here!"
            # (ash/src/hashmap_gpu.cuh:420-422) for a repeated key and goes on
            # with a heap counter that no longer matches the stored entries; an
            # index or heap entry outside 0 .. capacity-1 makes its later calls
            # write out of bounds.  Here such a state is refused: the map is
            # left empty.
            self.clear()
            raise RuntimeError(
                f"load_states: {refused} pairs were refused (duplicate keys, or indices / heap "
                "entries outside the capacity); nothing was loaded"
            )


class _MissingBackend:
    """Placeholder used when libash_hip.so cannot be loaded: every use raises."""

    def __init__(self, reason: str):
        self._reason = reason

    def __getattr__(self, name):
        raise RuntimeError(
            f"libash_hip.so is not available ({self._reason}); build it with "
            "`python torch-ash_amd/build.py`. There is no CPU or PyTorch fallback."
        )


_BACKEND = None


def _get_c_extension():
    """Counterpart of ash/common.py:4-15: returns the native backend object."""
    global _BACKEND
    if _BACKEND is None:
        try:
            _BACKEND = _Backend(load_library())
        except OSError as exc:
            warnings.warn(f"HIP extension {_LIB_NAME} could not be loaded: {exc}")
            _BACKEND = _MissingBackend(str(exc))
    return _BACKEND

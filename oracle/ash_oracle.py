"""Python face of the CPU oracle (oracle/ash_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  `OracleBackend` offers the same surface as the
native backend object of the package (a `HashMap` class plus the three
`query_*` functions, cf. ash/src/pybind.cpp:8-38) on CPU tensors, so a test can
run the package's Python layer against it or compare results op by op.
"""
import ctypes
import os
from typing import Dict, Tuple

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "libash_oracle.so")

_I64 = ctypes.c_int64
_PTR = ctypes.c_void_p
_INTERP = {"linear": 0, "smooth_step": 1}
_SUFFIX = {torch.float32: "f32", torch.float64: "f64"}


def load(build_if_missing: bool = True) -> ctypes.CDLL:
    if build_if_missing and not os.path.exists(LIB_PATH):
        import importlib.util

        spec = importlib.util.spec_from_file_location(
            "_ash_oracle_build", os.path.join(HERE, "build.py")
        )
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        mod.build(verbose=False)
    lib = ctypes.CDLL(LIB_PATH)
    lib.ash_oracle_map_create.restype = _PTR
    lib.ash_oracle_map_create.argtypes = [ctypes.c_int, _I64, _PTR]
    lib.ash_oracle_map_destroy.argtypes = [_PTR]
    lib.ash_oracle_map_find.argtypes = [_PTR, _PTR, _I64, _PTR, _PTR]
    lib.ash_oracle_map_insert_keys.argtypes = [_PTR, _PTR, _I64]
    lib.ash_oracle_map_insert.argtypes = [
        _PTR, _PTR, _I64, ctypes.c_int,
        ctypes.POINTER(_PTR), ctypes.POINTER(_PTR), ctypes.POINTER(_I64),
    ]
    lib.ash_oracle_map_erase.argtypes = [_PTR, _PTR, _I64]
    lib.ash_oracle_map_clear.argtypes = [_PTR]
    lib.ash_oracle_map_size.restype = _I64
    lib.ash_oracle_map_size.argtypes = [_PTR]
    lib.ash_oracle_map_dropped.restype = _I64
    lib.ash_oracle_map_dropped.argtypes = [_PTR]
    lib.ash_oracle_map_items.restype = _I64
    lib.ash_oracle_map_items.argtypes = [_PTR, _PTR, _PTR]
    lib.ash_oracle_map_load.restype = _I64
    lib.ash_oracle_map_load.argtypes = [_PTR, _PTR, _PTR, _I64, _PTR]
    for sfx in ("f32", "f64"):
        getattr(lib, f"ash_oracle_convolution_forward_{sfx}").argtypes = [_PTR] * 9 + [_I64] * 6
        iso = getattr(lib, f"ash_oracle_isosurface_{sfx}")
        iso.restype = _I64
        iso.argtypes = [_PTR] * 8 + [_I64, _I64, ctypes.c_int, ctypes.c_float, ctypes.c_float, _PTR]
        getattr(lib, f"ash_oracle_marching_cubes_{sfx}").argtypes = (
            [_PTR] * 8 + [_I64] * 3 + [ctypes.c_int, ctypes.c_float, ctypes.c_float] + [_PTR] * 6
        )
    lib.ash_oracle_ray_find_near_far.argtypes = (
        [_PTR] * 5 + [_I64, ctypes.c_float, ctypes.c_float, ctypes.c_float, _PTR, _PTR]
    )
    lib.ash_oracle_ray_sample.argtypes = (
        [_PTR] * 5 + [_I64, _I64, ctypes.c_float] + [_PTR] * 5
    )
    lib.ash_oracle_num_threads.restype = ctypes.c_int
    lib.ash_oracle_set_num_threads.argtypes = [ctypes.c_int]
    for sfx in ("f32", "f64"):
        getattr(lib, f"ash_oracle_query_forward_{sfx}").argtypes = (
            [_PTR] * 9 + [_I64, _I64, _I64, ctypes.c_int]
        )
        getattr(lib, f"ash_oracle_query_backward_forward_{sfx}").argtypes = (
            [_PTR] * 11 + [_I64, _I64, _I64, _I64, ctypes.c_int]
        )
        getattr(lib, f"ash_oracle_query_backward_backward_{sfx}").argtypes = (
            [_PTR] * 12 + [_I64, _I64, _I64, _I64, ctypes.c_int]
        )
    lib.ash_oracle_query_term_sums.argtypes = [_PTR] * 15 + [_I64] * 4 + [ctypes.c_int]
    return lib


_MC_TABLE = None


def _mc_table():
    """The 256 x 16 marching-cubes case table (rows of edge triples, -1 padded)
    with the reference's triangles: read from the fixture that
    tests/golden/make_mc_case_fixture.py derives from ash/src/mc_macros.h, not
    from the library's generator, so that the library's table is checked against
    an input it did not produce."""
    global _MC_TABLE
    if _MC_TABLE is None:
        import json

        path = os.path.join(HERE, os.pardir, "tests", "golden", "mc_case_boundaries.json")
        with open(path) as f:
            cases = json.load(f)
        table = []
        for case in range(256):
            flat = [e for tri in cases[str(case)]["set"] for e in tri]
            table.append(flat + [-1] * (16 - len(flat)))
        _MC_TABLE = table
    return _MC_TABLE


def _cpu(t: torch.Tensor, dtype=None) -> torch.Tensor:
    t = t.detach().to("cpu")
    if dtype is not None and t.dtype != dtype:
        t = t.to(dtype)
    return t.contiguous()


class OracleBackend:
    def __init__(self, threads: int = 0):
        self.lib = load()
        if threads > 0:
            self.lib.ash_oracle_set_num_threads(threads)
        outer = self

        class HashMap(_OracleHashMap):
            _oracle = outer

        self.HashMap = HashMap

    def num_threads(self) -> int:
        return self.lib.ash_oracle_num_threads()

    def set_num_threads(self, n: int) -> None:
        self.lib.ash_oracle_set_num_threads(n)

    # -- iso-surface points (ash/src/pybind.cpp:30) ---------------------------
    def isosurface_extraction(self, sdfs, weights, grid_indices, grid_coords_table,
                              lut_grid_nb2grid_idx, cell_coords_table, lut_cell_nb2cell_idx,
                              lut_cell_nb2grid_nb, grid_dim, iso_value, weight_thr):
        x = _cpu(sdfs)
        b, m = x.shape[0], x.shape[1]
        x = x.reshape(b, m).contiguous()
        held = [x, _cpu(weights, x.dtype).reshape(b, m).contiguous(),
                _cpu(grid_indices, torch.int64).view(-1), _cpu(grid_coords_table, torch.int32),
                _cpu(lut_grid_nb2grid_idx, torch.int64), _cpu(cell_coords_table, torch.int32),
                _cpu(lut_cell_nb2cell_idx, torch.int64), _cpu(lut_cell_nb2grid_nb, torch.int64)]
        fn = getattr(self.lib, f"ash_oracle_isosurface_{_SUFFIX[x.dtype]}")
        args = [t.data_ptr() for t in held] + [held[2].numel(), m, int(grid_dim),
                                               float(iso_value), float(weight_thr)]
        count = fn(*args, None)
        positions = torch.zeros((count, 3), dtype=torch.float32)
        if count:
            fn(*args, positions.data_ptr())
        return positions

    # -- marching cubes (ash/src/pybind.cpp:31) -------------------------------
    def marching_cubes(self, sdfs, weights, grid_indices, grid_coords_table,
                       lut_grid_nb2grid_idx, cell_coords_table, lut_cell_nb2cell_idx,
                       lut_cell_nb2grid_nb, grid_dim, iso_value, weight_thr):
        """(triangles int32 (T, 3), vertices float32 (V, 3)), cells in launch
        order, with the reference's case table (see _mc_table)."""
        x = _cpu(sdfs)
        b, m = x.shape[0], x.shape[1]
        x = x.reshape(b, m).contiguous()
        held = [x, _cpu(weights, x.dtype).reshape(b, m).contiguous(),
                _cpu(grid_indices, torch.int64).view(-1), _cpu(grid_coords_table, torch.int32),
                _cpu(lut_grid_nb2grid_idx, torch.int64), _cpu(cell_coords_table, torch.int32),
                _cpu(lut_cell_nb2cell_idx, torch.int64), _cpu(lut_cell_nb2grid_nb, torch.int64)]
        table = torch.tensor(_mc_table(), dtype=torch.int8).contiguous()
        case_ws = torch.empty(b * m, dtype=torch.int32)
        edge_ws = torch.empty(b * m * 3, dtype=torch.int32)
        counts = torch.zeros(2, dtype=torch.int64)
        fn = getattr(self.lib, f"ash_oracle_marching_cubes_{_SUFFIX[x.dtype]}")
        args = [t.data_ptr() for t in held] + [
            held[2].numel(), b, m, int(grid_dim), float(iso_value), float(weight_thr),
            table.data_ptr(), case_ws.data_ptr(), edge_ws.data_ptr(), counts.data_ptr()]
        fn(*args, None, None)
        vertices = torch.zeros((int(counts[0]), 3), dtype=torch.float32)
        triangles = torch.zeros((int(counts[1]), 3), dtype=torch.int32)
        if int(counts[0]):
            fn(*args, vertices.data_ptr(), triangles.data_ptr())
        return triangles, vertices

    # -- sparse convolution (ash/src/pybind.cpp:33) ---------------------------
    def convolution_forward(self, inputs, weights, masks, grid_indices, cell_indices,
                            lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
                            grid_dim):
        x = _cpu(inputs)
        b, m, e = x.shape
        w = _cpu(weights, x.dtype)
        held = [x, w, _cpu(masks, torch.bool).view(-1), _cpu(grid_indices, torch.int64).view(-1),
                _cpu(cell_indices, torch.int64).view(-1), _cpu(lut_grid_nb2grid_idx, torch.int64),
                _cpu(lut_cell_nb2cell_idx, torch.int64), _cpu(lut_cell_nb2grid_nb, torch.int64)]
        out = torch.empty_like(x)
        fn = getattr(self.lib, f"ash_oracle_convolution_forward_{_SUFFIX[x.dtype]}")
        fn(*[t.data_ptr() for t in held], out.data_ptr(), held[3].numel(), b, m, e,
           held[6].shape[1], held[5].shape[1])
        return out

    # -- rays (ash/src/pybind.cpp:35-37) --------------------------------------
    def ray_find_near_far(self, hashmap, ray_origins, ray_directions, bbox_min, bbox_max,
                          t_min, t_max, t_step, grid2cell_multiplier):
        o, d = _cpu(ray_origins, torch.float32), _cpu(ray_directions, torch.float32)
        lo, hi = _cpu(bbox_min, torch.float32), _cpu(bbox_max, torch.float32)
        n = o.shape[0]
        nears, fars = torch.zeros(n), torch.zeros(n)
        self.lib.ash_oracle_ray_find_near_far(
            hashmap._h, o.data_ptr(), d.data_ptr(), lo.data_ptr(), hi.data_ptr(), n,
            float(t_min), float(t_max), float(grid2cell_multiplier), nears.data_ptr(),
            fars.data_ptr())
        return nears, fars

    def ray_sample(self, hashmap, ray_origins, ray_directions, ray_nears, ray_fars,
                   bbox_min, bbox_max, max_samples_per_ray, grid2cell_multiplier):
        o, d = _cpu(ray_origins, torch.float32), _cpu(ray_directions, torch.float32)
        nears, fars = _cpu(ray_nears, torch.float32), _cpu(ray_fars, torch.float32)
        n = o.shape[0]
        counts = torch.zeros(n, dtype=torch.int64)
        args = (hashmap._h, o.data_ptr(), d.data_ptr(), nears.data_ptr(), fars.data_ptr(),
                n, int(max_samples_per_ray), float(grid2cell_multiplier))
        self.lib.ash_oracle_ray_sample(*args, counts.data_ptr(), None, None, None, None)
        prefix = torch.cumsum(counts, 0)
        total = int(prefix[-1]) if n else 0
        ray_indices = torch.zeros(total, dtype=torch.int64)
        t_nears, t_fars = torch.zeros(total), torch.zeros(total)
        self.lib.ash_oracle_ray_sample(*args, None, prefix.data_ptr(), ray_indices.data_ptr(),
                                       t_nears.data_ptr(), t_fars.data_ptr())
        return ray_indices, t_nears, t_fars, prefix

    # -- queries ------------------------------------------------------------
    @staticmethod
    def _tables(embeddings, offsets, grid_indices, cell_indices, masks, lut_g, lut_c2c, lut_c2g):
        emb = _cpu(embeddings)
        held = [
            emb,
            _cpu(offsets, torch.float32),
            _cpu(grid_indices, torch.int64).view(-1),
            _cpu(cell_indices, torch.int64).view(-1),
            _cpu(masks, torch.bool).view(-1),
            _cpu(lut_g, torch.int64),
            _cpu(lut_c2c, torch.int64),
            _cpu(lut_c2g, torch.int64),
        ]
        return held

    def query_forward(
        self, embeddings, offsets, grid_indices, cell_indices, masks,
        lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
        grid_dim, interpolation,
    ) -> torch.Tensor:
        if interpolation not in _INTERP:
            raise RuntimeError(f"Unknown interpolation functor: {interpolation}")
        held = self._tables(
            embeddings, offsets, grid_indices, cell_indices, masks,
            lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
        )
        emb = held[0]
        n = held[2].shape[0]
        _, m, e = emb.shape
        out = torch.empty((n, e), dtype=emb.dtype)
        fn = getattr(self.lib, f"ash_oracle_query_forward_{_SUFFIX[emb.dtype]}")
        fn(*[t.data_ptr() for t in held], out.data_ptr(), n, m, e, _INTERP[interpolation])
        return out

    def query_backward_forward(
        self, z, embeddings, offsets, grid_indices, cell_indices, masks,
        lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
        grid_dim, interpolation, need_embeddings=True, need_offsets=True, accumulate_into=None,
    ) -> Tuple[torch.Tensor, torch.Tensor]:
        if interpolation not in _INTERP:
            raise RuntimeError(f"Unknown interpolation functor: {interpolation}")
        held = self._tables(
            embeddings, offsets, grid_indices, cell_indices, masks,
            lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
        )
        emb = held[0]
        n = held[2].shape[0]
        b, m, e = emb.shape
        z = _cpu(z, emb.dtype)
        grad_emb = torch.empty_like(emb)
        grad_off = torch.empty((n, 3), dtype=emb.dtype)
        fn = getattr(self.lib, f"ash_oracle_query_backward_forward_{_SUFFIX[emb.dtype]}")
        fn(
            z.data_ptr(), *[t.data_ptr() for t in held], grad_emb.data_ptr(),
            grad_off.data_ptr(), n, b, m, e, _INTERP[interpolation],
        )
        if accumulate_into is not None:
            accumulate_into.add_(grad_emb.to(accumulate_into.device))
            grad_emb = accumulate_into
        return (grad_emb if need_embeddings else None), (grad_off if need_offsets else None)

    def query_backward_backward(
        self, grad_grad_embeddings, grad_grad_offsets, z, embeddings, offsets,
        grid_indices, cell_indices, masks, lut_grid_nb2grid_idx,
        lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, grid_dim, interpolation,
        need_z=True, need_embeddings=True, accumulate_into=None,
    ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        if interpolation not in _INTERP:
            raise RuntimeError(f"Unknown interpolation functor: {interpolation}")
        held = self._tables(
            embeddings, offsets, grid_indices, cell_indices, masks,
            lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
        )
        emb = held[0]
        n = held[2].shape[0]
        b, m, e = emb.shape
        z = _cpu(z, emb.dtype)
        gg_off = _cpu(grad_grad_offsets, emb.dtype)
        grad_z = torch.empty((n, e), dtype=emb.dtype)
        grad_emb = torch.empty_like(emb)
        fn = getattr(self.lib, f"ash_oracle_query_backward_backward_{_SUFFIX[emb.dtype]}")
        fn(
            gg_off.data_ptr(), z.data_ptr(), *[t.data_ptr() for t in held],
            grad_z.data_ptr(), grad_emb.data_ptr(), n, b, m, e, _INTERP[interpolation],
        )
        if accumulate_into is not None:
            accumulate_into.add_(grad_emb.to(accumulate_into.device))
            grad_emb = accumulate_into
        return (
            grad_z if need_z else None,
            grad_emb if need_embeddings else None,
            torch.zeros((n, 3), dtype=emb.dtype),
        )


    def query_term_sums(
        self, grad_grad_offsets, z, embeddings, offsets, grid_indices, cell_indices, masks,
        lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb, grid_dim, interpolation,
        dense: bool = True,
    ) -> Dict[str, torch.Tensor]:
        """Per output element of the three query functions, the sum of the
        absolute values of the terms that form it (float64): what a bound on
        the rounding of sums accumulated in another order scales with.  Keys:
        forward, bf_embeddings, bf_offsets, bb_z, bb_embeddings (the two dense
        ones only with `dense`)."""
        held = self._tables(
            embeddings, offsets, grid_indices, cell_indices, masks,
            lut_grid_nb2grid_idx, lut_cell_nb2cell_idx, lut_cell_nb2grid_nb,
        )
        held[0] = held[0].double()
        emb = held[0]
        n = held[2].shape[0]
        b, m, e = emb.shape
        z = _cpu(z, torch.float64)
        u = _cpu(grad_grad_offsets, torch.float64)
        out = {
            "forward": torch.empty((n, e), dtype=torch.float64),
            "bf_embeddings": torch.empty_like(emb) if dense else None,
            "bf_offsets": torch.empty((n, 3), dtype=torch.float64),
            "bb_z": torch.empty((n, e), dtype=torch.float64),
            "bb_embeddings": torch.empty_like(emb) if dense else None,
        }
        self.lib.ash_oracle_query_term_sums(
            u.data_ptr(), z.data_ptr(), *[t.data_ptr() for t in held],
            *[(t.data_ptr() if t is not None else None) for t in out.values()],
            n, b, m, e, _INTERP[interpolation],
        )
        return {k: v for k, v in out.items() if v is not None}


class _OracleHashMap:
    """Same methods as the package's native `HashMap` shim, on CPU tensors."""

    _oracle: OracleBackend = None

    def __init__(self, key_dim: int, capacity: int, heap: torch.Tensor, device=None):
        assert heap.device.type == "cpu" and heap.dtype == torch.int32
        assert heap.is_contiguous() and heap.numel() == capacity
        self._lib = self._oracle.lib
        self.key_dim = int(key_dim)
        self.capacity = int(capacity)
        self._heap = heap  # aliased, like ash/src/hashmap_impl.h:23
        self._h = self._lib.ash_oracle_map_create(self.key_dim, self.capacity, heap.data_ptr())
        if not self._h:
            raise RuntimeError("oracle map creation failed")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.ash_oracle_map_destroy(h)

    def _keys(self, keys: torch.Tensor) -> torch.Tensor:
        assert keys.dim() == 2 and keys.shape[1] == self.key_dim
        return _cpu(keys, torch.int32)

    def device(self):
        return torch.device("cpu")

    def size(self) -> int:
        return self._lib.ash_oracle_map_size(self._h)

    def status(self) -> Dict[str, int]:
        return {
            "size": self.size(),
            "dropped": self._lib.ash_oracle_map_dropped(self._h),
            "tombstones": 0,
            "exotic_pending": 0,
            "load_duplicates": getattr(self, "_load_dup", 0),
        }

    def find(self, keys) -> Tuple[torch.Tensor, torch.Tensor]:
        keys = self._keys(keys)
        n = keys.shape[0]
        indices = torch.empty(n, dtype=torch.int64)
        masks = torch.empty(n, dtype=torch.bool)
        self._lib.ash_oracle_map_find(self._h, keys.data_ptr(), n, indices.data_ptr(), masks.data_ptr())
        return indices, masks

    def insert_keys(self, keys) -> None:
        keys = self._keys(keys)
        self._lib.ash_oracle_map_insert_keys(self._h, keys.data_ptr(), keys.shape[0])

    def insert(self, keys, values: Dict[str, torch.Tensor], external_values: Dict[str, torch.Tensor]) -> None:
        keys = self._keys(keys)
        n = keys.shape[0]
        names = list(values.keys())
        if n == 0:
            return
        src = [_cpu(values[k]) for k in names]
        dst = [external_values[k] for k in names]
        for d in dst:
            assert d.device.type == "cpu" and d.is_contiguous()
        k = len(names)
        rows = (_I64 * k)(*[(s.numel() // n) * s.element_size() for s in src])
        c_src = (_PTR * k)(*[s.data_ptr() for s in src])
        c_dst = (_PTR * k)(*[d.data_ptr() for d in dst])
        self._lib.ash_oracle_map_insert(self._h, keys.data_ptr(), n, k, c_src, c_dst, rows)

    def erase(self, keys) -> None:
        keys = self._keys(keys)
        self._lib.ash_oracle_map_erase(self._h, keys.data_ptr(), keys.shape[0])

    def clear(self) -> None:
        self._lib.ash_oracle_map_clear(self._h)
        self._load_dup = 0

    def items(self) -> Tuple[torch.Tensor, torch.Tensor]:
        n = self.size()
        keys = torch.empty((n, self.key_dim), dtype=torch.int32)
        indices = torch.empty(n, dtype=torch.int64)
        got = self._lib.ash_oracle_map_items(self._h, keys.data_ptr(), indices.data_ptr())
        assert got == n
        return keys, indices

    def load_states(self, states: Dict[str, torch.Tensor]) -> None:
        keys = self._keys(states["active_keys"])
        indices = _cpu(states["active_indices"], torch.int64)
        heap = _cpu(states["heap"], torch.int32)
        assert heap.numel() == self.capacity
        self._load_dup = self._lib.ash_oracle_map_load(
            self._h, keys.data_ptr(), indices.data_ptr(), keys.shape[0], heap.data_ptr()
        )

"""The C-ABI library loads without a GPU, exports every function that
include/ash_hip.h declares, and rejects bad arguments on the host side before
touching a device."""
import ctypes
import os
import re

import numpy as np
import pytest

from ash import common

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ash_hip.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(ash_[a-z0-9_]+)\s*\(", text))


@pytest.fixture(scope="module")
def lib():
    return common.load_library()


def test_header_and_loader_agree():
    assert _declared_functions() == set(common.EXPORTED_SYMBOLS)


def test_every_declared_symbol_is_exported(lib):
    for name in sorted(_declared_functions()):
        assert getattr(lib, name) is not None, name


def test_abi_version(lib):
    assert lib.ash_abi_version() == 1


def test_library_is_built_from_the_sources_beside_it(lib):
    """The build compiles a fingerprint of the kernel sources into the library:
    a library left over from other sources (an edit without a rebuild) fails
    here instead of being measured or tested in their name."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(
        "ash_build", os.path.join(ROOT, "torch-ash_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    assert lib.ash_source_fingerprint().decode() == build.source_fingerprint()


def _error(lib):
    return lib.ash_last_error().decode()


def test_workspace_sizes(lib):
    table, general = ctypes.c_int64(0), ctypes.c_int64(0)
    assert lib.ash_map_workspace_bytes(3, 24_000_000, ctypes.byref(table), ctypes.byref(general)) == 0
    # 256-byte header + one 128-byte bucket per 6 entries of capacity, rounded up
    # to whole probe ranges of 512 buckets, + the key log (8 bytes per entry, in
    # 16-byte units, 256-byte aligned)
    assert table.value == 256 + 4_000_256 * 128 + 24_000_000 * 8
    assert general.value == 2**26 * 20  # next power of two >= 2 * capacity, 20 B per slot
    assert lib.ash_map_workspace_bytes(1, 1, ctypes.byref(table), ctypes.byref(general)) == 0
    assert table.value == 256 + 2 * 128 + 16
    for dim in (0, 5):
        assert lib.ash_map_workspace_bytes(dim, 10, ctypes.byref(table), ctypes.byref(general)) != 0
        assert "key_dim" in _error(lib)
    assert lib.ash_map_workspace_bytes(3, 0, ctypes.byref(table), ctypes.byref(general)) != 0
    assert "capacity" in _error(lib)


def _buckets(lib, capacity):
    table = ctypes.c_int64(0)
    assert lib.ash_map_workspace_bytes(3, capacity, ctypes.byref(table), None) == 0
    log_bytes = (capacity + 1) // 2 * 16
    return (table.value - log_bytes - 256) // 128   # (the log starts 256-byte aligned)


def _mix64(h):
    h = h ^ (h >> np.uint64(33))
    h = h * np.uint64(0xFF51AFD7ED558CCD)
    h = h ^ (h >> np.uint64(33))
    h = h * np.uint64(0xC4CEB9FE1A85EC53)
    return h ^ (h >> np.uint64(33))


@pytest.mark.parametrize("capacity", [3078, 6150, 122_886, 1_000_000])
def test_tables_of_several_probe_ranges_have_whole_ranges(lib, capacity):
    """A probe never leaves its aligned range of 512 buckets, and the hash
    spreads keys evenly over all buckets: a short last range (capacity 3078 used
    to get 513 buckets, i.e. a last range of one bucket) would overflow while
    the heap still has indices.  The bucket count is a multiple of 512 beyond
    one range, and with the table's hash no range of a map filled to capacity
    with distinct keys comes near its 5120 slots."""
    nb = _buckets(lib, capacity)
    assert nb >= (capacity + 5) // 6
    assert nb % 512 == 0
    worst = 0
    with np.errstate(over="ignore"):
        for seed in range(20):
            rng = np.random.default_rng(seed)
            codes = np.unique(rng.integers(0, 1 << 62, size=capacity + capacity // 8,
                                           dtype=np.uint64))[:capacity]
            rng.shuffle(codes)
            # bucket = high 32 bits of (high 32 bits of the mixed code x nb)
            bucket = ((_mix64(codes) >> np.uint64(32)) * np.uint64(nb)) >> np.uint64(32)
            per_range = np.bincount((bucket >> np.uint64(9)).astype(np.int64), minlength=nb // 512)
            worst = max(worst, int(per_range.max()))
    assert worst <= 3072 + 10 * 56 < 5120


def test_small_tables_are_one_probe_range(lib):
    for capacity in (1, 100, 3072):
        assert _buckets(lib, capacity) in (max(2, (capacity + 5) // 6), max(2, (capacity + 5) // 6) + 1)
        assert _buckets(lib, capacity) <= 513


def test_create_rejects_bad_buffers_without_a_device(lib):
    handle = ctypes.c_void_p()
    assert lib.ash_map_create(3, 100, None, None, 0, 0, None, ctypes.byref(handle)) != 0
    assert "null device buffer" in _error(lib)
    assert not handle.value
    assert lib.ash_map_create(3, 100, 4096, 4096 + 8, 1 << 20, 0, None, ctypes.byref(handle)) != 0
    assert "aligned" in _error(lib)
    assert lib.ash_map_create(3, 100, 4096, 4096, 64, 0, None, ctypes.byref(handle)) != 0
    assert "too small" in _error(lib)
    assert lib.ash_map_create(7, 100, 4096, 4096, 1 << 20, 0, None, ctypes.byref(handle)) != 0


def test_null_handles_are_errors(lib):
    out = (ctypes.c_int64 * 5)()
    assert lib.ash_map_find(None, None, 0, None, None, None) != 0
    assert "null map handle" in _error(lib)
    assert lib.ash_map_insert_keys(None, None, 0, None) != 0
    assert lib.ash_map_erase(None, None, 0, None) != 0
    assert lib.ash_map_clear(None, None) != 0
    assert lib.ash_map_status(None, out, None) != 0
    assert lib.ash_map_items(None, None, None, 0, None) != 0
    assert lib.ash_map_load(None, None, None, 0, None, None) != 0
    assert lib.ash_map_rebuild(None, None, None, 0, None) != 0
    assert lib.ash_map_should_rebuild(None, 1, 1, 1) == 0
    assert lib.ash_map_destroy(None) == 0


def test_insert_scratch_rule(lib):
    def needs(rows):
        arr = (ctypes.c_int64 * len(rows))(*rows)
        return lib.ash_map_insert_needs_scratch(len(rows), arr)

    assert needs([12, 4]) == 0            # configuration 2: fused into the insert kernel
    assert needs([64, 64, 64, 64]) == 0
    assert needs([68]) == 1               # wider than 16 dwords
    assert needs([3]) == 1                # not a multiple of 4 bytes
    assert needs([4, 4, 4, 4, 4]) == 1    # more than four value tensors


def test_query_argument_checks(lib):
    assert lib.ash_query_forward(None, None, None) != 0
    assert "null query arguments" in _error(lib)
    args = common._QueryArgs(1, 1, 1, 1, 1, 1, 1, 1, 4, 2, 8, 17, 0, 0)
    assert lib.ash_query_forward(ctypes.byref(args), 1, None) != 0
    assert "embedding_dim" in _error(lib)
    args = common._QueryArgs(1, 1, 1, 1, 1, 1, 1, 1, 4, 2, 8, 4, 7, 0)
    assert lib.ash_query_backward_forward(ctypes.byref(args), 1, 1, 1, None) != 0
    assert "Unknown interpolation" in _error(lib)
    args = common._QueryArgs(1, 1, 1, 1, 1, 1, 1, 1, 4, 2, 8, 4, 0, 3)
    assert lib.ash_query_backward_backward(ctypes.byref(args), 1, 1, 1, 1, None) != 0
    assert "dtype" in _error(lib)


def test_product_has_no_cpu_path():
    """A CPU device is refused like in the reference (ash/src/hashmap_cpu.cpp:8),
    CPU tensors are refused by the query functions, and a missing library makes
    every use raise instead of falling back."""
    import torch

    import ash

    with pytest.raises(RuntimeError, match="Not implemented"):
        ash.ASHEngine(3, 10, "cpu")
    emb = torch.zeros(2, 8, 4)
    with pytest.raises(RuntimeError, match="HIP device"):
        ash.core.backend.query_forward(
            emb, torch.zeros(1, 3), torch.zeros(1, dtype=torch.long), torch.zeros(1, dtype=torch.long),
            torch.ones(1, dtype=torch.bool), torch.zeros(2, 8, dtype=torch.long),
            torch.zeros(8, 8, dtype=torch.long), torch.zeros(8, 8, dtype=torch.long), 2, "linear",
        )
    missing = common._MissingBackend("simulated")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        missing.HashMap
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        missing.query_forward

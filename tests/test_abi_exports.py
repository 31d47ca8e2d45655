"""The C-ABI library loads without a GPU, exports every function that
include/ash_hip.h declares, and rejects bad arguments on the host side before
touching a device."""
import ctypes
import os
import re

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


def _error(lib):
    return lib.ash_last_error().decode()


def test_workspace_sizes(lib):
    table, general = ctypes.c_int64(0), ctypes.c_int64(0)
    assert lib.ash_map_workspace_bytes(3, 24_000_000, ctypes.byref(table), ctypes.byref(general)) == 0
    # 256-byte header + one 128-byte bucket per 6 entries of capacity + the key
    # log (8 bytes per entry, in 16-byte units, 256-byte aligned)
    assert table.value == 256 + 4_000_000 * 128 + 24_000_000 * 8
    assert general.value == 2**26 * 20  # next power of two >= 2 * capacity, 20 B per slot
    assert lib.ash_map_workspace_bytes(1, 1, ctypes.byref(table), ctypes.byref(general)) == 0
    assert table.value == 256 + 2 * 128 + 16
    for dim in (0, 5):
        assert lib.ash_map_workspace_bytes(dim, 10, ctypes.byref(table), ctypes.byref(general)) != 0
        assert "key_dim" in _error(lib)
    assert lib.ash_map_workspace_bytes(3, 0, ctypes.byref(table), ctypes.byref(general)) != 0
    assert "capacity" in _error(lib)


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

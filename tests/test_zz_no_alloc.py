"""The entry point that allocates nothing, ash_grid_activate_static, against
ash_grid_activate through the C ABI: two identical maps, the same positions,
two calls in a row (the second with fewer positions, so the array inside the
library still holds the first call's list); afterwards both maps hold the same
blocks, flag the same rows' coordinates and answer look-ups alike.  Integer
work: everything is compared bit for bit (row numbers through the coordinates
stored with them, since the order in which a parallel insert hands them out is
not fixed)."""
import ctypes

import pytest
import torch

from ash import common
from helpers import RawBlockMap

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
CAPACITY = 60_000
GRID_DIM = 8


def _Map(lib):
    return RawBlockMap(lib, CAPACITY, DEV)


def _positions(n, seed):
    g = torch.Generator().manual_seed(seed)
    # image-like ordering: neighbouring rows are neighbouring positions (cell units)
    return (((torch.rand(n, 3, generator=g).cumsum(0) * 0.3) % 260.0) - 50.0).to(DEV).contiguous()


def test_activate_static_equals_activate_on_two_calls_in_a_row():
    lib = common.load_library()
    plain, static = _Map(lib), _Map(lib)
    try:
        for n, seed, dilation, bidirectional in ((40_000, 410, 1, 1), (9_000, 411, 1, 0)):
            cells = _positions(n, seed)
            heads = torch.empty(64 + 3 * n, dtype=torch.int32, device=DEV)
            rc = lib.ash_grid_activate(plain.handle, cells.data_ptr(), n, GRID_DIM, dilation,
                                       bidirectional, -1000, 1000, plain.touched.data_ptr(),
                                       plain.coords.data_ptr(), heads.data_ptr(), plain.stream)
            assert rc == 0, lib.ash_last_error()
            rc = lib.ash_grid_activate_static(static.handle, cells.data_ptr(), n, GRID_DIM, dilation,
                                              bidirectional, -1000, 1000, static.touched.data_ptr(),
                                              static.coords.data_ptr(), static.stream)
            assert rc == 0, lib.ash_last_error()
            torch.cuda.synchronize()
            size = plain.size()
            assert static.size() == size and 100 < size < CAPACITY
            coords_p, rows_p = plain.touched_blocks()
            coords_s, rows_s = static.touched_blocks()
            assert coords_p.shape[0] > 100
            assert torch.equal(coords_s, coords_p)
            # each map answers a look-up of the touched blocks with the rows it flagged
            for m, rows in ((plain, rows_p), (static, rows_s)):
                idx, mask = m.find(coords_p.to(DEV))
                assert bool(mask.all()) and torch.equal(idx.cpu(), rows)
            # and both agree on arbitrary look-ups (hits and misses)
            probe = torch.cat([coords_p[::3] + 1, coords_p[::5]]).to(DEV).contiguous()
            _, mask_p = plain.find(probe)
            _, mask_s = static.find(probe)
            assert torch.equal(mask_p, mask_s)
    finally:
        plain.close()
        static.close()


def test_activate_static_refuses_more_than_its_array_holds():
    lib = common.load_library()
    m = _Map(lib)
    try:
        n = (1 << 20) + 1
        cells = torch.zeros((n, 3), dtype=torch.float32, device=DEV)
        rc = lib.ash_grid_activate_static(m.handle, cells.data_ptr(), n, GRID_DIM, 0, 0, -1000, 1000,
                                          m.touched.data_ptr(), m.coords.data_ptr(), m.stream)
        assert rc != 0
        assert "at most 1048576 positions" in lib.ash_last_error().decode()
        assert m.size() == 0
    finally:
        m.close()

"""Shared helpers of the test-suite: an independent pure-torch statement of
the trilinear query (used to pin the oracle through autograd), a dictionary
model of the hash map, and comparison utilities."""
import ctypes
from typing import Dict, Tuple

import numpy as np
import torch


def basis(x: torch.Tensor, interpolation: str) -> torch.Tensor:
    if interpolation == "linear":
        return x
    if interpolation == "smooth_step":
        return x * x * (3 - 2 * x)
    raise ValueError(interpolation)


def torch_query(
    embeddings, offsets, grid_indices, cell_indices, masks, lut_g, lut_c2c, lut_c2g, interpolation
) -> torch.Tensor:
    """y = sum_c w_c(offsets) * embeddings[g_c, cell_c], vectorised; zero rows
    for masked-out queries and for queries with a missing neighbour block.
    Differentiable in embeddings and offsets to any order."""
    dtype = embeddings.dtype
    nbn = lut_c2g[cell_indices]  # (N, 8)
    g = torch.gather(lut_g[grid_indices], 1, nbn)  # (N, 8)
    cell = lut_c2c[cell_indices]  # (N, 8)
    ok = masks & (g >= 0).all(dim=1)
    corner = torch.arange(8, device=offsets.device)
    bits = torch.stack([(corner >> d) & 1 for d in range(3)], dim=1).to(torch.bool)  # (8, 3)
    o = offsets.to(dtype)
    one_minus = (1.0 - offsets).to(dtype)  # computed in fp32 first, like the kernels
    x = torch.where(bits.unsqueeze(0), o.unsqueeze(1), one_minus.unsqueeze(1))  # (N, 8, 3)
    w = basis(x, interpolation).prod(dim=2)  # (N, 8)
    rows = embeddings[g.clamp(min=0), cell]  # (N, 8, E)
    y = (w.unsqueeze(-1) * rows).sum(dim=1)
    return y * ok.unsqueeze(-1).to(dtype)


def torch_term_sums(embeddings, offsets, grid_indices, cell_indices, masks, lut_g, lut_c2c,
                    lut_c2g, interpolation, z, u):
    """Sum of |terms| behind every output element of the three query functions
    (float64, vectorised): an independent statement of what the oracle's
    query_term_sums computes."""
    emb = embeddings.double()
    n = grid_indices.shape[0]
    nbn = lut_c2g[cell_indices]
    g = torch.gather(lut_g[grid_indices], 1, nbn)
    cell = lut_c2c[cell_indices]
    ok = (masks & (g >= 0).all(dim=1)).double()
    corner = torch.arange(8)
    bits = torch.stack([(corner >> d) & 1 for d in range(3)], dim=1).to(torch.bool)
    x = torch.where(bits.unsqueeze(0), offsets.unsqueeze(1), (1.0 - offsets).unsqueeze(1)).double()
    f = basis(x, interpolation)                                           # (N, 8, 3)
    df = (6 * x * (1 - x)).abs() if interpolation == "smooth_step" else torch.ones_like(x)
    w = f.prod(dim=2).abs() * ok.unsqueeze(1)                             # (N, 8)
    wg = torch.stack([df[..., d] * f[..., [e for e in range(3) if e != d]].prod(dim=2)
                      for d in range(3)], dim=2).abs() * ok.view(-1, 1, 1)  # (N, 8, 3)
    rows = emb[g.clamp(min=0), cell].abs()                                # (N, 8, E)
    za, ua = z.double().abs(), u.double().abs()
    du = (wg * ua.unsqueeze(1)).sum(dim=2)                                # (N, 8)
    flat = (g.clamp(min=0) * emb.shape[1] + cell).view(-1)
    dense = lambda t: torch.zeros(emb.shape[0] * emb.shape[1], emb.shape[2], dtype=torch.float64
                                  ).index_add_(0, flat, t.reshape(n * 8, -1)).view(emb.shape)
    return {
        "forward": (w.unsqueeze(-1) * rows).sum(dim=1),
        "bf_embeddings": dense(w.unsqueeze(-1) * za.unsqueeze(1)),
        "bf_offsets": (wg * (rows * za.unsqueeze(1)).sum(dim=2, keepdim=True)).sum(dim=1),
        "bb_z": (du.unsqueeze(-1) * rows).sum(dim=1),
        "bb_embeddings": dense(du.unsqueeze(-1) * za.unsqueeze(1)),
    }


# Bound on the difference between two evaluations of a sum of fp terms in
# different orders: K_ROUND * eps * sum|terms| on top of the stated tolerance.
# Each side rounds every term (a product of up to five factors: ~5 eps) and
# every partial sum (a tree or a chain of additions: ~log2(n)..n eps, sqrt(n)
# eps typically); 16 eps covers both sides for the sums met here (up to a few
# thousand terms per element) and is what the tests state.
K_ROUND = 16.0


def assert_close_sums(got, ref, term_sums, rtol, atol, eps, what=""):
    """|got - ref| <= rtol |ref| + atol + K_ROUND eps sum|terms|, elementwise."""
    got, ref = got.detach().cpu().double(), ref.detach().cpu().double()
    bound = rtol * ref.abs() + atol + K_ROUND * eps * term_sums
    excess = (got - ref).abs() - bound
    worst = int(excess.argmax())
    assert float(excess.view(-1)[worst]) <= 0, (
        f"{what}: |diff| {float((got - ref).abs().view(-1)[worst]):.3e} exceeds the bound "
        f"{float(bound.view(-1)[worst]):.3e} (sum|terms| {float(term_sums.reshape(-1)[worst]):.3e})")


class DictMap:
    """Sequential dictionary model of the map with the reference's heap
    protocol (ash/src/hashmap_gpu.cuh:211-232,316-336)."""

    def __init__(self, dim: int, capacity: int):
        self.dim, self.capacity = dim, capacity
        self.clear()

    def clear(self):
        self.table: Dict[Tuple[int, ...], int] = {}
        self.heap = list(range(self.capacity))
        self.counter = 0
        self.dropped = 0

    def insert(self, keys: np.ndarray):
        assigned = []
        for row in keys.tolist():
            k = tuple(row)
            if k in self.table:
                assigned.append(-1)
            elif self.counter >= self.capacity:
                self.dropped += 1
                assigned.append(-1)
            else:
                idx = self.heap[self.counter]
                self.counter += 1
                self.table[k] = idx
                assigned.append(idx)
        return assigned

    def find(self, keys: np.ndarray):
        idx = np.zeros(len(keys), dtype=np.int64)
        mask = np.zeros(len(keys), dtype=bool)
        for i, row in enumerate(keys.tolist()):
            v = self.table.get(tuple(row))
            if v is not None:
                idx[i], mask[i] = v, True
        return idx, mask

    def erase(self, keys: np.ndarray):
        for row in keys.tolist():
            v = self.table.pop(tuple(row), None)
            if v is not None:
                self.counter -= 1
                self.heap[self.counter] = v

    def size(self) -> int:
        return len(self.table)


def sort_rows(keys: torch.Tensor, *others: torch.Tensor):
    """Lexicographic sort of int rows; returns the sorted keys and the
    companions permuted the same way."""
    k = keys.detach().cpu().numpy()
    order = np.lexsort(k.T[::-1]) if k.shape[0] else np.zeros(0, dtype=np.int64)
    order_t = torch.from_numpy(order)
    return (keys.detach().cpu()[order_t],) + tuple(o.detach().cpu()[order_t] for o in others)


def assert_is_bijection_into(indices: torch.Tensor, capacity: int):
    idx = indices.detach().cpu()
    assert idx.numel() == idx.unique().numel(), "indices are not distinct"
    if idx.numel():
        assert int(idx.min()) >= 0 and int(idx.max()) < capacity


class RawBlockMap:
    """A 3-d map made through the C ABI, with the caller-owned arrays of a
    block activation (flags and block coordinates per row)."""

    def __init__(self, lib, capacity, device):
        self.lib, self.capacity, self.device = lib, capacity, device
        table, general = ctypes.c_int64(0), ctypes.c_int64(0)
        assert lib.ash_map_workspace_bytes(3, capacity, ctypes.byref(table), ctypes.byref(general)) == 0
        self.heap = torch.empty(capacity, dtype=torch.int32, device=device)
        self.table = torch.empty(table.value, dtype=torch.uint8, device=device)
        self.touched = torch.zeros(capacity, dtype=torch.uint8, device=device)
        self.coords = torch.zeros((capacity, 3), dtype=torch.int32, device=device)
        self.handle = ctypes.c_void_p()
        self.stream = torch.cuda.current_stream(device).cuda_stream
        rc = lib.ash_map_create(3, capacity, self.heap.data_ptr(), self.table.data_ptr(),
                                table.value, device.index or 0, self.stream,
                                ctypes.byref(self.handle))
        assert rc == 0, lib.ash_last_error()

    def close(self):
        self.lib.ash_map_destroy(self.handle)

    def touched_blocks(self):
        """(sorted coordinates of the flagged rows, their rows); clears the flags."""
        rows = self.touched.nonzero().view(-1)
        out = sort_rows(self.coords[rows], rows)
        self.touched.zero_()
        return out

    def size(self):
        n = ctypes.c_int64(-1)
        assert self.lib.ash_map_size(self.handle, ctypes.byref(n), self.stream) == 0
        return n.value

    def find(self, keys):
        n = keys.shape[0]
        idx = torch.empty(n, dtype=torch.int64, device=self.device)
        mask = torch.empty(n, dtype=torch.bool, device=self.device)
        rc = self.lib.ash_map_find(self.handle, keys.data_ptr(), n, idx.data_ptr(), mask.data_ptr(),
                                   self.stream)
        assert rc == 0, self.lib.ash_last_error()
        return idx, mask

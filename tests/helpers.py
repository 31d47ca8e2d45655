"""Shared helpers of the test-suite: an independent pure-torch statement of
the trilinear query (used to pin the oracle through autograd), a dictionary
model of the hash map, and comparison utilities."""
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

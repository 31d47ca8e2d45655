"""Neighbour offset enumeration shared by cell and block tables
(ash/grid_nns.py:5-47)."""
from typing import Callable, Tuple

import torch


def enumerate_neighbor_coord_offsets(
    dim: int, radius: int, bidirectional: bool, device: torch.device
) -> Tuple[torch.Tensor, Callable[[torch.Tensor], torch.Tensor]]:
    """Offsets of a (radius+1)^dim window (or (2*radius+1)^dim when
    bidirectional) and the inverse map offset -> row.

    Row k holds the offset whose first component varies fastest:
    o_d = (k // W**d) % W - pad, with W the window width and pad = radius for a
    bidirectional window, else 0.  For dim=3, radius=1, one-sided this is the
    bit pattern of k (x = bit 0, y = bit 1, z = bit 2).

    Returns (offsets int64[W**dim, dim], offset2idx) where offset2idx maps an
    (N, dim) tensor of offsets back to rows.
    """
    width = 2 * radius + 1 if bidirectional else radius + 1
    pad = radius if bidirectional else 0
    rows = torch.arange(width**dim, device=device)
    columns = [(torch.div(rows, width**d, rounding_mode="floor") % width) - pad for d in range(dim)]
    offsets = torch.stack(columns, dim=1).contiguous()

    def offset2idx(offset: torch.Tensor) -> torch.Tensor:
        assert offset.dim() == 2
        idx = torch.zeros_like(offset[:, 0])
        for d in reversed(range(dim)):
            idx = idx * width + (offset[:, d] + pad)
        return idx

    return offsets, offset2idx

"""HashEmbedding: one trainable row per inserted key.

Constructor arguments, attribute names (`embedding`, `engine`), `spatial_init_`
and the forward contract follow ash/embedding.py:9-38 of the reference: rows
of the keys that were inserted, zeros for all others.
"""
from typing import Union

import torch
import torch.nn as nn

from .core import ASHEngine, ASHModule


class HashEmbedding(ASHModule):
    """A table of `num_embeddings` rows of `embedding_dim` values addressed by
    integer keys of `in_dim` components.

    The key table has a fixed capacity: growing it would renumber nothing, but
    the parameter would have to change shape under the optimiser, so there is
    no `resize` here.
    """

    def __init__(
        self,
        in_dim: int,
        num_embeddings: int,
        embedding_dim: int,
        device: Union[str, torch.device] = "cpu",
    ):
        super().__init__()
        self.in_dim = int(in_dim)
        self.num_embeddings = int(num_embeddings)
        self.embedding_dim = int(embedding_dim)
        rows = torch.empty(self.num_embeddings, self.embedding_dim, device=device)
        self.embedding = nn.Parameter(rows)
        self.reset_parameters()
        self.engine = ASHEngine(self.in_dim, self.num_embeddings, device)

    def reset_parameters(self) -> None:
        """Standard normal rows (the draw `torch.randn` of that shape makes)."""
        with torch.no_grad():
            self.embedding.normal_()

    def extra_repr(self) -> str:
        return (
            f"in_dim={self.in_dim}, num_embeddings={self.num_embeddings}, "
            f"embedding_dim={self.embedding_dim}"
        )

    def spatial_init_(self, keys: torch.Tensor) -> None:
        """Gives every distinct key of `keys` (N, in_dim) a row."""
        self.engine.insert_keys(keys)

    def size(self) -> int:
        """Number of keys that own a row."""
        return self.engine.size()

    def forward(self, keys: torch.Tensor) -> torch.Tensor:
        """(N, embedding_dim): the row of every key that owns one, zeros for the
        rest.  Misses read row 0 (the look-up answers index 0 for them) and are
        then multiplied by their mask, so no gradient reaches that row through
        them."""
        indices, found = self.engine.find(keys)
        gate = found.unsqueeze(-1)
        return gate * self.embedding[indices]

"""HashEmbedding: one trainable row per inserted key (ash/embedding.py:9-38)."""
from typing import Union

import torch
import torch.nn as nn

from .core import ASHEngine, ASHModule


class HashEmbedding(ASHModule):
    """`num_embeddings` rows of width `embedding_dim`, addressed by int keys.
    The table cannot be resized, so the parameter keeps its shape for the
    optimiser."""

    def __init__(
        self,
        in_dim: int,
        num_embeddings: int,
        embedding_dim: int,
        device: Union[str, torch.device] = "cpu",
    ):
        super().__init__()
        self.embedding = nn.Parameter(torch.randn(num_embeddings, embedding_dim, device=device))
        self.engine = ASHEngine(in_dim, num_embeddings, device)

    def spatial_init_(self, keys: torch.Tensor) -> None:
        self.engine.insert_keys(keys)

    def forward(self, keys: torch.Tensor) -> torch.Tensor:
        """Rows of the inserted keys; zeros for keys that were never inserted."""
        indices, masks = self.engine.find(keys)
        return self.embedding[indices] * masks.unsqueeze(-1)

"""ash: sparse spatial hashing and sparse-dense grids on AMD MI355X (gfx950).

Drop-in for the hash map and trilinear-query parts of torch-ash: same module
and function names as the reference package (ash/__init__.py:1-14), backed by
libash_hip.so.
"""
from .common import DotDict
from .core import ASHEngine, ASHModule
from .embedding import HashEmbedding
from . import fusion
from .grid import BoundedSparseDenseGrid, SparseDenseGrid, UnBoundedSparseDenseGrid
from .grid_nns import enumerate_neighbor_coord_offsets
from .grid_query import SparseDenseGridQuery, SparseDenseGridQueryBackward, dense_grad
from .hashmap import HashMap, HashSet

__all__ = [
    "ASHEngine",
    "ASHModule",
    "BoundedSparseDenseGrid",
    "DotDict",
    "HashEmbedding",
    "HashMap",
    "HashSet",
    "SparseDenseGrid",
    "SparseDenseGridQuery",
    "SparseDenseGridQueryBackward",
    "UnBoundedSparseDenseGrid",
    "dense_grad",
    "enumerate_neighbor_coord_offsets",
    "fusion",
]

"""HashMap and HashSet: an ASHEngine plus (for the map) value tensors it owns.

Same constructor arguments, method names, return orders and buffer names as
the reference wrappers (ash/hashmap.py:7-178).
"""
from typing import Dict, List, Tuple, Union

import torch

from .core import ASHEngine, ASHModule

ValueSpec = Union[int, List[int], Dict[str, int]]
Values = Union[torch.Tensor, List[torch.Tensor], Dict[str, torch.Tensor]]


def _value_names(value_dims: ValueSpec) -> Dict[str, int]:
    """Buffer name -> row width for the three ways of declaring values
    (ash/hashmap.py:23-36): a single width is called "default", a list
    "default_<i>", a dict keeps its own names."""
    if isinstance(value_dims, int):
        return {"default": value_dims}
    if isinstance(value_dims, list):
        return {f"default_{i}": d for i, d in enumerate(value_dims)}
    if isinstance(value_dims, dict):
        return dict(value_dims)
    raise ValueError("value_dims must be int, list or dict")


class HashMap(ASHModule):
    """Hash map whose values live in float tensors registered as buffers under
    their value names, one row per index."""

    def __init__(
        self,
        key_dim: int,
        value_dims: ValueSpec,
        capacity: int,
        device: Union[str, torch.device] = torch.device("cpu"),
    ):
        super().__init__()
        self.engine = ASHEngine(key_dim, capacity, device)
        self.value_dims = value_dims
        self.values = {
            name: torch.zeros(capacity, width, device=device)
            for name, width in _value_names(value_dims).items()
        }
        for name, store in self.values.items():
            self.register_buffer(name, store)

    # -- value plumbing ----------------------------------------------------
    def _to_named(self, values: Values) -> Dict[str, torch.Tensor]:
        if isinstance(values, torch.Tensor):
            assert isinstance(self.value_dims, int)
            return {"default": values}
        if isinstance(values, list):
            assert isinstance(self.value_dims, list)
            return {f"default_{i}": v for i, v in enumerate(values)}
        if isinstance(values, dict):
            assert isinstance(self.value_dims, dict)
            return values
        raise ValueError("values must be Tensor, list, or dict")

    def reinterpret_value_dict(self, values: Dict[str, torch.Tensor]) -> Values:
        """Back from named values to the shape the map was declared with."""
        if isinstance(self.value_dims, int):
            return values["default"]
        if isinstance(self.value_dims, list):
            return [values[f"default_{i}"] for i in range(len(self.value_dims))]
        if isinstance(self.value_dims, dict):
            return values
        raise ValueError("values must be Tensor, list, or dict")

    def _gather(self, indices: torch.Tensor) -> Values:
        return self.reinterpret_value_dict(
            {name: store[indices] for name, store in self.values.items()}
        )

    # -- map operations ------------------------------------------------------
    def insert(self, keys: torch.Tensor, values: Values) -> None:
        self.engine.insert(keys, self._to_named(values), self.values)

    def find(
        self, keys: torch.Tensor, return_indices: bool = True, return_values: bool = False
    ) -> Tuple:
        """(masks[, indices][, values]) -- the mask comes first
        (ash/hashmap.py:82-95)."""
        assert return_indices or return_values, "Must return at least one of indices or values"
        indices, masks = self.engine.find(keys)
        out = (masks,)
        if return_indices:
            out += (indices,)
        if return_values:
            out += (self._gather(indices),)
        return out

    def erase(self, keys: torch.Tensor) -> None:
        self.engine.erase(keys)

    def clear(self) -> None:
        for store in self.values.values():
            store.zero_()
        self.engine.clear()

    def size(self) -> int:
        return self.engine.size()

    def resize(self, new_capacity: int) -> None:
        """Moves keys and value rows into freshly sized storage and swaps the
        registered buffers (ash/hashmap.py:108-122)."""
        grown = {
            name: torch.zeros(new_capacity, *store.shape[1:], device=self.engine.device)
            for name, store in self.values.items()
        }
        self.engine.resize(new_capacity, self.values, grown)
        for name in self.values:
            delattr(self, name)
        self.values = grown
        for name, store in grown.items():
            self.register_buffer(name, store)

    def keys(self) -> torch.Tensor:
        return self.engine.keys()

    def items(self, return_indices: bool = True, return_values: bool = False) -> Tuple:
        """(keys[, indices][, values]) of the live entries."""
        assert return_indices or return_values, "Must return at least one of indices or values"
        live_keys, live_indices = self.engine.items()
        out = (live_keys,)
        if return_indices:
            out += (live_indices,)
        if return_values:
            out += (self._gather(live_indices),)
        return out


class HashSet(ASHModule):
    """Keys only (ash/hashmap.py:149-178)."""

    def __init__(self, key_dim: int, capacity: int, device: torch.device):
        super().__init__()
        self.engine = ASHEngine(key_dim, capacity, device)

    def insert(self, keys: torch.Tensor) -> None:
        self.engine.insert_keys(keys)

    def find(self, keys: torch.Tensor) -> torch.Tensor:
        return self.engine.find(keys)[1]

    def erase(self, keys: torch.Tensor) -> None:
        self.engine.erase(keys)

    def clear(self) -> None:
        self.engine.clear()

    def size(self) -> int:
        return self.engine.size()

    def resize(self, new_capacity: int) -> None:
        self.engine.resize(new_capacity)

    def keys(self) -> torch.Tensor:
        return self.engine.keys()

"""HashSet and HashMap: an ASHEngine, plus (for the map) the value tensors it
addresses.

Constructor arguments, method names, return orders and buffer names are those
of the reference wrappers (ash/hashmap.py:7-178); how values are declared and
handed over is kept in one place, `_ValueLayout`.
"""
from typing import Dict, List, Tuple, Union

import torch

from . import core
from .core import ASHEngine, ASHModule

ValueSpec = Union[int, List[int], Dict[str, int]]
Values = Union[torch.Tensor, List[torch.Tensor], Dict[str, torch.Tensor]]


class _ValueLayout:
    """The three ways of declaring a map's values (ash/hashmap.py:23-36) and
    the matching shapes in which values are passed in and handed back: one
    width -> one tensor, stored as "default"; a list of widths -> a list of
    tensors, stored as "default_<i>"; a dict -> a dict under its own names."""

    def __init__(self, value_dims: ValueSpec):
        if not isinstance(value_dims, (int, list, dict)):
            raise ValueError("value_dims must be int, list or dict")
        self.kind = next(k for k in (int, list, dict) if isinstance(value_dims, k))
        if self.kind is int:
            self.widths = {"default": value_dims}
        elif self.kind is list:
            self.widths = {f"default_{i}": width for i, width in enumerate(value_dims)}
        else:
            self.widths = dict(value_dims)

    @property
    def names(self) -> Tuple[str, ...]:
        return tuple(self.widths)

    def storage(self, capacity: int, device) -> Dict[str, torch.Tensor]:
        """Zeroed (capacity, width) tensors, one per value."""
        return {
            name: torch.zeros(capacity, width, device=device)
            for name, width in self.widths.items()
        }

    def named(self, values: Values) -> Dict[str, torch.Tensor]:
        """Values as passed by the caller -> name -> tensor; the shape has to
        be the declared one."""
        if isinstance(values, torch.Tensor):
            assert self.kind is int
            return {"default": values}
        if isinstance(values, list):
            assert self.kind is list
            return {f"default_{i}": v for i, v in enumerate(values)}
        if isinstance(values, dict):
            assert self.kind is dict
            return values
        raise ValueError("values must be Tensor, list, or dict")

    def declared(self, named: Dict[str, torch.Tensor]) -> Values:
        """name -> tensor back to the declared shape."""
        if self.kind is int:
            return named["default"]
        if self.kind is list:
            return [named[name] for name in self.names]
        return named


class HashSet(ASHModule):
    """Keys only (ash/hashmap.py:149-178)."""

    def __init__(self, key_dim: int, capacity: int, device: torch.device):
        super().__init__()
        self.engine = ASHEngine(key_dim, capacity, device)

    def insert(self, keys: torch.Tensor) -> None:
        self.engine.insert_keys(keys)

    def find(self, keys: torch.Tensor) -> torch.Tensor:
        """Mask of the keys that are stored."""
        _, masks = self.engine.find(keys)
        return masks

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


class HashMap(ASHModule):
    """Keys with values.  Every value is a float tensor with one row per index
    of the engine, registered as a buffer under its name (so it travels with
    `state_dict`) and also reachable through `self.values`."""

    def __init__(
        self,
        key_dim: int,
        value_dims: ValueSpec,
        capacity: int,
        device: Union[str, torch.device] = torch.device("cpu"),
    ):
        super().__init__()
        self._layout = _ValueLayout(value_dims)
        self.value_dims = value_dims
        self.engine = ASHEngine(key_dim, capacity, device)
        self.values: Dict[str, torch.Tensor] = {}
        self._adopt(self._layout.storage(capacity, device))

    def _adopt(self, storage: Dict[str, torch.Tensor]) -> None:
        """Makes `storage` the map's value tensors and buffers."""
        for name in self.values:
            delattr(self, name)
        self.values = storage
        for name, rows in storage.items():
            self.register_buffer(name, rows)

    def reinterpret_value_dict(self, values: Dict[str, torch.Tensor]) -> Values:
        """name -> tensor in the shape the map was declared with."""
        return self._layout.declared(values)

    def _rows(self, indices: torch.Tensor) -> Values:
        """The value rows at `indices` (ash/hashmap.py:87-95,138-146 index every
        tensor with torch); the native backend gathers all tensors in one
        launch."""
        gather = getattr(core.backend, "gather_rows", None)
        if gather is not None:
            return self._layout.declared(gather(self.values, indices))
        return self._layout.declared({name: rows[indices] for name, rows in self.values.items()})

    def _answer(self, first, indices, return_indices: bool, return_values: bool) -> Tuple:
        assert return_indices or return_values, "Must return at least one of indices or values"
        answer = [first]
        if return_indices:
            answer.append(indices)
        if return_values:
            answer.append(self._rows(indices))
        return tuple(answer)

    def insert(self, keys: torch.Tensor, values: Values) -> None:
        self.engine.insert(keys, self._layout.named(values), self.values)

    def find(
        self, keys: torch.Tensor, return_indices: bool = True, return_values: bool = False
    ) -> Tuple:
        """(masks[, indices][, values]) -- the mask comes first
        (ash/hashmap.py:82-95)."""
        indices, masks = self.engine.find(keys)
        return self._answer(masks, indices, return_indices, return_values)

    def items(self, return_indices: bool = True, return_values: bool = False) -> Tuple:
        """(keys[, indices][, values]) of the stored entries."""
        keys, indices = self.engine.items()
        if return_values and getattr(self.engine.backend, "last_items_in_index_order", False):
            # entry i sits under index i: values[name][indices] (ash/hashmap.py:138-146)
            # is a copy of the first rows
            assert return_indices or return_values
            n = indices.shape[0]
            gather = getattr(core.backend, "gather_rows", None)
            if gather is not None:
                rows = self._layout.declared(gather(self.values, None, first=n))   # one launch
            else:
                rows = self._layout.declared({name: v[:n].clone() for name, v in self.values.items()})
            return (keys, indices, rows) if return_indices else (keys, rows)
        return self._answer(keys, indices, return_indices, return_values)

    def keys(self) -> torch.Tensor:
        return self.engine.keys()

    def erase(self, keys: torch.Tensor) -> None:
        self.engine.erase(keys)

    def clear(self) -> None:
        """Empties the table and zeroes the values (ash/hashmap.py:100-103)."""
        for rows in self.values.values():
            rows.zero_()
        self.engine.clear()

    def size(self) -> int:
        return self.engine.size()

    def resize(self, new_capacity: int) -> None:
        """New storage of `new_capacity` rows per value; the engine moves keys
        and rows over, then the buffers are swapped (ash/hashmap.py:108-122)."""
        roomier = {
            name: torch.zeros(new_capacity, *rows.shape[1:], device=self.engine.device)
            for name, rows in self.values.items()
        }
        self.engine.resize(new_capacity, self.values, roomier)
        self._adopt(roomier)

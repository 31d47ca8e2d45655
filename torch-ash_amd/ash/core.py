"""ASHEngine: the key -> index map and its serialisable state.

API, buffer names, dtypes and warning behaviour follow the reference engine
(ash/core.py:39-371) so that checkpoints and calling code carry over; the work
itself happens in the HIP table behind `backend.HashMap`.
"""
import warnings
from typing import Dict, Optional, Tuple, Union

import torch
import torch.nn as nn

from .common import _get_c_extension

backend = _get_c_extension()

DeviceLike = Union[str, torch.device]


def _as_device(device: DeviceLike) -> torch.device:
    return torch.device(device) if isinstance(device, str) else device


class ASHEngine(nn.Module):
    """Collision-free map from int32[dim] keys to dense indices in [0, capacity).

    The index of a key addresses rows of value / embedding tensors owned by the
    caller.  State (ash/core.py:69-90): `_heap` int32[capacity] is the free list
    shared with the native table; `_keys`, `_indices`, `_size` are only filled
    when a state dict is taken.
    """

    def __init__(self, dim: int, capacity: int, device: DeviceLike = torch.device("cpu")):
        super().__init__()
        assert dim > 0, "dim must be positive"
        assert capacity > 0, "capacity must be positive"
        self.dim = dim
        self.capacity = capacity
        self.device = _as_device(device)
        self._hooked = False
        self._allocate_state()
        self.backend = backend.HashMap(self.dim, self.capacity, self._heap, self.device)

    # ------------------------------------------------------------ state
    def _allocate_state(self) -> None:
        """(Re)creates the four buffers (ash/core.py:69-90)."""
        dev, cap = self.device, self.capacity
        self.register_buffer("_heap", torch.arange(cap, dtype=torch.int32, device=dev))
        self.register_buffer("_keys", torch.zeros((cap, self.dim), dtype=torch.int32, device=dev))
        self.register_buffer("_indices", torch.zeros(cap, dtype=torch.int64, device=dev))
        self.register_buffer("_size", torch.zeros(1, dtype=torch.int32, device=dev))
        if not self._hooked:
            self.register_load_state_dict_post_hook(self._restore_backend)
            self._hooked = True

    def state_dict(self, destination=None, prefix: str = "", keep_vars: bool = False):
        """Snapshots the live (key, index) pairs into the buffers before the
        usual collection (ash/core.py:92-115)."""
        state = super().state_dict(destination=destination, prefix=prefix, keep_vars=keep_vars)
        live_keys, live_indices = self.items()
        count = live_keys.shape[0]
        self._size.fill_(count)
        if count:
            self._keys[:count] = live_keys
            self._indices[:count] = live_indices
        return state

    def _restore_backend(self, module, incompatible_keys) -> None:
        """Rebuilds the native table from freshly loaded buffers
        (ash/core.py:117-135)."""
        count = int(self._size.item())
        assert self._heap.shape[0] == self.capacity
        loaded_keys = self._keys[:count]
        self._key_check(loaded_keys)
        self.backend.load_states(
            {
                "active_keys": loaded_keys,
                "active_indices": self._indices[:count],
                "heap": self._heap,
            }
        )
        self._dropped_seen = 0

    # ----------------------------------------------------------- checks
    def _key_check(self, keys: torch.Tensor) -> None:
        assert keys.dim() == 2 and keys.shape[1] == self.dim, "keys shape mismatch"
        if keys.dtype != torch.int32:
            warnings.warn("keys are not int32, conversion might reduce precision.")

    def _value_check(
        self, values: Dict[str, torch.Tensor], external_values: Dict[str, torch.Tensor]
    ) -> None:
        assert values.keys() == external_values.keys()
        for name, rows in values.items():
            store = external_values[name]
            assert rows.is_contiguous() and store.is_contiguous()
            assert rows.ndim == store.ndim
            assert rows.dtype == store.dtype
            assert rows.shape[1:] == store.shape[1:]
            assert store.shape[0] == self.capacity

    def _prepare(self, keys: torch.Tensor) -> torch.Tensor:
        return keys.to(self.device, torch.int32).contiguous()

    def _warn_if_overfull(self, inserted: int, dropped_before: int) -> None:
        """The reference notices an overflow by comparing sizes before and after
        (ash/core.py:203-211); here the table refuses the surplus keys and
        counts them, and the same warning is raised from that count."""
        read = getattr(self.backend, "status_after_insert", self.backend.status)
        status = read()
        dropped = status["dropped"] - dropped_before
        self._dropped_seen = status["dropped"]
        if dropped > 0:
            warnings.warn(
                f"Insertion of {inserted} keys exceeds the hash map capacity {self.capacity}: "
                f"{dropped} keys were not stored (size is {status['size']}). "
                "Please resize the hash map or the behavior could be unexpected."
            )

    # ------------------------------------------------------------- ops
    def find(self, keys: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """Returns (indices int64[N], masks bool[N]); index 0 where not found."""
        self._key_check(keys)
        if keys.shape[0] == 0:
            warnings.warn("empty keys")
            return (
                torch.empty((0,), dtype=torch.int64, device=self.device),
                torch.empty((0,), dtype=torch.bool, device=self.device),
            )
        return self.backend.find(self._prepare(keys))

    def insert_keys(self, keys: torch.Tensor) -> None:
        self._key_check(keys)
        if keys.shape[0] == 0:
            warnings.warn("empty keys")
            return
        dropped_before = self._dropped()
        room = self._room_known()
        self.backend.insert_keys(self._prepare(keys))
        if not self._surely_stored(keys.shape[0], room):
            self._warn_if_overfull(keys.shape[0], dropped_before)

    def insert(
        self,
        keys: torch.Tensor,
        values: Dict[str, torch.Tensor],
        external_values: Dict[str, torch.Tensor],
    ) -> None:
        """Inserts keys and copies `values[name][i]` to
        `external_values[name][index_of(keys[i])]` for every new key."""
        self._key_check(keys)
        if keys.shape[0] == 0:
            warnings.warn("empty keys")
            return
        self._value_check(values, external_values)
        for rows in values.values():
            assert rows.shape[0] == keys.shape[0]
        dropped_before = self._dropped()
        room = self._room_known()
        self.backend.insert(self._prepare(keys), values, external_values)
        if not self._surely_stored(keys.shape[0], room):
            self._warn_if_overfull(keys.shape[0], dropped_before)

    def _room_known(self) -> Optional[int]:
        """Free indices before an insert, if the backend knows the size without
        asking the device."""
        known = getattr(self.backend, "known_size", None)
        size = known() if known is not None else None
        return None if size is None else self.capacity - size

    def _surely_stored(self, inserted: int, room: Optional[int]) -> bool:
        """Whether the overflow check can be left out: the backend has returned
        from a streaming insert without reading its counters, and the batch
        fitted the free indices, so no key was refused for lack of room.  The
        counters are looked at by the next call that needs them."""
        return (
            room is not None
            and inserted <= room
            and getattr(self.backend, "counters_queued", False)
        )

    def _dropped(self) -> int:
        # kept on the host: the count only changes inside insert calls
        return getattr(self, "_dropped_seen", 0)

    def erase(self, keys: torch.Tensor) -> None:
        self._key_check(keys)
        if keys.shape[0] == 0:
            warnings.warn("empty keys")
            return
        self.backend.erase(self._prepare(keys))

    def clear(self) -> None:
        self.backend.clear()
        self._dropped_seen = 0

    def size(self) -> int:
        return self.backend.size()

    def resize(
        self,
        capacity: int,
        old_external_values: Optional[Dict[str, torch.Tensor]] = None,
        new_external_values: Optional[Dict[str, torch.Tensor]] = None,
    ) -> None:
        """Rebuilds the map with a new capacity, moving value rows along when
        both value dicts are given (ash/core.py:266-302)."""
        live_keys, old_indices = self.items()
        count = live_keys.shape[0]
        assert capacity >= count, "new capacity is smaller than the current size"
        assert capacity > 0, "new capacity is 0"

        del self.backend
        self.capacity = capacity
        self._allocate_state()
        self.backend = backend.HashMap(self.dim, self.capacity, self._heap, self.device)
        self._dropped_seen = 0
        if count == 0:
            return
        if old_external_values is not None and new_external_values is not None:
            carried = {name: store[old_indices] for name, store in old_external_values.items()}
            self.backend.insert(live_keys, carried, new_external_values)
        else:
            self.backend.insert_keys(live_keys)

    def keys(self) -> torch.Tensor:
        return self.items()[0]

    def items(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """Live keys int32[n, dim] and their indices int64[n], in table order."""
        return self.backend.items()

    # ------------------------------------------------------- placement
    def to(self, device: DeviceLike):
        """As in the reference (ash/core.py:325-337) moving an engine yields a
        new, empty engine on the target device."""
        return ASHEngine(self.dim, self.capacity, _as_device(device))

    def cpu(self):
        return self.to("cpu")

    def cuda(self, device: Optional[DeviceLike] = None):
        return self.to("cuda" if device is None else device)

    def __repr__(self) -> str:
        return (
            f"ASHEngine (dim={self.dim}, capacity={self.capacity}, "
            f"size={self.size()}) at {self.device}"
        )


class ASHModule(nn.Module):
    """Base of the modules that own an engine; keeps `.to()` consistent
    (ash/core.py:351-371)."""

    def __init__(self):
        super().__init__()
        self.engine = None

    def to(self, device):
        assert self.engine is not None, "engine is not initialized"
        moved = super().to(device)
        moved.engine = moved.engine.to(device)
        return moved

    def cpu(self):
        return self.to(torch.device("cpu"))

    def cuda(self, device: Optional[DeviceLike] = None):
        return self.to(torch.device("cuda") if device is None else device)

"""Device memory behind the cache manager's page ids and state slots."""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class SlotStore:
    """What one mixer call sees: the paged arrays of its cache slot
    (``arrays[name]`` is [num_pages, elems_per_token * page_size], each with the
    width and dtype its mixer asked for), its group's index into
    ``batch.block_tables``, and its per-request state arrays
    (``state[name]`` is [num_state_slots, *shape]) if it keeps any."""

    group: int = 0
    page_size: int = 0
    arrays: dict[str, torch.Tensor] = field(default_factory=dict)
    state: dict[str, torch.Tensor] = field(default_factory=dict)


class CacheStorage:
    def __init__(self, model, pages_per_group: list[int], page_size: int, num_state_slots: int,
                 *, dtype: torch.dtype, device) -> None:
        groups, layouts = model.cache_layout()
        self.page_size = page_size
        self._slots: dict[int, SlotStore] = {}
        for slot, layout in layouts.items():
            arrays = {
                name: torch.zeros((pages_per_group[layout.group], array.elems_per_token * page_size),
                                  dtype=array.dtype or dtype, device=device)
                for name, array in layout.request.arrays
            }
            self._slots[slot] = SlotStore(layout.group, page_size, arrays)
        for slot, request in model.state_requests().items():
            store = self._slots.setdefault(slot, SlotStore(0, page_size))
            store.state = {name: torch.zeros((num_state_slots, *array.shape), dtype=array.dtype, device=device)
                           for name, array in request.items()}
        self._empty = SlotStore(0, page_size)

    def slot(self, index: int) -> SlotStore:
        return self._slots.get(index, self._empty)

    def reset_state(self, state_slot: int) -> None:
        """Zero the fixed-size state of one request slot (on admission)."""
        for store in self._slots.values():
            for array in store.state.values():
                array[state_slot].zero_()

    def bytes(self) -> int:
        total = 0
        for store in self._slots.values():
            for t in (*store.arrays.values(), *store.state.values()):
                total += t.numel() * t.element_size()
        return total

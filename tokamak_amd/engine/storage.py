"""Device memory behind the cache manager's page ids and state slots."""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


@dataclass
class SlotStore:
    """What one mixer call sees: the paged arrays of its cache slot
    (``arrays[name]`` is [num_pages, elems_per_token * page_size]), its group's
    index into ``batch.block_tables``, and its per-request state
    ([num_state_slots, *shape]) if it keeps any."""

    group: int = 0
    page_size: int = 0
    arrays: dict[str, torch.Tensor] = field(default_factory=dict)
    state: torch.Tensor | None = None


class CacheStorage:
    def __init__(self, model, pages_per_group: list[int], page_size: int, num_state_slots: int,
                 *, dtype: torch.dtype, device) -> None:
        groups, layouts = model.cache_layout()
        self.page_size = page_size
        self._slots: dict[int, SlotStore] = {}
        for slot, layout in layouts.items():
            elems = layout.request.elems_per_token * page_size
            arrays = {
                name: torch.zeros((pages_per_group[layout.group], elems), dtype=dtype, device=device)
                for name in layout.request.arrays
            }
            self._slots[slot] = SlotStore(layout.group, page_size, arrays)
        for slot, shape in model.state_shapes().items():
            store = self._slots.setdefault(slot, SlotStore(0, page_size))
            store.state = torch.zeros((num_state_slots, *shape), dtype=torch.float32, device=device)
        self._empty = SlotStore(0, page_size)

    def slot(self, index: int) -> SlotStore:
        return self._slots.get(index, self._empty)

    def reset_state(self, state_slot: int) -> None:
        """Zero the fixed-size state of one request slot (on admission)."""
        for store in self._slots.values():
            if store.state is not None:
                store.state[state_slot].zero_()

    def bytes(self) -> int:
        total = 0
        for store in self._slots.values():
            for t in store.arrays.values():
                total += t.numel() * t.element_size()
            if store.state is not None:
                total += store.state.numel() * 4
        return total

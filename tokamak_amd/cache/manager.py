"""The cache manager: pages for every group, and fixed-size state slots.

Reference behaviour kept (src/tokamak/memory/block_manager.py:74-145):
growth on demand, append-only tables, all-or-nothing allocation that leaves
the state intact when it fails, idempotent free.  Added: several groups, early
release behind a window, and slots for per-request state of fixed size.
"""

from __future__ import annotations

from tokamak_amd.cache.pages import CacheGroupSpec, GroupTables, OutOfPagesError


class OutOfSlotsError(RuntimeError):
    """Every state slot is taken."""


class StateSlots:
    """``num_slots`` slots for per-request state of fixed size.  A request gets
    the lowest free slot at admission and loses it when it ends or is
    preempted; whoever owns state indexed by the slot resets it on acquire."""

    def __init__(self, num_slots: int) -> None:
        if num_slots < 1:
            raise ValueError(f"num_slots must be >= 1, got {num_slots}")
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._slot_of: dict[object, int] = {}

    @property
    def num_free(self) -> int:
        return len(self._free)

    def slot_of(self, request) -> int | None:
        return self._slot_of.get(request)

    def acquire(self, request) -> int:
        if request in self._slot_of:
            return self._slot_of[request]
        if not self._free:
            raise OutOfSlotsError(f"all {self.num_slots} state slots are taken")
        slot = self._free.pop()
        self._slot_of[request] = slot
        return slot

    def release(self, request) -> None:
        slot = self._slot_of.pop(request, None)
        if slot is not None:
            self._free.append(slot)

    def check(self) -> None:
        held = sorted(self._slot_of.values())
        both = sorted(held + self._free)
        if both != list(range(self.num_slots)):
            raise AssertionError("a state slot is lost, or held twice")


class CacheManager:
    """Pages of all groups plus the state slots, behind one interface.

    ``pages_per_group`` gives each group's pool size (an int applies to all).
    """

    def __init__(
        self,
        groups: list[CacheGroupSpec],
        pages_per_group: int | list[int],
        page_size: int,
        num_state_slots: int,
    ) -> None:
        if isinstance(pages_per_group, int):
            pages_per_group = [pages_per_group] * len(groups)
        if len(pages_per_group) != len(groups):
            raise ValueError("one pool size per cache group is required")
        self.page_size = page_size
        self.groups = [GroupTables(g, n, page_size) for g, n in zip(groups, pages_per_group)]
        self.slots = StateSlots(num_state_slots)
        self.group_of_slot: dict[int, int] = {}
        for gi, g in enumerate(groups):
            for s in g.slots:
                if s in self.group_of_slot:
                    raise ValueError(f"cache slot {s} is in two groups")
                self.group_of_slot[s] = gi

    # -- pages ---------------------------------------------------------------
    def pages_needed(self, num_tokens: int) -> int:
        return -(-num_tokens // self.page_size)

    def num_free_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_free

    def num_pages(self, group: int = 0) -> int:
        return self.groups[group].pool.num_pages

    def can_hold(self, request, num_tokens: int) -> bool:
        return all(g.shortfall(request, num_tokens) <= g.pool.num_free for g in self.groups)

    def ensure_capacity(self, request, num_tokens: int) -> None:
        """Grow every group's table to cover ``num_tokens``; all or nothing."""
        for g in self.groups:
            need = g.shortfall(request, num_tokens)
            if need > g.pool.num_free:
                raise OutOfPagesError(
                    f"request {request!r} needs {need} more page(s) of group {g.spec.name!r} for "
                    f"{num_tokens} tokens, but only {g.pool.num_free} of {g.pool.num_pages} are free"
                )
        for g in self.groups:
            g.grow(request, num_tokens)

    def release_behind_window(self, request, num_cached_tokens: int) -> int:
        """Before a step whose first query sits at position ``num_cached_tokens``:
        windowed groups give back pages no present or future query can see."""
        released = 0
        for g in self.groups:
            if g.spec.window is not None:
                released += g.release_before(request, num_cached_tokens - g.spec.window + 1)
        return released

    def block_table(self, request, group: int = 0) -> list[int]:
        return self.groups[group].tables.get(request, [])

    def reserved_tokens(self, request, group: int = 0) -> int:
        return self.groups[group].live_pages(request) * self.page_size

    # -- lifetime ------------------------------------------------------------
    def admit(self, request) -> int:
        """Give the request a state slot (its pages come with ``ensure_capacity``)."""
        return self.slots.acquire(request)

    def free(self, request) -> None:
        """Give back everything the request holds; a no-op for unknown requests."""
        for g in self.groups:
            g.free(request)
        self.slots.release(request)

    def check(self) -> None:
        for g in self.groups:
            g.pool.check()
            held = [p for t in g.tables.values() for p in t if p != -1]
            if len(set(held)) != len(held):
                raise AssertionError("a page is in two block tables")
            if len(held) + g.pool.num_free != g.pool.num_pages:
                raise AssertionError("a page is lost")
        self.slots.check()

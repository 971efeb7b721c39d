"""Cache manager: paged storage accounting and per-request state slots."""

from tokamak_amd.cache.manager import CacheManager, OutOfSlotsError, StateSlots
from tokamak_amd.cache.pages import (
    RELEASED,
    CacheGroupSpec,
    GroupTables,
    OutOfPagesError,
    PagePool,
)

__all__ = [
    "RELEASED",
    "CacheGroupSpec",
    "CacheManager",
    "GroupTables",
    "OutOfPagesError",
    "OutOfSlotsError",
    "PagePool",
    "StateSlots",
]

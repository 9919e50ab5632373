from .manager import NO_PAGE, CacheManager, OutOfSlots, PagedGroup, SequenceHandle, StateSlots
from .page_pool import OutOfPages, PagePool
from .requirements import PagedKv, SlotState

__all__ = ["NO_PAGE", "CacheManager", "OutOfSlots", "PagedGroup", "SequenceHandle", "StateSlots", "OutOfPages",
           "PagePool", "PagedKv", "SlotState"]

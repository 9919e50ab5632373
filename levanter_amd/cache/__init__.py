from .manager import NO_PAGE, CacheManager, group_units, OutOfSlots, PagedGroup, SequenceHandle, StateSlots
from .page_pool import OutOfPages, PagePool
from .requirements import PagedKv, SlotState
from .sizing import pages_per_group

__all__ = ["NO_PAGE", "CacheManager", "OutOfSlots", "PagedGroup", "SequenceHandle", "StateSlots", "OutOfPages",
           "PagePool", "PagedKv", "SlotState", "group_units", "pages_per_group"]

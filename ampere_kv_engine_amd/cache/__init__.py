from .pages import RELEASED, BlockTable, PageAllocator, PagePoolExhausted
from .slots import SlotsExhausted, SlotTable
from .manager import CacheManager, LayerCache, PagedGroup, Sequence

__all__ = ["RELEASED", "BlockTable", "PageAllocator", "PagePoolExhausted", "SlotsExhausted", "SlotTable",
           "CacheManager", "LayerCache", "PagedGroup", "Sequence"]

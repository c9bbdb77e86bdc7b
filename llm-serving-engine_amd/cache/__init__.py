from .cell import CacheCell
from .manager import CacheManager, PageGroup, Reservation, SequenceRecord
from .pool import CacheFullError, PagePool

__all__ = ["CacheCell", "CacheFullError", "CacheManager", "PageGroup", "PagePool", "Reservation", "SequenceRecord"]

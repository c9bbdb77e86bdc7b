from .manager import CacheManager, PageGroup, Reservation, SequenceRecord
from .pool import CacheFullError, PagePool

__all__ = ["CacheFullError", "CacheManager", "PageGroup", "PagePool", "Reservation", "SequenceRecord"]

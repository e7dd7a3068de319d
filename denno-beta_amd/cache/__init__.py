from .manager import CacheError, CacheManager, GroupLayout, OutOfPages, PAGED, STATE, SlotState
from .storage import CacheStorage

__all__ = ["CacheError", "CacheManager", "GroupLayout", "OutOfPages", "PAGED", "STATE", "SlotState", "CacheStorage"]

from .manager import CacheError, CacheManager, GroupSpec, OutOfPages, OutOfSlots

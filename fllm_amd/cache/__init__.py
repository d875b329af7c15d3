from .manager import CacheManager, GroupSpec
from .pages import OutOfPages, PagePool

__all__ = ["CacheManager", "GroupSpec", "OutOfPages", "PagePool"]

from .manager import CacheManager, CacheView, PagedGroup
from .native import CoreError, HostCore, xorshift64_stream
from .spec import FixedState, PagedKV

__all__ = ["CacheManager", "CacheView", "PagedGroup", "CoreError", "HostCore", "xorshift64_stream",
           "FixedState", "PagedKV"]

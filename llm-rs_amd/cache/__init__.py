from .manager import CacheManager, PagedGroup
from .native import CoreError, HostCore, xorshift64_stream
from .spec import CacheKind, CacheView, FixedState, PagedKV, cache_kind, register_cache_kind

__all__ = ["CacheManager", "CacheView", "PagedGroup", "CoreError", "HostCore", "xorshift64_stream",
           "CacheKind", "FixedState", "PagedKV", "cache_kind", "register_cache_kind"]

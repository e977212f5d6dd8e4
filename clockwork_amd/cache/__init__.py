from clockwork_amd.cache.allocator import OutOfPages, PagePool
from clockwork_amd.cache.manager import NO_PAGE, CacheManager, GroupLayout, plan_groups
from clockwork_amd.cache.prefix import PrefixCache, PrefixMatch

__all__ = [
    "OutOfPages",
    "PagePool",
    "NO_PAGE",
    "CacheManager",
    "GroupLayout",
    "plan_groups",
    "PrefixCache",
    "PrefixMatch",
]

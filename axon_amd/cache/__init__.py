from .manager import CacheError, CacheGroup, CacheManager, GroupPlan, OutOfPages, host_lib

__all__ = ["CacheError", "CacheGroup", "CacheManager", "GroupPlan", "OutOfPages", "host_lib"]

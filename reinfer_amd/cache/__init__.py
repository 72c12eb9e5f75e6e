from .manager import (BlockPool, CacheGroupSpec, CacheManager, OutOfBlocks, OutOfSlots, RequestCache,
                      SlotPool, plan_groups)

__all__ = ["BlockPool", "CacheGroupSpec", "CacheManager", "OutOfBlocks", "OutOfSlots", "RequestCache",
           "SlotPool", "plan_groups"]

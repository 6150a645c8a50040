from .manager import (CacheError, CacheManager, GroupSpec, OutOfPages, PagePool, RequestCache,
                      StateSlots, chain_hash)
from .plan import CachePlan, KVNeed, StateNeed, plan_cache

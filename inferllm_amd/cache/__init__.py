from .manager import PAGE_SIZE, CacheManager, KVGroup, KVSpec, StateSpec, TokenTensor, round_up
from .slots import CacheError, CacheFull, FreeList

__all__ = ["PAGE_SIZE", "CacheManager", "KVGroup", "KVSpec", "StateSpec", "TokenTensor", "round_up",
           "CacheError", "CacheFull", "FreeList"]

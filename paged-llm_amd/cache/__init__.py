from .block_manager import NO_PAGE, CacheManager, GroupSpec, PageCopy, PagePool, StateSlotPool, chain_digest

__all__ = ["NO_PAGE", "CacheManager", "GroupSpec", "PageCopy", "PagePool", "StateSlotPool", "chain_digest"]

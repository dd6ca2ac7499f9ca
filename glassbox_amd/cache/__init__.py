from .manager import FULL, WINDOW, CacheError, CacheManager, GroupSpec, OutOfPages, chain_hash

__all__ = ["FULL", "WINDOW", "CacheError", "CacheManager", "GroupSpec", "OutOfPages", "chain_hash"]

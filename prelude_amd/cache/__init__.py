from .manager import (CacheError, KVLayerCache, OutOfPages, PageTables, StateLayerCache, allocate_storage,
                      bytes_per_token, plan_groups)

__all__ = ["CacheError", "KVLayerCache", "OutOfPages", "PageTables", "StateLayerCache", "allocate_storage",
           "bytes_per_token", "plan_groups"]

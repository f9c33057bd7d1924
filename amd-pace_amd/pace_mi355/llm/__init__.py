from .cache import (  # noqa: F401
    KVCacheBase,
    KVCacheManager,
    KVCacheType,
    PagedKVCache,
    PagedKVView,
    get_kv_cache_class,
)
from .contiguous import BMCKVCache, DynamicKVCache  # noqa: F401
from .ops import LLMBackendType, LLMOperatorType  # noqa: F401
from . import speculative  # noqa: F401

__all__ = [
    "KVCacheType", "KVCacheManager", "KVCacheBase", "PagedKVCache", "PagedKVView",
    "DynamicKVCache", "BMCKVCache", "LLMOperatorType", "LLMBackendType", "get_kv_cache_class",
]

from .kv_cache import DynamicKVCache, KVCache, PagedKVCache, StaticKVCache
from .layers import Embedding, Linear, RMSNorm
from .module import Module

__all__ = ["Module", "Linear", "RMSNorm", "Embedding", "KVCache", "DynamicKVCache", "StaticKVCache", "PagedKVCache"]

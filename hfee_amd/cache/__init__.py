from .manager import CacheManager, CacheGroupSpec, PagePool, RequestCache, OutOfPages, CacheError
from .storage import CacheStorage, bytes_per_token
from . import capacity

from .manager import CacheManager, GroupSpec, RequestCache
from .pages import CacheAccountingError, IdPool
from .storage import CacheStorage

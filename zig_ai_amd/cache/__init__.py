"""Cache manager: pages with block tables per request and group, state slots."""

from .pages import OutOfPages, OutOfSlots, Pool, PoolError  # noqa: F401
from .manager import FREED, CacheManager, CacheView, PagedGroup  # noqa: F401

from .page_pool import PagePool  # noqa: F401
from .specs import PagedKV, FixedState  # noqa: F401
from .manager import CacheManager, PagedView, StateView  # noqa: F401

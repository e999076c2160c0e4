from .page_pool import PagePool  # noqa: F401
from .specs import PagedKV, FixedState  # noqa: F401
from .manager import CacheManager, View, PagedView, StateView, bytes_per_page  # noqa: F401

from .page_pool import PagePool  # noqa: F401
from .specs import PagedKV, FixedState, PagedLatent, States, Bundle  # noqa: F401
from .manager import CacheManager, View, PagedView, StateView, BundleView, bytes_per_page, flatten_specs  # noqa: F401

"""lasp_cache under the reference's module path (lasp/lasp_cache.py:539-652)."""
from .lasp_naive import LaspCache, lasp_cache, lasp_cache_  # noqa: F401

__all__ = ["LaspCache", "lasp_cache_", "lasp_cache"]

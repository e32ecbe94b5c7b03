from .paged import PAGE, CacheError, GroupSpec, PagePool, PagedCache, group_entries, pages_for  # noqa: F401
from . import layout  # noqa: F401

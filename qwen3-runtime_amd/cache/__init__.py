from .manager import CacheManager  # noqa: F401
from .pages import CacheFull, PagePool  # noqa: F401
from .slots import StateSlots  # noqa: F401

from .pages import PagePool, SlotTable  # noqa: F401
from .sequence_cache import PAGE, CacheGroup, SequenceCache, pages_for  # noqa: F401

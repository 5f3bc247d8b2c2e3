"""Import path of the reference's tidal.utils.kv_cache; the classes are defined in ``paged``."""
from .paged import KvCache, KvPool  # noqa: F401

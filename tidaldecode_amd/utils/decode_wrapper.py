"""Import path of the reference's tidal.utils.decode_wrapper; the class is defined in ``paged``."""
from .paged import BatchDecodeWithPagedKVCacheWrapper, _check_kv_layout  # noqa: F401

"""Import path of the reference's tidal.utils.utils; the enum is defined in ``paged``."""
from .paged import TensorLayout  # noqa: F401

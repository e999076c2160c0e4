from .base import Part, register_part, build_part, registered_parts  # noqa: F401
from . import linear, norm, position, attention, feedforward, block, embedding  # noqa: F401

"""Parts of a layer: importing this package registers the built-in kinds."""
from . import attention, block, ends, feed_forward, norm, position  # noqa: F401
from .base import BuildContext, Part, ResidualStream, build_part  # noqa: F401

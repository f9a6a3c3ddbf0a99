"""Parts a layer is put together from.  Importing the package registers the
built-in kinds."""
from .registry import register_part, build_part, registered_parts
from .base import Part
from . import builtin  # noqa: F401  (registration)
from .builtin import NativePart

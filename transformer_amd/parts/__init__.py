"""Parts a block is put together from. Importing the package registers the
built-in kinds; ``register_part`` adds others."""
from .base import Part, PartError, build_part, register_part  # noqa: F401
from . import norm, position, attention, ffn, block  # noqa: F401

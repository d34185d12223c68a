"""Registry entries. Importing the package registers them."""
from . import llama  # noqa: F401

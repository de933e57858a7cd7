"""Registry entries. Importing the package registers them."""
from . import llama, vametar  # noqa: F401

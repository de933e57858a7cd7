"""Registry entries. Importing the package registers them."""
from . import kunitar, llama, vametar  # noqa: F401

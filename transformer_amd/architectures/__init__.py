"""Registry entries. Importing the package registers them."""
from . import kunitar, llama, luduvik, vametar  # noqa: F401

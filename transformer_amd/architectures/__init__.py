"""Registry entries. Importing the package registers them."""
from . import kunitar, llama, luduvik, saredra, vametar  # noqa: F401

"""Built-in architectures; importing the package registers them."""
from . import qwen2, rasizen, tatelorn  # noqa: F401

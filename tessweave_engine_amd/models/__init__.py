"""Built-in architectures; importing this package registers them."""
from . import qwen2  # noqa: F401

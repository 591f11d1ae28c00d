"""Built-in architectures; importing this package registers them."""
from . import pekasun, qwen2  # noqa: F401

"""Built-in architectures; importing this package registers them."""
from . import nebanex, pekasun, qwen2  # noqa: F401

"""Built-in model families; importing this package registers them."""
from . import qwen3  # noqa: F401

"""Built-in architectures; importing this package registers them."""

from . import larozen, mogilorn, qwen2, talolorn, videdra  # noqa: F401

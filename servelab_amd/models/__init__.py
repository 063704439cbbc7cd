"""Importing this package registers the architectures it holds."""
from . import futezen, qwen2, topelorn, vekanex, vunadra  # noqa: F401

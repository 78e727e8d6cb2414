"""Architectures built in; importing the package registers them."""
from . import dipisun, qwen2, tiverax  # noqa: F401
from . import gosulorn, lelutar  # noqa: F401

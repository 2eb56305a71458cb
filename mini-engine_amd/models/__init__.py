"""Architecture modules. Importing this package registers every architecture it holds."""

from . import bezurax, gonurax, kifezen, qwen3, sevadra  # noqa: F401

"""Built-in model families; importing this package registers them."""
from . import gimudra, qwen3, pavitar, vupuzen  # noqa: F401

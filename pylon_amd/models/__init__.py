"""Built-in model families; importing this package registers them."""
from . import gimudra, qwen3, pavitar, tukarax, vupuzen  # noqa: F401

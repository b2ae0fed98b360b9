"""Import path kept for code written against the reference; the class lives in ``fifth_order``."""
from .fifth_order import Tsit5  # noqa: F401

"""Import path kept for code written against the reference; the class lives in ``fifth_order``."""
from .fifth_order import Dopri5  # noqa: F401

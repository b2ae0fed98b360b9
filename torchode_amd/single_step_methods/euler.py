"""Import path kept for code written against the reference; the class lives in ``low_order``."""
from .low_order import Euler, LinearInterpolationData  # noqa: F401

"""Per-sample solver status codes.

Integer values and names follow torchode/status_codes.py:9-33 so that code
written against the reference keeps working: any value above ``SUCCESS``
signals an abnormal stop, and the loop stops the whole batch as soon as one
sample reports one.
"""
from enum import Enum

SUCCESS = 0
GENERAL_ERROR = 1
REACHED_DT_MIN = 2
REACHED_MAX_STEPS = 3
INFINITE_NORM = 4


class Status(Enum):
    """User-facing names for the integer status codes."""

    SUCCESS = SUCCESS
    GENERAL_ERROR = GENERAL_ERROR
    REACHED_DT_MIN = REACHED_DT_MIN
    REACHED_MAX_STEPS = REACHED_MAX_STEPS
    # The error-ratio norm was not finite (NaN or inf in y or in the error estimate).
    INFINITE_NORM = INFINITE_NORM

"""Per-sample solver status codes.

Integer values and names follow torchode/status_codes.py:9-33 so that code
written against the reference keeps working: any value above ``SUCCESS``
signals an abnormal stop, and the loop stops the whole batch as soon as one
sample reports one.
"""
from enum import Enum


class Status(Enum):
    """User-facing names for the integer status codes."""

    SUCCESS = 0
    GENERAL_ERROR = 1
    REACHED_DT_MIN = 2
    REACHED_MAX_STEPS = 3
    INFINITE_NORM = 4  # the error-ratio norm was not finite (NaN or inf in y or in the error estimate)


# the plain integers, as the kernels and the status tensors carry them
SUCCESS, GENERAL_ERROR, REACHED_DT_MIN, REACHED_MAX_STEPS, INFINITE_NORM = (code.value for code in Status)

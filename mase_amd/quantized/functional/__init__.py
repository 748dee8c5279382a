from .linear import linearBlockFP, linearInteger, linearMinifloatDenorm, linearMinifloatIEEE  # noqa: F401
from .mx_linear import mx_linear  # noqa: F401

from .linear import linearBlockFP, linearInteger, linearMinifloatDenorm, linearMinifloatIEEE  # noqa: F401

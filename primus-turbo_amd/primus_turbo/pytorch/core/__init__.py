from . import low_precision, utils  # noqa: F401

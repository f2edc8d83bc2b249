from . import quant  # noqa: F401

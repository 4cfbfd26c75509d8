from .operator import Operator  # noqa: F401

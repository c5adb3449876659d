from .ops import HipOps  # noqa: F401

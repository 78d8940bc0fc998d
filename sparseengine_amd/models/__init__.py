"""Architectures.  Importing the package registers each one in ``config.registry``."""
from . import minimax_m2  # noqa: F401

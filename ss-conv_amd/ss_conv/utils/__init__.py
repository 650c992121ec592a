from . import utils
from . import SO3
from . import kernel

__all__ = ["utils", "SO3", "kernel"]

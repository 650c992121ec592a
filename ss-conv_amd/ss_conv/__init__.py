"""ss_conv for MI355X: drop-in module layout of the reference package
(SS_Conv_lib/ss_conv/__init__.py) over hand-written gfx950 kernels."""
from . import _ext  # noqa: F401  fails loudly when libssc.so is not built
from . import sp_ops
from . import utils
from . import convolution
from . import activation
from . import batchnorm
from . import pool
from . import dropout

__all__ = ["sp_ops", "utils", "convolution", "activation", "batchnorm", "pool", "dropout"]

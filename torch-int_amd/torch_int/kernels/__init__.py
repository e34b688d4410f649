"""Alias of :mod:`torch_int._CUDA` under the name of the upstream source
directory (``torch_int/kernels``)."""
from .._CUDA import *  # noqa: F401,F403
from .._CUDA import __all__  # noqa: F401

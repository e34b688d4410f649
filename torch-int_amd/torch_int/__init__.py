"""INT8 W8A8 operators for AMD MI355X (gfx950).

Drop-in for the operator set of torch-int: the native entry points live in
``torch_int._CUDA`` (same names and signatures as upstream
``torch_int/kernels/bindings.cpp:5-20``) and are backed by hand-written HIP
kernels in ``libtorch_int_hip.so``; ``torch_int.nn`` and ``torch_int.models``
hold the modules built on them.
"""
from . import _CUDA  # noqa: F401  (fails loudly when the HIP library is missing)
from . import functional, nn  # noqa: F401

__all__ = ["_CUDA", "functional", "nn"]

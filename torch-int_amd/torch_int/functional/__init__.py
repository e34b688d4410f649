from . import bmm, fused, quantization  # noqa: F401

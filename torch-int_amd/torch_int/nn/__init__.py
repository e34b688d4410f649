from . import bmm, fused, linear  # noqa: F401
from .bmm import BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T, BMM_S8T_S8N_S32T  # noqa: F401
from .fused import DQ_Add_LayerNorm_Q, LayerNormQ  # noqa: F401
from .linear import (W8A8B8O8Linear, W8A8B8O8LinearReLU, W8A8B32O32Linear,  # noqa: F401
                     W8A8B32O32LinearWithoutScaling, W8A8BFP32OFP32Linear)
from .linear import W8A16Linear, W8FakeA8Linear  # noqa: F401  (upstream torch_int/nn/__init__.py exports these two)

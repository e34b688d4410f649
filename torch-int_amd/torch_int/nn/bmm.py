"""Modules around the batched INT8 products A . B^T (upstream
``torch_int/nn/bmm.py:5-58``).  ``a`` is the per-tensor output scale, kept as
a 0-dim fp32 buffer so state dicts stay interchangeable."""
import torch

from .. import _CUDA
from ._scalars import ScalarCacheMixin


class _ScaledBMM(ScalarCacheMixin, torch.nn.Module):
    _kernel = None  # name of the _CUDA entry point

    def __init__(self, alpha):
        super().__init__()
        self.register_buffer("a", torch.tensor(alpha))

    def forward(self, a, b):
        """a: int8 [B, M, K]; b: int8 [B, N, K]; returns [B, M, N].  (Integer inputs, outputs from
        torch.empty: nothing can require grad, so no torch.no_grad() context per call.)"""
        return getattr(_CUDA, self._kernel)(a, b, self._scalar("a"))

    @staticmethod
    def _as_tensor(alpha):
        return alpha if torch.is_tensor(alpha) else torch.tensor(alpha)


class BMM_S8T_S8N_S8T(_ScaledBMM):
    """int8 output: sat_s8(round(a * A.B^T))."""
    _kernel = "bmm_s8t_s8n_s8t"

    @staticmethod
    def from_scale(a_scale, b_scale, output_scale):
        mod = BMM_S8T_S8N_S8T(1.0)
        mod.a = _ScaledBMM._as_tensor(a_scale * b_scale / output_scale)
        return mod


class BMM_S8T_S8N_F32T(_ScaledBMM):
    """fp32 output: a * A.B^T."""
    _kernel = "bmm_s8t_s8n_f32t"

    @staticmethod
    def from_scale(a_scale, b_scale):
        mod = BMM_S8T_S8N_F32T(1.0)
        mod.a = _ScaledBMM._as_tensor(a_scale * b_scale)
        return mod


class BMM_S8T_S8N_S32T(torch.nn.Module):
    """int32 output: the raw accumulators."""

    def forward(self, a, b):
        return _CUDA.bmm_s8t_s8n_s32t(a, b)

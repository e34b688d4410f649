"""LayerNorm layers that emit int8 (upstream ``torch_int/nn/fused.py:5-43``)."""
import torch
import torch.nn.functional as F

from .. import _hip_ext
from ..functional.fused import dq_add_layernorm_q_cpp


class _QuantLayerNormBase(torch.nn.Module):
    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.input_scale = 1.0
        self.eps = eps
        self.register_buffer("weight", torch.ones(dim, dtype=torch.float32))
        self.register_buffer("bias", torch.zeros(dim, dtype=torch.float32))


class LayerNormQ(_QuantLayerNormBase):
    """fp -> int8: LayerNorm in fp32, round half-even, clamp to [-128, 127].
    ``from_float`` folds the output scale into weight and bias."""

    def forward(self, x, add=None):
        """int8 LayerNorm of ``x``.  With ``add`` given, ``x`` is first updated in place
        (``x.add_(add)``, the residual update of the decoder layer) -- fused into the same
        kernel when ``x`` is a contiguous fp32 or fp16 HIP tensor (an fp32 ``add`` on an fp16 ``x`` is rounded to
        fp16 first, as ``x.add_(add.to(x.dtype))`` does)."""
        if _hip_ext.can_fuse_layernorm(x, self.weight, self.bias) and (
                add is None or _hip_ext.can_fuse_layernorm_add(add, x)):
            return _hip_ext.add_layernorm_q(add, x, self.weight, self.bias, self.eps, checked=True)  # one pass, same maths
        if add is not None:
            x.add_(add.to(x.dtype))
        x = x.to(self.weight.dtype)  # upstream nn/fused.py:14: an fp16 input of an fp32 layer is promoted first
        if _hip_ext.can_fuse_layernorm(x, self.weight, self.bias):
            return _hip_ext.add_layernorm_q(None, x, self.weight, self.bias, self.eps, checked=True)
        y = F.layer_norm(x, x.shape[-1:], self.weight, self.bias, self.eps)
        return y.round().clamp(-128, 127).to(torch.int8)

    @staticmethod
    def from_float(module: torch.nn.LayerNorm, output_scale: float):
        dim = module.normalized_shape[0]
        assert dim == module.weight.numel() == module.bias.numel()
        q = LayerNormQ(dim, module.eps)
        q.weight = module.weight / output_scale
        q.bias = module.bias / output_scale
        return q


class DQ_Add_LayerNorm_Q(_QuantLayerNormBase):
    """(fp residual, int32 branch output) -> (new fp residual, int8 LayerNorm of it),
    one fused kernel.  Note the argument order: residual first."""

    def forward(self, residual_input_fp, input_int32):
        return dq_add_layernorm_q_cpp(input_int32, self.input_scale, residual_input_fp,
                                      self.weight, self.bias, self.eps)

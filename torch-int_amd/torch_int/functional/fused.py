"""Dequantise + residual add + LayerNorm (+ quantise) in three flavours
(upstream ``torch_int/functional/fused.py:5-25``): two compositions of stock
torch ops and the fused HIP kernel."""
import torch
import torch.nn.functional as F

from .._CUDA import dq_add_layernorm_q


def dq_add_layernorm(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    """(residual + scale*input, its LayerNorm) with stock torch ops, no quantisation."""
    summed = torch.add(residual_input_fp, input_int32, alpha=input_scale_fp)
    return summed, F.layer_norm(summed, summed.shape[-1:], gamma, beta, eps)


def dq_add_layernorm_q_py(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    """Stock-torch composition: clamp to [-128,127], round half-even, cast to int8."""
    summed, normed = dq_add_layernorm(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps)
    return summed, normed.clamp(-128, 127).round().to(torch.int8)


def dq_add_layernorm_q_cpp(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps):
    """The fused single-pass kernel."""
    return dq_add_layernorm_q(input_int32, input_scale_fp, residual_input_fp, gamma, beta, eps)

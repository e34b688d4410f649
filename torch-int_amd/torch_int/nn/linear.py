"""W8A8 linear layers (upstream ``torch_int/nn/linear.py:16-229``) and the two weight-only
layers ``W8A16Linear`` / ``W8FakeA8Linear`` (``:232-337``).

Every class keeps upstream's constructor signature, buffer names/shapes/dtypes
(``weight`` int8 [out, in], ``bias`` [1, out], 0-dim fp32 ``a``/``b``) and
``from_float`` algebra; ``forward`` flattens the leading dimensions, calls one
``torch_int._CUDA`` entry point and restores the shape.
"""
import torch

from .. import _CUDA, _hip_ext
from ..functional.quantization import (fake_quantize_activation_per_tensor_absmax,
                                       fake_quantize_activation_per_token_absmax,
                                       quantize_per_tensor_absmax, quantize_weight_per_channel_absmax)
from ._scalars import ScalarCacheMixin


class _W8A8Base(ScalarCacheMixin, torch.nn.Module):
    _bias_dtype = torch.int8

    def __init__(self, in_features, out_features):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        weight = torch.randint(-127, 127, (out_features, in_features), dtype=torch.int8)
        self.register_buffer("weight", weight)
        self.register_buffer("bias", torch.zeros((1, out_features), dtype=self._bias_dtype))

    def _register_scales(self, alpha, beta=None):
        self.register_buffer("a", torch.tensor(alpha))
        if beta is not None:
            self.register_buffer("b", torch.tensor(beta))

    def to(self, *args, **kwargs):
        # integer buffers must follow device moves but never a floating dtype cast
        super().to(*args, **kwargs)
        device = torch._C._nn._parse_to(*args, **kwargs)[0]
        if device is not None:
            self.weight = self.weight.to(device)
            self.bias = self.bias.to(device)
        return self

    def _run(self, x):
        raise NotImplementedError

    def _wb(self):
        """(weight, bias) without the cost of two nn.Module.__getattr__ calls; from_float may have left
        either as a Parameter (it assigns the float module's tensors), hence the fallback."""
        b = self._buffers
        w, bias = b.get("weight"), b.get("bias")
        return (w if w is not None else self.weight), (bias if bias is not None else self.bias)

    # No torch.no_grad() here (upstream decorates forward): the inputs are integer tensors and the outputs
    # come from torch.empty, so nothing can require grad, and the context manager costs a microsecond or two
    # on a path where a decode-sized kernel takes about five.
    def forward(self, x):
        if x.dim() == 2:
            return self._run(x)
        lead = x.shape[:-1]
        y = self._run(x.reshape(-1, x.shape[-1]))
        return y.view(*lead, -1)

    @staticmethod
    def _quantize_weight(module):
        return quantize_per_tensor_absmax(module.weight)


class W8A8B8O8Linear(_W8A8Base):
    """int8 in, int8 bias, int8 out (q/k/v projections)."""

    def __init__(self, in_features, out_features, alpha=1.0, beta=1.0):
        super().__init__(in_features, out_features)
        self._register_scales(alpha, beta)

    def _run(self, x):
        w, bias = self._wb()
        return _CUDA.linear_a8_w8_b8_o8(x, w, bias, self._scalar("a"), self._scalar("b"))

    @classmethod
    def from_float(cls, module, input_scale, output_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, w_scale = cls._quantize_weight(module)
        q.bias, b_scale = quantize_per_tensor_absmax(module.bias)
        q.a = input_scale * w_scale / output_scale
        q.b = b_scale / output_scale
        return q


class W8A8B8O8LinearReLU(W8A8B8O8Linear):
    """As W8A8B8O8Linear with a fused ReLU: outputs in [0, 127] (fc1)."""

    def _run(self, x):
        w, bias = self._wb()
        return _CUDA.linear_relu_a8_w8_b8_o8(x, w, bias, self._scalar("a"), self._scalar("b"))


class W8A8B32O32LinearWithoutScaling(_W8A8Base):
    """int8 in, int32 bias, raw int32 accumulators out."""
    _bias_dtype = torch.int32

    def _run(self, x):
        return _CUDA.linear_a8_w8_b32_o32(x, self.weight, self.bias)


class W8A8B32O32Linear(_W8A8Base):
    """int8 in, int32 bias, int32 out = round(a*acc + b*bias)."""
    _bias_dtype = torch.int32

    def __init__(self, in_features, out_features, alpha=1.0, beta=1.0):
        super().__init__(in_features, out_features)
        self._register_scales(alpha, beta)

    def _run(self, x):
        return _CUDA.linear_a8_w8_b32_o32_with_scaling(x, self.weight, self.bias, self._scalar("a"),
                                                       self._scalar("b"))

    @classmethod
    def from_float(cls, module, input_scale, output_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, w_scale = cls._quantize_weight(module)
        module.bias = module.bias.float()
        b_scale = module.bias.abs().max() / (2 ** 31 - 1)
        q.bias = (module.bias / b_scale).round().to(torch.int32)
        q.a = input_scale * w_scale / output_scale
        q.b = b_scale / output_scale
        q.input_scale, q.output_scale = input_scale, output_scale
        q.weight_scale, q.bias_scale = w_scale, b_scale
        return q


class W8A8BFP32OFP32Linear(_W8A8Base):
    """int8 in, fp32 bias, fp32 out = a*acc + bias (out_proj, fc2).  The bias
    stays fp32 through ``.half()`` / ``.to(dtype)``."""
    _bias_dtype = torch.float32

    def __init__(self, in_features, out_features, alpha=1.0, beta=1.0):
        super().__init__(in_features, out_features)
        self._register_scales(alpha)

    def _apply(self, fn, *args, **kwargs):
        super()._apply(fn, *args, **kwargs)
        self.bias = self.bias.to(torch.float32)
        return self

    def to(self, *args, **kwargs):
        super().to(*args, **kwargs)
        self.bias = self.bias.to(torch.float32)
        return self

    def _run(self, x):
        w, bias = self._wb()
        if bias.dtype != torch.float32:
            self.bias = bias = bias.to(torch.float32)
        return _CUDA.linear_a8_w8_bfp32_ofp32(x, w, bias, self._scalar("a"), 1)

    def forward(self, x, add_to=None):
        """``add_to`` (not in upstream): a contiguous fp32 tensor shaped like the output; the result is added
        into it in place by the GEMM epilogue (``add_to.add_(linear(x))`` without the intermediate) and
        ``add_to`` is returned.  Falls back to that expression when the tensor does not qualify."""
        if add_to is None:
            return super().forward(x)
        # Beyond a few thousand rows the GEMM takes its 256x256-tile kernel, whose read-modify-write epilogue
        # costs more than the separate add it saves (8192x5120x20480: 985 us against 936 us); below that the
        # fused form wins (2048x5120x20480: 209 against 223 us; 4 rows: one launch less).
        fits = (x.is_cuda and add_to.dtype is torch.float32 and add_to.is_contiguous() and add_to.device == x.device
                and add_to.shape == x.shape[:-1] + (self.out_features,) and add_to.numel() <= 4096 * self.out_features
                and hasattr(_CUDA, "_linear_a8_w8_bfp32_ofp32_acc"))
        if not fits:
            with torch.no_grad():
                y = super().forward(x)
                if (add_to.dtype is torch.float16 and y.is_cuda and add_to.is_contiguous() and add_to.shape == y.shape
                        and add_to.device == y.device):
                    return _hip_ext.add_rounded_(add_to, y)  # the cast and the add in one pass, same bits
                return add_to.add_(y.to(add_to.dtype))
        w, bias = self._wb()
        if bias.dtype != torch.float32:
            self.bias = bias = bias.to(torch.float32)
        _CUDA._linear_a8_w8_bfp32_ofp32_acc(x.reshape(-1, x.shape[-1]), w, bias, self._scalar("a"), 1, add_to)
        return add_to

    @classmethod
    def from_float(cls, module, input_scale):
        q = cls(module.in_features, module.out_features)
        q.weight, w_scale = cls._quantize_weight(module)
        q.bias = module.bias.to(torch.float32)
        q.a = input_scale * w_scale
        q.input_scale, q.weight_scale = input_scale, w_scale
        return q


class _W8FloatActivationBase(torch.nn.Module):
    """Shared part of the weight-only layers: int8 ``weight`` [out, in], fp16 ``bias`` [1, out] (or None)
    and fp16 ``weight_scales``; the forward pass dequantises the weight and runs a floating-point linear
    (upstream ``torch_int/nn/linear.py:232-337``).  These layers do not touch the INT8 kernels."""

    def __init__(self, in_features, out_features, bias=True):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.register_buffer("weight", torch.randint(-127, 127, (out_features, in_features), dtype=torch.int8))
        self.register_buffer("bias", torch.zeros((1, out_features), dtype=torch.float16) if bias else None)
        self.register_buffer("weight_scales", torch.ones(out_features, dtype=torch.float16))

    def to(self, *args, **kwargs):
        super().to(*args, **kwargs)
        device = torch._C._nn._parse_to(*args, **kwargs)[0]
        if device is not None:  # the int8 weight follows device moves, never a dtype cast
            self.weight = self.weight.to(device)
        return self

    def _dequantized_weight(self, dtype):
        w = self.weight.to(dtype)
        s = self.weight_scales.to(dtype)
        # one scale per output channel ([out] or [out, 1]) or a single per-tensor scale
        return w.mul_(s.reshape(-1, 1) if s.numel() == self.out_features else s.reshape(()))

    def _bias_for(self, x):
        return None if self.bias is None else self.bias.to(x.dtype).reshape(-1)

    def extra_repr(self):
        return f"{self.in_features}, {self.out_features}, bias={self.bias is not None}"


class W8A16Linear(_W8FloatActivationBase):
    """int8 weights, floating-point activations: y = x @ (weight * weight_scales)^T + bias."""

    @torch.no_grad()
    def forward(self, x):
        return torch.nn.functional.linear(x, self._dequantized_weight(x.dtype), self._bias_for(x))

    @staticmethod
    def from_float(module, weight_quant="per_channel"):
        assert isinstance(module, torch.nn.Linear)
        q = W8A16Linear(module.in_features, module.out_features, module.bias is not None)
        if weight_quant == "per_channel":
            q.weight, q.weight_scales = quantize_weight_per_channel_absmax(module.weight)
        elif weight_quant == "per_tensor":
            q.weight, q.weight_scales = quantize_per_tensor_absmax(module.weight)
        else:
            raise ValueError('weight_quant must be "per_channel" or "per_tensor"')
        if module.bias is not None:
            q.bias = module.bias.to(torch.float16)
        return q


class W8FakeA8Linear(_W8FloatActivationBase):
    """int8 weights, activations fake-quantised to the int8 grid (per token or per tensor) and kept in
    floating point: the accuracy-simulation layer.  The activation tensor is quantised in place."""

    def __init__(self, in_features, out_features, bias=True, act_quant="per_token"):
        super().__init__(in_features, out_features, bias)
        if act_quant == "per_token":
            self.activation_fake_quantizer = fake_quantize_activation_per_token_absmax
        elif act_quant == "per_tensor":
            self.activation_fake_quantizer = fake_quantize_activation_per_tensor_absmax
        else:
            raise ValueError('act_quant must be "per_token" or "per_tensor"')

    @torch.no_grad()
    def forward(self, x):
        w = self._dequantized_weight(x.dtype)
        x = self.activation_fake_quantizer(x)
        return torch.nn.functional.linear(x, w, self._bias_for(x))

    @staticmethod
    def from_float(module, act_quant="per_token"):
        assert isinstance(module, torch.nn.Linear)
        q = W8FakeA8Linear(module.in_features, module.out_features, module.bias is not None, act_quant)
        q.weight, q.weight_scales = quantize_weight_per_channel_absmax(module.weight)
        if module.bias is not None:
            q.bias = module.bias.to(torch.float16)
        return q

"""Per-tensor / per-channel / per-token absmax quantisers used by the
``from_float`` converters (upstream ``torch_int/functional/quantization.py``).

Like upstream, the in-place variants overwrite their argument (they exist to
convert large checkpoints without a second copy)."""
import torch

_EPS = 1e-8


def _as_float_on_cpu(t):
    # CPU has no half-precision rounding kernels
    return t if t.is_cuda else t.float()


@torch.no_grad()
def quantize_per_tensor_absmax(t):
    """-> (int8 tensor, 0-dim scale) with scale = max|t| / 127.  Overwrites ``t`` when it is fp32."""
    scale = t.abs().max() / 127
    t = _as_float_on_cpu(t)
    t.div_(scale).round_()
    return t.to(torch.int8), scale


@torch.no_grad()
def quantize_weight_per_channel_absmax(w):
    """w [out, in] -> (int8 [out, in], scales [out, 1]), one scale per output channel."""
    scales = (w.abs().max(dim=1)[0] / 127).view(-1, 1)
    w = _as_float_on_cpu(w)
    w.div_(scales).round_().clamp_(-128, 127)
    return w.to(torch.int8), scales


@torch.no_grad()
def dynamic_quantize_activation_per_tensor_zeropoint(t):
    """Asymmetric per-tensor quantisation -> (int8, scale, zero_point).  Shifts ``t`` in place."""
    hi, lo = t.max(), t.min()
    step = (hi - lo) / 254
    zp = ((hi + lo) / 2 / step).round() * step
    t -= zp
    scale = torch.clamp((hi - lo) / 2, min=_EPS) / 127
    return (t / scale).round().clamp(-128, 127).to(torch.int8), scale, zp


@torch.no_grad()
def dynamic_quantize_activation_per_tensor_absmax(t):
    scale = torch.clamp(t.abs().max(), min=_EPS) / 127
    return (t / scale).round().clamp(-128, 127).to(torch.int8), scale


@torch.no_grad()
def dynamic_quantize_activation_per_token_absmax(t):
    """One scale per row of the last dimension.  Overwrites ``t``."""
    scale = torch.clamp(t.abs().max(dim=-1, keepdim=True)[0], min=_EPS) / 127
    t.div_(scale).round_().clamp_(-128, 127)
    return t.to(torch.int8), scale


@torch.no_grad()
def fake_quantize_activation_per_tensor_absmax(t):
    scale = torch.clamp(t.abs().max(), min=_EPS) / 127
    return t.div_(scale).round_().clamp_(-128, 127).mul_(scale)


@torch.no_grad()
def fake_quantize_activation_per_token_absmax(t):
    scale = torch.clamp(t.abs().max(dim=-1, keepdim=True)[0], min=_EPS) / 127
    return t.div_(scale).round_().clamp_(-128, 127).mul_(scale)


@torch.no_grad()
def dequantize_activation_w_per_channel_a_per_token(q_act, w_scales, a_scales):
    """q_act [B, dim] * w_scales [dim] * a_scales [B, 1], returned in a_scales' dtype."""
    out = q_act.to(torch.float32)
    out.mul_(w_scales.reshape(1, -1)).mul_(a_scales.reshape(-1, 1))
    return out.to(a_scales.dtype)


@torch.no_grad()
def dequantize_activation_w_per_channel_a_per_tensor(q_act, w_scales, a_scales):
    """q_act [..., dim] * w_scales [dim] * a_scales [1], returned in a_scales' dtype."""
    out = q_act.to(torch.float32) * w_scales.reshape(1, -1) * a_scales
    return out.to(a_scales.dtype)

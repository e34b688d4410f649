"""``torch_int._CUDA``: the nine native INT8 entry points, on MI355X.

Mirrors the pybind11 module of upstream torch-int
(``torch_int/kernels/bindings.cpp:5-20``): same function names, positional
arguments and return types.  Each function validates its tensors, allocates the
output with torch, and hands raw device pointers plus the current HIP stream
to the C ABI of ``libtorch_int_hip.so`` (see ``include/torch_int_hip.h``).

There is no CPU implementation behind these functions: CPU tensors, a missing
library or a missing GPU raise instead of silently computing elsewhere.
"""
import ctypes
import os

import torch

__all__ = [
    "linear_a8_w8_b32_o32",
    "linear_a8_w8_b32_o32_with_scaling",
    "linear_a8_w8_bfp32_ofp32",
    "linear_a8_w8_b8_o8",
    "linear_relu_a8_w8_b8_o8",
    "bmm_s8t_s8n_f32t",
    "bmm_s8t_s8n_s8t",
    "bmm_s8t_s8n_s32t",
    "dq_add_layernorm_q",
]

# TORCH_INT_HIP_LIB points at another build of the same library (e.g. an experiment)
LIB_PATH = os.environ.get("TORCH_INT_HIP_LIB") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "lib", "libtorch_int_hip.so")

_vp, _i64, _f32, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int

# name -> argument types, in the order of include/torch_int_hip.h
_SIGNATURES = {
    "ti_linear_a8_w8_b32_o32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp],
    "ti_linear_a8_w8_b32_o32_with_scaling": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _vp, _i64, _vp],
    "ti_linear_a8_w8_bfp32_ofp32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _vp, _i64, _vp],
    "ti_linear_a8_w8_b8_o8": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _vp, _i64, _vp],
    "ti_linear_relu_a8_w8_b8_o8": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _vp, _i64, _vp],
    "ti_bmm_s8t_s8n_f32t": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp],
    "ti_bmm_s8t_s8n_s8t": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp],
    "ti_bmm_s8t_s8n_s32t": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "ti_dq_add_layernorm_q": [_vp, _f32, _vp, _vp, _vp, _f32, _vp, _vp, _i64, _i64, _vp],
}


def _load_library():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python torch-int_amd/build.py` "
            "(hipcc, --offload-arch=gfx950). torch_int has no fallback implementation.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _int
    lib.ti_last_error.restype = ctypes.c_char_p
    lib.ti_version.restype = _int
    lib.ti_init.restype = _int
    lib.ti_linear_workspace_bytes.argtypes = [_i64, _i64, _i64]
    lib.ti_linear_workspace_bytes.restype = _i64
    return lib


_lib = _load_library()
_workspaces = {}  # device index -> uint8 tensor used as split-K scratch


def _fail(op, msg):
    raise RuntimeError(f"torch_int._CUDA.{op}: {msg}")


def _check(op, name, t, dtype, ndim, device=None):
    if not isinstance(t, torch.Tensor):
        _fail(op, f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if t.dtype != dtype:
        _fail(op, f"{name} must be {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        _fail(op, f"{name} must be {ndim}-D, got shape {tuple(t.shape)}")
    if not t.is_cuda:
        _fail(op, f"{name} is on {t.device}; the INT8 kernels only run on a HIP (cuda) device")
    if device is not None and t.device != device:
        _fail(op, f"{name} is on {t.device}, expected {device}")
    if not t.is_contiguous():
        _fail(op, f"{name} must be contiguous (packed row-major), got strides {t.stride()}")


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _call(op, fn, device, *args):
    if device.index != torch.cuda.current_device():
        with torch.cuda.device(device):
            rc = fn(*args)
    else:
        rc = fn(*args)
    if rc != 0:
        _fail(op, f"{_lib.ti_last_error().decode()} (status {rc})")


def _workspace(device, nbytes):
    if nbytes <= 0:
        return None, 0
    ws = _workspaces.get(device.index)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=device)
        _workspaces[device.index] = ws
    return ws, ws.numel()


def _linear(op, fn, x, w, bias, bias_dtype, out_dtype, scalars):
    _check(op, "input", x, torch.int8, 2)
    dev = x.device
    _check(op, "weight", w, torch.int8, 2, dev)
    if not isinstance(bias, torch.Tensor):
        _fail(op, f"bias must be a torch.Tensor, got {type(bias).__name__}")
    if bias.device != dev:
        bias = bias.to(dev)  # upstream does bias.to(device) too (linear.cu:83)
    M, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K:
        _fail(op, f"input is [{M},{K}] but weight is {tuple(w.shape)}: inner dimensions differ")
    if bias.numel() != N:
        _fail(op, f"bias has {bias.numel()} elements, weight has {N} output rows")
    bias = bias.reshape(-1)
    _check(op, "bias", bias, bias_dtype, 1, dev)
    out = torch.empty((M, N), dtype=out_dtype, device=dev)
    if M == 0 or N == 0:
        return out
    ws, ws_bytes = _workspace(dev, _lib.ti_linear_workspace_bytes(M, N, K))
    _call(op, fn, dev, x.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), M, N, K, *scalars,
          ws.data_ptr() if ws is not None else None, ws_bytes, _stream(dev))
    return out


def linear_a8_w8_b32_o32(input, weight, bias):
    """int32 [M,N] = input[M,K] . weight[N,K]^T + bias[N]  (upstream linear.cu:13-136)."""
    return _linear("linear_a8_w8_b32_o32", _lib.ti_linear_a8_w8_b32_o32, input, weight, bias,
                   torch.int32, torch.int32, ())


def linear_a8_w8_b32_o32_with_scaling(input, weight, bias, alpha, beta):
    """int32 [M,N] = sat(round(alpha*acc + beta*bias))  (upstream linear.cu:139-243)."""
    return _linear("linear_a8_w8_b32_o32_with_scaling", _lib.ti_linear_a8_w8_b32_o32_with_scaling,
                   input, weight, bias, torch.int32, torch.int32, (float(alpha), float(beta)))


def linear_a8_w8_bfp32_ofp32(input, weight, bias, alpha, beta):
    """fp32 [M,N] = alpha*acc + beta*bias, fp32 bias  (upstream linear.cu:246-365)."""
    return _linear("linear_a8_w8_bfp32_ofp32", _lib.ti_linear_a8_w8_bfp32_ofp32, input, weight, bias,
                   torch.float32, torch.float32, (float(alpha), float(beta)))


def linear_a8_w8_b8_o8(input, weight, bias, alpha, beta):
    """int8 [M,N] = sat_s8(round(alpha*acc + beta*bias)), int8 bias  (upstream linear.cu:369-473)."""
    return _linear("linear_a8_w8_b8_o8", _lib.ti_linear_a8_w8_b8_o8, input, weight, bias,
                   torch.int8, torch.int8, (float(alpha), float(beta)))


def linear_relu_a8_w8_b8_o8(input, weight, bias, alpha, beta):
    """int8 [M,N] in [0,127] = sat_s8(round(relu(alpha*acc + beta*bias)))  (upstream linear.cu:476-625)."""
    return _linear("linear_relu_a8_w8_b8_o8", _lib.ti_linear_relu_a8_w8_b8_o8, input, weight, bias,
                   torch.int8, torch.int8, (float(alpha), float(beta)))


def _bmm(op, fn, a, b, out_dtype, scalars):
    _check(op, "A", a, torch.int8, 3)
    dev = a.device
    _check(op, "B", b, torch.int8, 3, dev)
    batch, M, K = a.shape
    if b.shape[0] != batch or b.shape[2] != K:
        _fail(op, f"A is {tuple(a.shape)} and B is {tuple(b.shape)}: batch and inner dimensions must match")
    N = b.shape[1]
    out = torch.empty((batch, M, N), dtype=out_dtype, device=dev)
    if out.numel() == 0:
        return out
    _call(op, fn, dev, a.data_ptr(), b.data_ptr(), out.data_ptr(), batch, M, N, K, *scalars, _stream(dev))
    return out


def bmm_s8t_s8n_f32t(A, B, alpha):
    """fp32 [B,M,N] = alpha * (A[B,M,K] . B[B,N,K]^T)  (upstream bmm.cu:10-108)."""
    return _bmm("bmm_s8t_s8n_f32t", _lib.ti_bmm_s8t_s8n_f32t, A, B, torch.float32, (float(alpha),))


def bmm_s8t_s8n_s8t(A, B, alpha):
    """int8 [B,M,N] = sat_s8(round(alpha * (A . B^T)))  (upstream bmm.cu:110-208)."""
    return _bmm("bmm_s8t_s8n_s8t", _lib.ti_bmm_s8t_s8n_s8t, A, B, torch.int8, (float(alpha),))


def bmm_s8t_s8n_s32t(A, B):
    """int32 [B,M,N] = A . B^T  (upstream bmm.cu:210-295)."""
    return _bmm("bmm_s8t_s8n_s32t", _lib.ti_bmm_s8t_s8n_s32t, A, B, torch.int32, ())


def dq_add_layernorm_q(input, input_scale, residual_input, gamma, beta, epsilon):
    """(residual_output fp32, ln_output int8)  (upstream fused.cu:5-25).

    residual_output = residual_input + input_scale * input;
    ln_output = int8(round(clamp(layer_norm(residual_output) * gamma + beta, -128, 127))).
    """
    op = "dq_add_layernorm_q"
    _check(op, "input", input, torch.int32, None)
    dev = input.device
    if input.dim() < 1:
        _fail(op, "input must have at least one dimension")
    _check(op, "residual_input", residual_input, torch.float32, None, dev)
    if residual_input.shape != input.shape:
        _fail(op, f"input is {tuple(input.shape)} but residual_input is {tuple(residual_input.shape)}")
    H = input.shape[-1]
    gamma = gamma.detach() if isinstance(gamma, torch.Tensor) else gamma
    beta = beta.detach() if isinstance(beta, torch.Tensor) else beta
    _check(op, "gamma", gamma, torch.float32, 1, dev)
    _check(op, "beta", beta, torch.float32, 1, dev)
    if gamma.numel() != H or beta.numel() != H:
        _fail(op, f"gamma/beta must have {H} elements, got {gamma.numel()} and {beta.numel()}")
    r_out = torch.empty_like(residual_input)
    q_out = torch.empty(input.shape, dtype=torch.int8, device=dev)
    if input.numel() == 0:
        return r_out, q_out
    _call(op, _lib.ti_dq_add_layernorm_q, dev, input.data_ptr(), float(input_scale), residual_input.data_ptr(),
          gamma.data_ptr(), beta.data_ptr(), float(epsilon), r_out.data_ptr(), q_out.data_ptr(),
          input.numel() // H, H, _stream(dev))
    return r_out, q_out

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
import weakref

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
    "ti_linear_a8_w8_bfp32_ofp32_acc": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _vp, _i64, _vp],
    "ti_linear_relu_a8_w8_b8_o8": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _vp, _i64, _vp],
    "ti_bmm_s8t_s8n_f32t": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp],
    "ti_bmm_s8t_s8n_s8t": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp],
    "ti_bmm_s8t_s8n_s32t": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp],
    "ti_bmm_s8t_s8n_f32t_ws": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp, _i64, _vp],
    "ti_bmm_s8t_s8n_s8t_ws": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp, _i64, _vp],
    "ti_bmm_s8t_s8n_s32t_ws": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _vp],
    "ti_dq_add_layernorm_q": [_vp, _f32, _vp, _vp, _vp, _f32, _vp, _vp, _i64, _i64, _vp],
    "ti_dq_add_layernorm_q_f16": [_vp, _f32, _vp, _vp, _vp, _f32, _vp, _vp, _i64, _i64, _vp],
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
    lib.ti_bmm_workspace_bytes.argtypes = [_i64, _i64, _i64, _i64]
    lib.ti_bmm_workspace_bytes.restype = _i64
    return lib


_lib = _load_library()


def _load_fastcall():
    """The optional CPython forwarder built next to the library (csrc/fastcall.c).  It calls the
    same C ABI; without it the calls go through ctypes, a few microseconds slower each."""
    if os.environ.get("TORCH_INT_HIP_LIB"):
        return None  # the forwarder is linked against the default library
    import glob
    import importlib.util
    hits = glob.glob(os.path.join(os.path.dirname(LIB_PATH), "_ti_fastcall*.so"))
    if not hits:
        return None
    try:
        spec = importlib.util.spec_from_file_location("_ti_fastcall", hits[0])
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        return mod
    except Exception:  # pragma: no cover - e.g. built for another interpreter
        return None


_fast = _load_fastcall()
_workspaces = {}  # (device index, stream) -> uint8 tensor used as split-K scratch
_raw_stream = torch._C._cuda_getCurrentRawStream
_current_device = torch.cuda.current_device
_empty = torch.empty
_I8, _I32, _F32 = torch.int8, torch.int32, torch.float32

# kind codes shared with csrc/ti_common.h (EpiKind) and csrc/fastcall.c
_K_B32, _K_B32S, _K_F32, _K_S8, _K_RELU, _K_BMM_F32, _K_BMM_S8, _K_BMM_S32, _K_F32_ACC = range(9)
_LINEAR_CTYPES = {_K_B32: _lib.ti_linear_a8_w8_b32_o32, _K_B32S: _lib.ti_linear_a8_w8_b32_o32_with_scaling,
                  _K_F32: _lib.ti_linear_a8_w8_bfp32_ofp32, _K_S8: _lib.ti_linear_a8_w8_b8_o8,
                  _K_RELU: _lib.ti_linear_relu_a8_w8_b8_o8, _K_F32_ACC: _lib.ti_linear_a8_w8_bfp32_ofp32_acc}
_BMM_CTYPES = {_K_BMM_F32: _lib.ti_bmm_s8t_s8n_f32t, _K_BMM_S8: _lib.ti_bmm_s8t_s8n_s8t,
               _K_BMM_S32: _lib.ti_bmm_s8t_s8n_s32t}
_BMM_WS_CTYPES = {_K_BMM_F32: _lib.ti_bmm_s8t_s8n_f32t_ws, _K_BMM_S8: _lib.ti_bmm_s8t_s8n_s8t_ws,
                  _K_BMM_S32: _lib.ti_bmm_s8t_s8n_s32t_ws}


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


def _status(op, rc):
    if rc != 0:
        msg = _fast.last_error() if _fast is not None else _lib.ti_last_error().decode()
        _fail(op, f"{msg} (status {rc})")


_ws_need = {}  # (M, N, K) -> bytes of workspace the library can use for that linear


def _ws_bytes(M, N, K):
    key = (M, N, K)
    n = _ws_need.get(key)
    if n is None:
        n = _ws_need[key] = int(_lib.ti_linear_workspace_bytes(M, N, K))
    return n


_bmm_ws_need = {}  # (batch, M, N, K) -> bytes of workspace the library can use for that batched product


def _bmm_ws_bytes(batch, M, N, K):
    key = (batch, M, N, K)
    n = _bmm_ws_need.get(key)
    if n is None:
        n = _bmm_ws_need[key] = int(_lib.ti_bmm_workspace_bytes(batch, M, N, K))
    return n


def _workspace(dev_index, stream, nbytes):
    """Split-K scratch (int32 partial tiles; contents need no initialisation).  One buffer per
    (device, stream), grown on demand, so that calls on different streams never share it."""
    if nbytes <= 0:
        return 0, 0
    key = (dev_index, stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=torch.device("cuda", dev_index))
        _workspaces[key] = ws
    return ws.data_ptr(), ws.numel()


def _pad_inner(a, b, K, macs, weight=False):
    """Operands whose inner dimension is not a multiple of 16 have no aligned rows for the tiled kernels, and the
    library then runs a one-thread-per-output kernel (40 x 1500 x 128 x 1500: 32 ms).  From a size at which that
    hurts, both operands are copied with K padded by zeros to a multiple of 64 first: the added products are zero,
    the results the same (upstream rejects such shapes: "cutlass cannot implement")."""
    if K % 16 == 0 or macs < (1 << 26):
        return a, b, K
    pad = -K % 64
    return torch.nn.functional.pad(a, (0, pad)), _padded_weight(b, pad) if weight else torch.nn.functional.pad(b, (0, pad)), K + pad


_padded = {}  # id(weight) -> (weak reference, version counter, padded copy)


def _padded_weight(w, pad):
    """The zero-padded copy of a linear's weight, made once per weight tensor and version (a module calls with the
    same tensor object every time) instead of once per forward.  Entries go when their tensor does."""
    key = id(w)
    hit = _padded.get(key)
    if hit is not None and hit[0]() is w and hit[1] == w._version and hit[2].shape[1] == w.shape[1] + pad:
        return hit[2]
    if len(_padded) >= 256:
        _padded.clear()
    padded = torch.nn.functional.pad(w, (0, pad))
    _padded[key] = (weakref.ref(w, lambda _r, k=key: _padded.pop(k, None)), w._version, padded)
    return padded


def _linear(op, kind, x, w, bias, bias_dtype, out_dtype, alpha, beta, inout=None):
    # fast accept path first; the slow path below names what is wrong
    if not (type(x) is torch.Tensor and type(w) is torch.Tensor and x.dtype is _I8 and w.dtype is _I8
            and x.dim() == 2 and w.dim() == 2 and x.is_cuda and w.device == x.device
            and x.is_contiguous() and w.is_contiguous()):
        _check(op, "input", x, _I8, 2)
        _check(op, "weight", w, _I8, 2, x.device)
    dev = x.device
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
    if bias.dtype is not bias_dtype:
        _fail(op, f"bias must be {bias_dtype}, got {bias.dtype}")
    if not bias.is_contiguous():
        bias = bias.contiguous()
    if inout is None:
        out = _empty((M, N), dtype=out_dtype, device=dev)
    else:  # the accumulate-into-output variant writes where the caller says
        out = inout
        if not (type(out) is torch.Tensor and out.dtype is out_dtype and out.device == dev and out.is_contiguous()
                and out.numel() == M * N and out.dim() >= 1 and out.shape[-1] == N):
            _fail(op, f"the tensor to add into must be a contiguous {out_dtype} tensor of {M}x{N} elements on {dev}")
    if M == 0 or N == 0:
        return out
    x, w, K = _pad_inner(x, w, K, M * N * K, weight=True)
    idx = dev.index
    switch = idx != _current_device()
    if switch:
        prev = _current_device()
        torch.cuda.set_device(idx)
    try:
        stream = _raw_stream(idx)
        # split-K scratch is only ever wanted for mid-sized M (see choose_splits in csrc/gemm_s8.hip)
        ws_ptr, ws_bytes = _workspace(idx, stream, _ws_bytes(M, N, K)) if M > 16 else (0, 0)
        if _fast is not None:
            rc = _fast.linear(kind, x.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), M, N, K,
                              alpha, beta, ws_ptr, ws_bytes, stream)
        else:
            scal = () if kind == _K_B32 else (alpha, beta)
            rc = _LINEAR_CTYPES[kind](x.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), M, N, K, *scal,
                                      ws_ptr or None, ws_bytes, stream or None)
    finally:
        if switch:
            torch.cuda.set_device(prev)
    if rc:
        _status(op, rc)
    return out


def linear_a8_w8_b32_o32(input, weight, bias):
    """int32 [M,N] = input[M,K] . weight[N,K]^T + bias[N]  (upstream linear.cu:13-136)."""
    return _linear("linear_a8_w8_b32_o32", _K_B32, input, weight, bias, _I32, _I32, 1.0, 1.0)


def linear_a8_w8_b32_o32_with_scaling(input, weight, bias, alpha, beta):
    """int32 [M,N] = sat(round(alpha*acc + beta*bias))  (upstream linear.cu:139-243)."""
    return _linear("linear_a8_w8_b32_o32_with_scaling", _K_B32S, input, weight, bias, _I32, _I32,
                   float(alpha), float(beta))


def linear_a8_w8_bfp32_ofp32(input, weight, bias, alpha, beta):
    """fp32 [M,N] = alpha*acc + beta*bias, fp32 bias  (upstream linear.cu:246-365)."""
    return _linear("linear_a8_w8_bfp32_ofp32", _K_F32, input, weight, bias, _F32, _F32, float(alpha), float(beta))


def _linear_a8_w8_bfp32_ofp32_acc(input, weight, bias, alpha, beta, inout):
    """inout += alpha*acc + beta*bias, in place (no counterpart upstream; used by the OPT decoder layer for
    ``residual.add_(fc2(x))``).  Returns ``inout``."""
    return _linear("linear_a8_w8_bfp32_ofp32_acc", _K_F32_ACC, input, weight, bias, _F32, _F32, float(alpha),
                   float(beta), inout)


def linear_a8_w8_b8_o8(input, weight, bias, alpha, beta):
    """int8 [M,N] = sat_s8(round(alpha*acc + beta*bias)), int8 bias  (upstream linear.cu:369-473)."""
    return _linear("linear_a8_w8_b8_o8", _K_S8, input, weight, bias, _I8, _I8, float(alpha), float(beta))


def linear_relu_a8_w8_b8_o8(input, weight, bias, alpha, beta):
    """int8 [M,N] in [0,127] = sat_s8(round(relu(alpha*acc + beta*bias)))  (upstream linear.cu:476-625)."""
    return _linear("linear_relu_a8_w8_b8_o8", _K_RELU, input, weight, bias, _I8, _I8, float(alpha), float(beta))


def _bmm(op, kind, a, b, out_dtype, alpha):
    _check(op, "A", a, _I8, 3)
    dev = a.device
    _check(op, "B", b, _I8, 3, dev)
    batch, M, K = a.shape
    if b.shape[0] != batch or b.shape[2] != K:
        _fail(op, f"A is {tuple(a.shape)} and B is {tuple(b.shape)}: batch and inner dimensions must match")
    N = b.shape[1]
    out = _empty((batch, M, N), dtype=out_dtype, device=dev)
    if out.numel() == 0:
        return out
    a, b, K = _pad_inner(a, b, K, batch * M * N * K)
    idx = dev.index
    switch = idx != _current_device()
    if switch:
        prev = _current_device()
        torch.cuda.set_device(idx)
    try:
        stream = _raw_stream(idx)
        # few output tiles and a long inner dimension (never an attention product): split-K with a workspace
        need = _bmm_ws_bytes(batch, M, N, K) if K >= 1024 and M > 16 else 0
        if need:
            ws_ptr, ws_bytes = _workspace(idx, stream, need)
            scal = () if kind == _K_BMM_S32 else (alpha,)
            rc = _BMM_WS_CTYPES[kind](a.data_ptr(), b.data_ptr(), out.data_ptr(), batch, M, N, K, *scal, ws_ptr, ws_bytes,
                                      stream or None)
        elif _fast is not None:
            rc = _fast.bmm(kind, a.data_ptr(), b.data_ptr(), out.data_ptr(), batch, M, N, K, alpha, stream)
        else:
            scal = () if kind == _K_BMM_S32 else (alpha,)
            rc = _BMM_CTYPES[kind](a.data_ptr(), b.data_ptr(), out.data_ptr(), batch, M, N, K, *scal, stream or None)
    finally:
        if switch:
            torch.cuda.set_device(prev)
    if rc:
        _status(op, rc)
    return out


def bmm_s8t_s8n_f32t(A, B, alpha):
    """fp32 [B,M,N] = alpha * (A[B,M,K] . B[B,N,K]^T)  (upstream bmm.cu:10-108)."""
    return _bmm("bmm_s8t_s8n_f32t", _K_BMM_F32, A, B, _F32, float(alpha))


def bmm_s8t_s8n_s8t(A, B, alpha):
    """int8 [B,M,N] = sat_s8(round(alpha * (A . B^T)))  (upstream bmm.cu:110-208)."""
    return _bmm("bmm_s8t_s8n_s8t", _K_BMM_S8, A, B, _I8, float(alpha))


def bmm_s8t_s8n_s32t(A, B):
    """int32 [B,M,N] = A . B^T  (upstream bmm.cu:210-295)."""
    return _bmm("bmm_s8t_s8n_s32t", _K_BMM_S32, A, B, _I32, 1.0)


def dq_add_layernorm_q(input, input_scale, residual_input, gamma, beta, epsilon):
    """(residual_output, ln_output int8)  (upstream fused.cu:5-25).

    residual_output = residual_input + input_scale * input;
    ln_output = int8(round(clamp(layer_norm(residual_output) * gamma + beta, -128, 127))).
    residual_input, gamma and beta are fp32, or all three fp16 (as upstream's benchmark/bench_dq_add_ln_q.py:37-45
    calls it); residual_output has the residual's dtype.  With fp16 the arithmetic is fp32 and rounds to fp16 where
    upstream's chain of ATen ops does (the updated residual, the LayerNorm output).
    """
    op = "dq_add_layernorm_q"
    _check(op, "input", input, _I32, None)
    dev = input.device
    if input.dim() < 1:
        _fail(op, "input must have at least one dimension")
    fdt = residual_input.dtype if isinstance(residual_input, torch.Tensor) else None
    if fdt is not torch.float16:
        fdt = _F32
    _check(op, "residual_input", residual_input, fdt, None, dev)
    if residual_input.shape != input.shape:
        _fail(op, f"input is {tuple(input.shape)} but residual_input is {tuple(residual_input.shape)}")
    H = input.shape[-1]
    gamma = gamma.detach() if isinstance(gamma, torch.Tensor) else gamma
    beta = beta.detach() if isinstance(beta, torch.Tensor) else beta
    for name, t in (("gamma", gamma), ("beta", beta)):
        if isinstance(t, torch.Tensor) and t.dtype is not fdt and t.dtype in (_F32, torch.float16):
            _fail(op, f"{name} is {t.dtype} but residual_input is {fdt}: residual_input, gamma and beta must share one "
                      "dtype (float32 or float16)")
    _check(op, "gamma", gamma, fdt, 1, dev)
    _check(op, "beta", beta, fdt, 1, dev)
    if gamma.numel() != H or beta.numel() != H:
        _fail(op, f"gamma/beta must have {H} elements, got {gamma.numel()} and {beta.numel()}")
    r_out = torch.empty_like(residual_input)
    q_out = _empty(input.shape, dtype=_I8, device=dev)
    if input.numel() == 0:
        return r_out, q_out
    idx = dev.index
    switch = idx != _current_device()
    if switch:
        prev = _current_device()
        torch.cuda.set_device(idx)
    try:
        stream = _raw_stream(idx)
        args = (input.data_ptr(), float(input_scale), residual_input.data_ptr(), gamma.data_ptr(), beta.data_ptr(),
                float(epsilon), r_out.data_ptr(), q_out.data_ptr(), input.numel() // H, H)
        if fdt is torch.float16:
            rc = _lib.ti_dq_add_layernorm_q_f16(*args, stream or None)
        else:
            rc = _fast.ln_q(*args, stream) if _fast is not None else _lib.ti_dq_add_layernorm_q(*args, stream or None)
    finally:
        if switch:
            torch.cuda.set_device(prev)
    if rc:
        _status(op, rc)
    return r_out, q_out

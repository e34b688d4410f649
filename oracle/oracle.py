"""TEST INFRASTRUCTURE ONLY: Python face of the CPU oracle (``ti_oracle.c``).

Only tests, ``__graft_entry__.smoke()`` and the CPU-baseline leg of ``bench.py``
may import this module.  The shipped package never does.

Every function takes CPU tensors and returns new CPU tensors with the same
positional signature as the ``torch_int._CUDA`` entry point of the same name
(upstream ``torch_int/kernels/bindings.cpp:5-20``).
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libti_oracle.so")
_lib = None


def build(force=False):
    """Compile ``ti_oracle.c`` with gcc (see the Makefile beside it)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libti_oracle.so"])


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def num_threads():
    return int(_load().orc_num_threads())


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _i64(v):
    return ctypes.c_int64(int(v))


def _f32(v):
    # pybind11 narrows a Python float to C float at the call boundary
    # (upstream bindings.cpp); np.float32() is the same round-to-nearest.
    return ctypes.c_float(float(np.float32(v)))


def _chk(t, dtype, name):
    assert t.device.type == "cpu", f"{name}: oracle takes CPU tensors"
    assert t.dtype == dtype, f"{name}: expected {dtype}, got {t.dtype}"
    return t.contiguous()


def gemm_acc(a, b):
    """int32 accumulators of A . B^T.  a: [M,K] or [B,M,K]; b: [N,K] or [B,N,K]."""
    a = _chk(a, torch.int8, "a")
    b = _chk(b, torch.int8, "b")
    if a.dim() == 2:
        batch, (M, K), N = 1, a.shape, b.shape[0]
        out = torch.empty((M, N), dtype=torch.int32)
    else:
        batch, M, K = a.shape
        N = b.shape[1]
        out = torch.empty((batch, M, N), dtype=torch.int32)
    assert b.shape[-1] == K
    _load().orc_gemm_s8_acc(_p(a), _p(b), _p(out), _i64(batch), _i64(M), _i64(N), _i64(K))
    return out


def gemm_acc_naive64(a, b):
    a = _chk(a, torch.int8, "a")
    b = _chk(b, torch.int8, "b")
    if a.dim() == 2:
        a3, b3 = a[None], b[None]
    else:
        a3, b3 = a, b
    batch, M, K = a3.shape
    N = b3.shape[1]
    out = torch.empty((batch, M, N), dtype=torch.int64)
    _load().orc_gemm_s8_acc_naive64(_p(a3.contiguous()), _p(b3.contiguous()), _p(out),
                                    _i64(batch), _i64(M), _i64(N), _i64(K))
    return out if a.dim() == 3 else out[0]


def gemm_acc_torch(a, b):
    """The reference's CPU integer emulation: torch int32 matmul."""
    return torch.matmul(a.to(torch.int32), b.to(torch.int32).transpose(-1, -2))


# ---- epilogues on a ready accumulator (used with either accumulation route) ----

def epi_b32_o32(acc, bias):
    acc = _chk(acc, torch.int32, "acc")
    bias = _chk(bias.reshape(-1), torch.int32, "bias")
    out = torch.empty_like(acc)
    N = acc.shape[-1]
    _load().orc_epi_b32_o32(_p(acc), _p(bias), _p(out), _i64(acc.numel() // N), _i64(N))
    return out


def epi_b32_o32_scaled(acc, bias, alpha, beta):
    acc = _chk(acc, torch.int32, "acc")
    bias = _chk(bias.reshape(-1), torch.int32, "bias")
    out = torch.empty_like(acc)
    N = acc.shape[-1]
    _load().orc_epi_b32_o32_scaled(_p(acc), _p(bias), _p(out), _i64(acc.numel() // N), _i64(N),
                                   _f32(alpha), _f32(beta))
    return out


def epi_bfp32_ofp32(acc, bias, alpha, beta):
    acc = _chk(acc, torch.int32, "acc")
    bias = _chk(bias.reshape(-1), torch.float32, "bias")
    out = torch.empty(acc.shape, dtype=torch.float32)
    N = acc.shape[-1]
    _load().orc_epi_bfp32_ofp32(_p(acc), _p(bias), _p(out), _i64(acc.numel() // N), _i64(N),
                                _f32(alpha), _f32(beta))
    return out


def epi_b8_o8(acc, bias, alpha, beta, relu=False):
    acc = _chk(acc, torch.int32, "acc")
    bias = _chk(bias.reshape(-1), torch.int8, "bias")
    out = torch.empty(acc.shape, dtype=torch.int8)
    N = acc.shape[-1]
    fn = _load().orc_epi_relu_b8_o8 if relu else _load().orc_epi_b8_o8
    fn(_p(acc), _p(bias), _p(out), _i64(acc.numel() // N), _i64(N), _f32(alpha), _f32(beta))
    return out


def epi_f32t(acc, alpha):
    acc = _chk(acc, torch.int32, "acc")
    out = torch.empty(acc.shape, dtype=torch.float32)
    _load().orc_epi_f32t(_p(acc), _p(out), _i64(acc.numel()), _f32(alpha))
    return out


def epi_s8t(acc, alpha):
    acc = _chk(acc, torch.int32, "acc")
    out = torch.empty(acc.shape, dtype=torch.int8)
    _load().orc_epi_s8t(_p(acc), _p(out), _i64(acc.numel()), _f32(alpha))
    return out


# ---- the nine entry points ----

def linear_a8_w8_b32_o32(x, w, bias, acc_fn=gemm_acc):
    return epi_b32_o32(acc_fn(x, w), bias)


def linear_a8_w8_b32_o32_with_scaling(x, w, bias, alpha, beta, acc_fn=gemm_acc):
    return epi_b32_o32_scaled(acc_fn(x, w), bias, alpha, beta)


def linear_a8_w8_bfp32_ofp32(x, w, bias, alpha, beta, acc_fn=gemm_acc):
    return epi_bfp32_ofp32(acc_fn(x, w), bias, alpha, beta)


def linear_a8_w8_b8_o8(x, w, bias, alpha, beta, acc_fn=gemm_acc):
    return epi_b8_o8(acc_fn(x, w), bias, alpha, beta)


def linear_relu_a8_w8_b8_o8(x, w, bias, alpha, beta, acc_fn=gemm_acc):
    return epi_b8_o8(acc_fn(x, w), bias, alpha, beta, relu=True)


def bmm_s8t_s8n_f32t(a, b, alpha, acc_fn=gemm_acc):
    return epi_f32t(acc_fn(a, b), alpha)


def bmm_s8t_s8n_s8t(a, b, alpha, acc_fn=gemm_acc):
    return epi_s8t(acc_fn(a, b), alpha)


def bmm_s8t_s8n_s32t(a, b, acc_fn=gemm_acc):
    return acc_fn(a, b)


def dq_add_layernorm_q(inp, input_scale, residual, gamma, beta, eps):
    inp = _chk(inp, torch.int32, "input")
    residual = _chk(residual, torch.float32, "residual")
    gamma = _chk(gamma, torch.float32, "gamma")
    beta = _chk(beta, torch.float32, "beta")
    H = inp.shape[-1]
    assert residual.shape == inp.shape and gamma.numel() == H and beta.numel() == H
    r = torch.empty(inp.shape, dtype=torch.float32)
    q = torch.empty(inp.shape, dtype=torch.int8)
    rows = inp.numel() // H if H else 0
    _load().orc_dq_add_layernorm_q(_p(inp), _f32(input_scale), _p(residual), _p(gamma), _p(beta),
                                   _f32(eps), _p(r), _p(q), _i64(rows), _i64(H))
    return r, q


def _ln_f16(mode, inp, scale, residual, gamma, beta, eps):
    residual = _chk(residual, torch.float16, "residual")
    gamma = _chk(gamma, torch.float16, "gamma")
    beta = _chk(beta, torch.float16, "beta")
    H = residual.shape[-1]
    rows = residual.numel() // H if H else 0
    assert gamma.numel() == H and beta.numel() == H
    r = torch.empty_like(residual)
    q = torch.empty(residual.shape, dtype=torch.int8)
    _load().orc_layernorm_q_f16(ctypes.c_int(mode), _p(inp) if inp is not None else None, _f32(scale), _p(residual),
                                _p(gamma), _p(beta), _f32(eps), _p(r), _p(q), _i64(rows), _i64(H))
    return r, q


def dq_add_layernorm_q_f16(inp, input_scale, residual, gamma, beta, eps):
    """dq_add_layernorm_q on fp16 residual / gamma / beta: (fp16 residual output, int8)."""
    inp = _chk(inp, torch.int32, "input")
    assert inp.shape == residual.shape
    return _ln_f16(0, inp, input_scale, residual, gamma, beta, eps)


def add_layernorm_q_f16(x, residual, gamma, beta, eps):
    """add_layernorm_q on fp16 tensors; x may be None, or fp32 (then it is rounded to fp16 before the add)."""
    if x is None:
        return _ln_f16(2, None, 1.0, residual, gamma, beta, eps)
    if x.dtype is torch.float32:
        x = _chk(x, torch.float32, "x")
        assert x.shape == residual.shape
        return _ln_f16(3, x, 1.0, residual, gamma, beta, eps)
    x = _chk(x, torch.float16, "x")
    assert x.shape == residual.shape
    return _ln_f16(1, x, 1.0, residual, gamma, beta, eps)


def f16_round_trip(x):
    """fp32 tensor -> (uint16 bit patterns of the oracle's fp16 conversion, and their fp32 values)."""
    x = _chk(x, torch.float32, "x")
    lib = _load()
    lib.orc_f16_of_f32.restype = ctypes.c_uint16
    lib.orc_f16_of_f32.argtypes = [ctypes.c_float]
    lib.orc_f32_of_f16.restype = ctypes.c_float
    lib.orc_f32_of_f16.argtypes = [ctypes.c_uint16]
    bits = [lib.orc_f16_of_f32(float(v)) for v in x.reshape(-1).tolist()]
    back = [lib.orc_f32_of_f16(b) for b in bits]
    return torch.tensor(bits, dtype=torch.int32), torch.tensor(back, dtype=torch.float32)


# ---- fused chains of the OPT blocks (ti_add_layernorm_q / ti_attn_softmax_q) ----

def add_layernorm_q(x, residual, gamma, beta, eps):
    """(updated residual, int8 LayerNorm of it); x may be None (no add; residual returned as is)."""
    residual = _chk(residual, torch.float32, "residual")
    gamma = _chk(gamma, torch.float32, "gamma")
    beta = _chk(beta, torch.float32, "beta")
    H = residual.shape[-1]
    rows = residual.numel() // H if H else 0
    q = torch.empty(residual.shape, dtype=torch.int8)
    if x is None:
        _load().orc_add_layernorm_q(None, _p(residual), _p(gamma), _p(beta), _f32(eps), None, _p(q),
                                    _i64(rows), _i64(H))
        return residual, q
    x = _chk(x, torch.float32, "x")
    assert x.shape == residual.shape
    r = torch.empty_like(residual)
    _load().orc_add_layernorm_q(_p(x), _p(residual), _p(gamma), _p(beta), _f32(eps), _p(r), _p(q), _i64(rows), _i64(H))
    return r, q


def attn_softmax_q(scores, mask, heads):
    """int8 round(127 softmax(max(scores + mask, finfo.min))); scores [batch*heads, T, S], mask [batch,1,T,S] or None."""
    scores = _chk(scores, torch.float32, "scores")
    BH, T, S = scores.shape
    batch = BH // heads
    assert batch * heads == BH
    out = torch.empty(scores.shape, dtype=torch.int8)
    mp = None
    if mask is not None:
        mask = _chk(mask, torch.float32, "mask")
        assert mask.shape == (batch, 1, T, S)
        mp = _p(mask)
    _load().orc_attn_softmax_q(_p(scores), mp, _p(out), _i64(batch), _i64(heads), _i64(T), _i64(S))
    return out


def bmm_s8t_s8t_s8t(a, b, alpha):
    """P.V with V row-major: a [B,M,K], b [B,K,N] (ti_bmm_s8t_s8t_s8t) = bmm_s8t_s8n_s8t on b transposed."""
    return bmm_s8t_s8n_s8t(a, b.transpose(1, 2).contiguous(), alpha)


def decode_attn_s8(q, k_new, v_new, k_buf, v_buf, filled, mask, heads, alpha_qk, alpha_pv):
    """ti_decode_attn_s8: the chain of upstream's decode step (torch_int/models/opt.py:128-190) on
    [BH, T, d] q / k_new / v_new and cache buffers [BH, cap, d] holding ``filled`` positions.  Returns
    (ctx, probs, k_buf', v_buf') with the new rows appended in copies of the buffers."""
    T = q.shape[1]
    S = filled + T
    k_buf, v_buf = k_buf.clone(), v_buf.clone()
    k_buf[:, filled:S] = k_new
    v_buf[:, filled:S] = v_new
    scores = bmm_s8t_s8n_f32t(q, k_buf[:, :S].contiguous(), alpha_qk)
    probs = attn_softmax_q(scores, mask, heads)
    ctx = bmm_s8t_s8t_s8t(probs, v_buf[:, :S].contiguous(), alpha_pv)
    return ctx, probs, k_buf, v_buf


def linear_a8_w8_bfp32_ofp32_acc(x, w, bias, alpha, beta, inout, acc_fn=gemm_acc):
    """ti_linear_a8_w8_bfp32_ofp32_acc: the fp32 linear, rounded, then one fp32 add into ``inout`` (returns a new tensor)."""
    return inout + linear_a8_w8_bfp32_ofp32(x, w, bias, alpha, beta, acc_fn=acc_fn).view(inout.shape)


def linear_a8_w8_b8_o8_group(x, weights, biases, alphas, betas):
    """ti_linear_a8_w8_b8_o8_group: the separate linears, one after the other."""
    return tuple(linear_a8_w8_b8_o8(x, w, b, a, be) for w, b, a, be in zip(weights, biases, alphas, betas))


def linear_a8_w8_b8_o8_heads(x, w, bias, alpha, beta, bsz, seq_len, heads, head_dim):
    """ti_linear_a8_w8_b8_o8_heads: the plain linear, then the head split as torch writes it."""
    y = linear_a8_w8_b8_o8(x, w, bias, alpha, beta)
    return y.view(bsz, seq_len, heads, head_dim).transpose(1, 2).contiguous()

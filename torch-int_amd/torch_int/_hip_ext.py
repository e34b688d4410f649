"""Fused element-wise kernels of the OPT blocks that upstream runs as chains of torch ops.

These are *not* part of the reference's ``torch_int._CUDA`` surface; the modules in
``torch_int.nn.fused`` and ``torch_int.models.opt`` call them when their input is an fp32
tensor on a HIP device and fall back to the upstream torch-op chain otherwise.

* :func:`add_layernorm_q` -- ``residual.add_(x)`` + ``LayerNormQ`` (upstream models/opt.py:281-283,
  nn/fused.py:13-18) in one pass.
* :func:`attn_softmax_q` -- mask add, clamp to finfo.min, softmax, ``*127``, round, int8 cast
  (upstream models/opt.py:144-178) in one pass.
* :func:`split_heads`, :func:`merge_heads`, :func:`transpose_last2` -- the int8 layout changes around
  the two attention products (upstream models/opt.py:80-81, 180, 189-196).
* :func:`bmm_s8t_s8t_s8t` -- P.V on V as the KV cache stores it (no transposed copy), for the few
  query rows of incremental decoding.
"""
import ctypes

import torch

from . import _CUDA

_lib = _CUDA._lib
_vp, _i64, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float
_lib.ti_add_layernorm_q.argtypes = [_vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]
_lib.ti_add_layernorm_q.restype = ctypes.c_int
_lib.ti_add_layernorm_q_f16.argtypes = [_vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]
_lib.ti_add_layernorm_q_f16.restype = ctypes.c_int
_lib.ti_add_layernorm_q_f16_xf32.argtypes = [_vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]
_lib.ti_add_layernorm_q_f16_xf32.restype = ctypes.c_int
_lib.ti_add_f16_xf32.argtypes = [_vp, _vp, _i64, _vp]
_lib.ti_add_f16_xf32.restype = ctypes.c_int
_lib.ti_attn_softmax_q.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]
_lib.ti_attn_softmax_q.restype = ctypes.c_int
_lib.ti_permute_0213_s8.argtypes = [_vp, _vp, _i64, _i64, _i64, _i64, _vp]
_lib.ti_permute_0213_s8.restype = ctypes.c_int
_lib.ti_transpose_last2_s8.argtypes = [_vp, _vp, _i64, _i64, _i64, _vp]
_lib.ti_transpose_last2_s8.restype = ctypes.c_int
_lib.ti_bmm_s8t_s8t_s8t.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _f32, _vp]
_lib.ti_bmm_s8t_s8t_s8t.restype = ctypes.c_int
_lib.ti_bmm_s8t_s8n_f32t_strided.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp]
_lib.ti_bmm_s8t_s8n_f32t_strided.restype = ctypes.c_int
_lib.ti_kv_append_s8.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp]
_lib.ti_kv_append_s8.restype = ctypes.c_int
_lib.ti_attn_qk_softmax_q_supported.argtypes = [_i64, _i64, _i64]
_lib.ti_attn_qk_softmax_q_supported.restype = ctypes.c_int
_lib.ti_attn_prefill_supported.argtypes = [_i64, _i64, _i64]
_lib.ti_attn_prefill_supported.restype = ctypes.c_int
_lib.ti_attn_qk_softmax_q.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp]
_lib.ti_attn_qk_softmax_q.restype = ctypes.c_int
_lib.ti_attn_prefill_s8.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp]
_lib.ti_attn_prefill_s8.restype = ctypes.c_int
_lib.ti_attn_qk_softmax_q_mc.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _vp]
_lib.ti_attn_qk_softmax_q_mc.restype = ctypes.c_int
_lib.ti_attn_prefill_s8_mc.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _f32, _vp]
_lib.ti_attn_prefill_s8_mc.restype = ctypes.c_int
_lib.ti_attn_mask_classes_bytes.argtypes = [_i64, _i64, _i64]
_lib.ti_attn_mask_classes_bytes.restype = _i64
_lib.ti_attn_mask_classes.argtypes = [_vp, _vp, _i64, _i64, _i64, _vp]
_lib.ti_attn_mask_classes.restype = ctypes.c_int
_lib.ti_decode_attn_supported.argtypes = [_i64, _i64, _i64]
_lib.ti_decode_attn_supported.restype = ctypes.c_int
_lib.ti_decode_attn_s8.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32,
                                   _f32, _vp]
_lib.ti_decode_attn_s8.restype = ctypes.c_int
_lib.ti_decode_attn_s8_devlen.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _vp, _i64, _f32,
                                              _f32, _vp]
_lib.ti_decode_attn_s8_devlen.restype = ctypes.c_int
_lib.ti_linear_a8_w8_b8_o8_heads.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _f32, _f32, _i64, _i64, _vp, _i64, _vp]
_lib.ti_linear_a8_w8_b8_o8_heads.restype = ctypes.c_int
_pp = ctypes.POINTER(ctypes.c_void_p)
_lib.ti_linear_a8_w8_b8_o8_group.argtypes = [_vp, _pp, _pp, _pp, ctypes.POINTER(_f32), ctypes.POINTER(_f32), _i64, _i64,
                                            _i64, _i64, _vp]
_lib.ti_linear_a8_w8_b8_o8_group.restype = ctypes.c_int
_lib.ti_linear_a8_w8_b8_o8_group_heads.argtypes = [_vp, _pp, _pp, _pp, ctypes.POINTER(_f32), ctypes.POINTER(_f32), _i64,
                                                   _i64, _i64, _i64, _i64, _i64, _vp]
_lib.ti_linear_a8_w8_b8_o8_group_heads.restype = ctypes.c_int
_lib.ti_diag_mfma_loop.argtypes = [ctypes.c_int, _vp, _i64, _i64, _vp, _vp]
_lib.ti_diag_mfma_loop.restype = ctypes.c_int
_lib.ti_diag_mfma_loop_ops.argtypes = [_i64]
_lib.ti_diag_mfma_loop_ops.restype = _i64
_lib.ti_diag_store_loop.argtypes = [_vp, _i64, _i64, ctypes.c_int, ctypes.c_int, _vp]
_lib.ti_diag_store_loop.restype = ctypes.c_int
_lib.ti_linear_group_is_one_launch.argtypes = [_i64, _i64, _i64, ctypes.c_int]
_lib.ti_linear_group_is_one_launch.restype = ctypes.c_int
_group_one_launch = {}
_lib.ti_diag_copy_loop.argtypes = [ctypes.c_int, _vp, _i64, _i64, _vp, _vp]
_lib.ti_diag_copy_loop.restype = ctypes.c_int
_lib.ti_diag_read_loop.argtypes = [ctypes.c_int, _vp, _i64, _i64, _vp, _vp]
_lib.ti_diag_read_loop.restype = ctypes.c_int
_lib.ti_diag_copy_loop_bytes.argtypes = [_i64]
_lib.ti_diag_copy_loop_bytes.restype = _i64
_lib.ti_diag_mix_loop.argtypes = [ctypes.c_int, ctypes.c_int, _vp, _i64, _i64, _vp, _vp]
_lib.ti_diag_mix_loop.restype = ctypes.c_int
_lib.ti_diag_mix_loop_ops.argtypes = [ctypes.c_int, _i64]
_lib.ti_diag_mix_loop_ops.restype = _i64


class OptDecodeLayer(ctypes.Structure):
    """``TiOptDecodeLayer`` of include/torch_int_hip.h: what one decoder layer's decode step reads."""
    _fields_ = ([(n, _i64) for n in ("embed", "heads", "head_dim", "ffn")]
                + [("half", ctypes.c_int32), ("ln1_eps", _f32), ("ln2_eps", _f32)]
                + [(n, _vp) for n in ("ln1_gamma", "ln1_beta", "ln2_gamma", "ln2_beta", "wq", "wk", "wv", "bq", "bk", "bv")]
                + [(n, _f32) for n in ("alpha_q", "alpha_k", "alpha_v", "beta_q", "beta_k", "beta_v", "alpha_qk", "alpha_pv")]
                + [("wo", _vp), ("bo", _vp), ("alpha_o", _f32), ("w1", _vp), ("b1", _vp), ("alpha_1", _f32), ("beta_1", _f32),
                   ("w2", _vp), ("b2", _vp), ("alpha_2", _f32)])


_lib.ti_opt_decoder_layer_decode_scratch_bytes.argtypes = [_i64, _i64, _i64]
_lib.ti_opt_decoder_layer_decode_scratch_bytes.restype = _i64
_lib.ti_opt_decoder_layer_decode.argtypes = [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]
_lib.ti_opt_decoder_layer_decode.restype = ctypes.c_int
_lib.ti_opt_decoder_layer_prefill_scratch_bytes.argtypes = [_i64, _i64, _i64]
_lib.ti_opt_decoder_layer_prefill_scratch_bytes.restype = _i64
_lib.ti_opt_decoder_layer_prefill.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _i64, _vp, _i64, _vp]
_lib.ti_opt_decoder_layer_prefill.restype = ctypes.c_int
_raw_stream = torch._C._cuda_getCurrentRawStream
_fast_opt_layer_decode = getattr(_CUDA._fast, "opt_layer_decode", None)
_fast_opt_layer_prefill = getattr(_CUDA._fast, "opt_layer_prefill", None)
_fast = _CUDA._fast if getattr(_CUDA._fast, "kv_append", None) is not None else None
_fast_decode_attn = getattr(_CUDA._fast, "decode_attn", None)
_fast_group3 = getattr(_CUDA._fast, "linear_group3", None)
_fast_add_ln_q = getattr(_CUDA._fast, "add_ln_q", None)
_fast_softmax_q = getattr(_CUDA._fast, "softmax_q", None)
_fast_bmm_strided = getattr(_CUDA._fast, "bmm_f32t_strided", None)
_fast_bmm_rowmajor = getattr(_CUDA._fast, "bmm_rowmajor", None)


class _NoSwitch:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_SWITCH = _NoSwitch()
_current_device = torch.cuda.current_device


def _on(dev):
    """Context that makes ``dev`` current; free when it already is (the usual case)."""
    return _NO_SWITCH if dev.index == _current_device() else torch.cuda.device(dev)


def _ok(t, dtype):
    return isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous()


def can_fuse_layernorm(x, weight, bias):
    """True when the fused kernel applies: contiguous HIP tensors that are all fp32 or all fp16, last dim = len(weight)."""
    dt = x.dtype if isinstance(x, torch.Tensor) else None
    return (dt in (torch.float32, torch.float16) and _ok(x, dt) and _ok(weight, dt) and _ok(bias, dt)
            and x.dim() >= 1 and x.shape[-1] == weight.numel() == bias.numel() and x.numel() > 0)


def can_fuse_layernorm_add(add, x):
    """True when ``add`` can be the addend of the fused residual update of ``x``: same shape and device, contiguous,
    and of ``x``'s dtype -- or fp32 on an fp16 stream, which the kernel rounds to fp16 first, as
    ``x.add_(add.to(x.dtype))`` does."""
    return (isinstance(add, torch.Tensor) and add.shape == x.shape and add.device == x.device and add.is_contiguous()
            and (add.dtype == x.dtype or (add.dtype is torch.float32 and x.dtype is torch.float16)))


def add_rounded_(residual, x):
    """``residual.add_(x.to(residual.dtype))`` for an fp16 ``residual`` and an fp32 ``x`` (contiguous HIP tensors of one
    shape) in one kernel; returns ``residual``."""
    if not (_ok(residual, torch.float16) and _ok(x, torch.float32) and x.shape == residual.shape
            and x.device == residual.device):
        raise RuntimeError("torch_int._hip_ext.add_rounded_: needs a contiguous fp16 and a contiguous fp32 HIP tensor "
                           "of one shape")
    with _on(residual.device):
        rc = _lib.ti_add_f16_xf32(x.data_ptr(), residual.data_ptr(), residual.numel(),
                                  _raw_stream(residual.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.add_rounded_: {_lib.ti_last_error().decode()} (status {rc})")
    return residual


def add_layernorm_q(x, residual, weight, bias, eps, checked=False):
    """``residual += x`` in place (skipped when ``x`` is None; an fp32 ``x`` on an fp16 residual is rounded to fp16
    first), returns int8
    ``clamp(round(layer_norm(residual) * weight + bias), -128, 127)``.  ``checked=True``: the caller has
    already established the conditions below (the modules do, via the ``can_*`` predicates)."""
    op = "add_layernorm_q"
    if not checked:
        if not can_fuse_layernorm(residual, weight, bias):
            raise RuntimeError(f"torch_int._hip_ext.{op}: needs contiguous HIP tensors, all fp32 or all fp16")
        if x is not None and not can_fuse_layernorm_add(x, residual):
            raise RuntimeError(f"torch_int._hip_ext.{op}: x must be a contiguous tensor shaped like residual, of its "
                               "dtype (or fp32 on an fp16 residual)")
    dev = residual.device
    H = residual.shape[-1]
    q = torch.empty(residual.shape, dtype=torch.int8, device=dev)
    with _on(dev):
        if residual.dtype is torch.float16 and x is not None and x.dtype is torch.float32:
            rc = _lib.ti_add_layernorm_q_f16_xf32(x.data_ptr(), residual.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                                  float(eps), q.data_ptr(), residual.numel() // H, H,
                                                  _raw_stream(dev.index) or None)
        elif residual.dtype is torch.float16:
            rc = _lib.ti_add_layernorm_q_f16(x.data_ptr() if x is not None else None, residual.data_ptr(),
                                             weight.data_ptr(), bias.data_ptr(), float(eps), q.data_ptr(),
                                             residual.numel() // H, H, _raw_stream(dev.index) or None)
        elif _fast_add_ln_q is not None:
            rc = _fast_add_ln_q(x.data_ptr() if x is not None else 0, residual.data_ptr(), weight.data_ptr(),
                                bias.data_ptr(), float(eps), q.data_ptr(), residual.numel() // H, H,
                                _raw_stream(dev.index))
        else:
            rc = _lib.ti_add_layernorm_q(x.data_ptr() if x is not None else None, residual.data_ptr(),
                                         weight.data_ptr(), bias.data_ptr(), float(eps), q.data_ptr(),
                                         residual.numel() // H, H, _raw_stream(dev.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.{op}: {_lib.ti_last_error().decode()} (status {rc})")
    return q


def can_fuse_softmax(scores, mask, bsz, heads):
    if not (_ok(scores, torch.float32) and scores.dim() == 3 and scores.shape[0] == bsz * heads and scores.numel() > 0):
        return False
    if mask is None:
        return True
    return (_ok(mask, torch.float32) and mask.device == scores.device
            and tuple(mask.shape) == (bsz, 1, scores.shape[1], scores.shape[2]))


def attn_softmax_q(scores, mask, heads, checked=False):
    """scores fp32 [bsz*heads, T, S], mask fp32 [bsz, 1, T, S] or None ->
    int8 ``round(127 * softmax(max(scores + mask, finfo.min), dim=-1))``."""
    op = "attn_softmax_q"
    BH, T, S = scores.shape
    bsz = BH // heads
    if not checked and (bsz * heads != BH or not can_fuse_softmax(scores, mask, bsz, heads)):
        raise RuntimeError(f"torch_int._hip_ext.{op}: needs contiguous fp32 HIP tensors, scores [bsz*heads,T,S], "
                           f"mask [bsz,1,T,S]")
    dev = scores.device
    out = torch.empty((BH, T, S), dtype=torch.int8, device=dev)
    with _on(dev):
        if _fast_softmax_q is not None:
            rc = _fast_softmax_q(scores.data_ptr(), mask.data_ptr() if mask is not None else 0, out.data_ptr(), bsz,
                                 heads, T, S, _raw_stream(dev.index))
        else:
            rc = _lib.ti_attn_softmax_q(scores.data_ptr(), mask.data_ptr() if mask is not None else None,
                                        out.data_ptr(), bsz, heads, T, S, _raw_stream(dev.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.{op}: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def split_heads(t, bsz, seq_len, heads, head_dim):
    """int8 [bsz, seq, heads*head_dim] -> contiguous [bsz, heads, seq, head_dim]
    (``view(bsz, seq, heads, d).transpose(1, 2).contiguous()``)."""
    if (seq_len == 1 or heads == 1) and t.is_contiguous():
        return t.view(bsz, heads, seq_len, head_dim)  # the permutation moves nothing
    if not (_ok(t, torch.int8) and t.numel() == bsz * seq_len * heads * head_dim and t.numel() > 0):
        return t.view(bsz, seq_len, heads, head_dim).transpose(1, 2).contiguous()
    out = torch.empty((bsz, heads, seq_len, head_dim), dtype=torch.int8, device=t.device)
    with _on(t.device):
        rc = _lib.ti_permute_0213_s8(t.data_ptr(), out.data_ptr(), bsz, seq_len, heads, head_dim,
                                     _raw_stream(t.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.split_heads: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def merge_heads(t, bsz, heads, seq_len, head_dim):
    """int8 [bsz*heads, seq, head_dim] -> contiguous [bsz, seq, heads*head_dim]."""
    if (seq_len == 1 or heads == 1) and t.is_contiguous():
        return t.view(bsz, seq_len, heads * head_dim)
    if not (_ok(t, torch.int8) and t.numel() == bsz * seq_len * heads * head_dim and t.numel() > 0):
        return t.view(bsz, heads, seq_len, head_dim).transpose(1, 2).reshape(bsz, seq_len, heads * head_dim).contiguous()
    out = torch.empty((bsz, seq_len, heads * head_dim), dtype=torch.int8, device=t.device)
    with _on(t.device):
        rc = _lib.ti_permute_0213_s8(t.data_ptr(), out.data_ptr(), bsz, heads, seq_len, head_dim,
                                     _raw_stream(t.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.merge_heads: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def transpose_last2(t):
    """int8 [B, R, C] -> contiguous [B, C, R]."""
    if not (_ok(t, torch.int8) and t.dim() == 3 and t.numel() > 0 and t.shape[0] <= 65535):
        return t.transpose(1, 2).contiguous()
    B, R, C = t.shape
    out = torch.empty((B, C, R), dtype=torch.int8, device=t.device)
    with _on(t.device):
        rc = _lib.ti_transpose_last2_s8(t.data_ptr(), out.data_ptr(), B, R, C, _raw_stream(t.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.transpose_last2: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def _batch_strided(t):
    """int8 HIP tensor [B, R, C] whose [R, C] matrices are packed; the batch stride may exceed R*C
    (a view into a buffer with spare rows, such as a KV cache with room to grow)."""
    return (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.int8 and t.dim() == 3
            and (t.shape[2] == 1 or t.stride(2) == 1) and (t.shape[1] == 1 or t.stride(1) == t.shape[2])
            and (t.shape[0] == 1 or t.stride(0) >= t.shape[1] * t.shape[2]))


def can_bmm_rowmajor(a, b):
    return (_ok(a, torch.int8) and _batch_strided(b) and a.dim() == 3 and a.device == b.device
            and a.shape[0] == b.shape[0] and a.shape[2] == b.shape[1] and a.shape[0] <= 65535)


def bmm_s8t_s8t_s8t(a, b, alpha, checked=False):
    """int8 a [B, M, K], int8 b [B, K, N] (row-major, *not* transposed; batch stride free) -> int8
    ``clamp(round(alpha * a @ b), -128, 127)`` [B, M, N].  Streams b once per 16 rows of a."""
    if not checked and not can_bmm_rowmajor(a, b):
        raise RuntimeError("torch_int._hip_ext.bmm_s8t_s8t_s8t: needs int8 HIP tensors a [B,M,K] (contiguous), "
                           "b [B,K,N] (each matrix packed)")
    B, M, K = a.shape
    N = b.shape[2]
    out = torch.empty((B, M, N), dtype=torch.int8, device=a.device)
    with _on(a.device):
        if _fast_bmm_rowmajor is not None:
            rc = _fast_bmm_rowmajor(a.data_ptr(), b.data_ptr(), out.data_ptr(), B, M, N, K,
                                    b.stride(0) if B > 1 else 0, float(alpha), _raw_stream(a.device.index))
        else:
            rc = _lib.ti_bmm_s8t_s8t_s8t(a.data_ptr(), b.data_ptr(), out.data_ptr(), B, M, N, K,
                                         b.stride(0) if B > 1 else 0, float(alpha),
                                         _raw_stream(a.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.bmm_s8t_s8t_s8t: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def can_bmm_strided(a, b):
    return (_batch_strided(a) and _batch_strided(b) and a.device == b.device and a.shape[0] == b.shape[0]
            and a.shape[2] == b.shape[2] and a.shape[0] <= 65535 and a.numel() > 0 and b.numel() > 0)


def bmm_s8t_s8n_f32t_strided(a, b, alpha, checked=False):
    """``_CUDA.bmm_s8t_s8n_f32t`` for operands that are packed per matrix but not along the batch dimension:
    a [B, M, K], b [B, N, K] -> fp32 alpha * a @ b^T [B, M, N]."""
    if not checked and not can_bmm_strided(a, b):
        raise RuntimeError("torch_int._hip_ext.bmm_s8t_s8n_f32t_strided: needs int8 HIP tensors a [B,M,K], b [B,N,K] "
                           "whose matrices are packed")
    B, M, K = a.shape
    N = b.shape[1]
    out = torch.empty((B, M, N), dtype=torch.float32, device=a.device)
    with _on(a.device):
        if _fast_bmm_strided is not None:
            rc = _fast_bmm_strided(a.data_ptr(), b.data_ptr(), out.data_ptr(), B, M, N, K,
                                   a.stride(0) if B > 1 else 0, b.stride(0) if B > 1 else 0, float(alpha),
                                   _raw_stream(a.device.index))
        else:
            rc = _lib.ti_bmm_s8t_s8n_f32t_strided(a.data_ptr(), b.data_ptr(), out.data_ptr(), B, M, N, K,
                                                  a.stride(0) if B > 1 else 0, b.stride(0) if B > 1 else 0,
                                                  float(alpha), _raw_stream(a.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.bmm_s8t_s8n_f32t_strided: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def can_kv_append(k_new, v_new, k_buf, v_buf):
    """int8 HIP tensors: new [B, H, T, d] contiguous, buffers [B, H, cap, d] contiguous, all on one device."""
    return (_ok(k_new, torch.int8) and _ok(v_new, torch.int8) and _ok(k_buf, torch.int8) and _ok(v_buf, torch.int8)
            and k_new.dim() == 4 and k_new.shape == v_new.shape and k_buf.shape == v_buf.shape
            and k_buf.shape[:2] == k_new.shape[:2] and k_buf.shape[3] == k_new.shape[3]
            and k_new.device == v_new.device == k_buf.device == v_buf.device)


def kv_append(k_new, v_new, k_buf, v_buf, filled, checked=False):
    """k_buf[:, :, filled:filled+T] = k_new and the same for v, one launch."""
    if not checked and not can_kv_append(k_new, v_new, k_buf, v_buf):
        raise RuntimeError("torch_int._hip_ext.kv_append: needs contiguous int8 HIP tensors new [B,H,T,d], buffers [B,H,cap,d]")
    B, H, T, d = k_new.shape
    cap = k_buf.shape[2]
    dev = k_new.device
    with _on(dev):
        stream = _raw_stream(dev.index)
        if _fast is not None:
            rc = _fast.kv_append(k_new.data_ptr(), v_new.data_ptr(), k_buf.data_ptr(), v_buf.data_ptr(), B * H, T, d,
                                 cap, filled, stream)
        else:
            rc = _lib.ti_kv_append_s8(k_new.data_ptr(), v_new.data_ptr(), k_buf.data_ptr(), v_buf.data_ptr(), B * H, T,
                                      d, cap, filled, stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.kv_append: {_lib.ti_last_error().decode()} (status {rc})")


def can_attn_qk_softmax_q(q, k, mask, bsz, heads):
    """int8 HIP q [bsz*heads, T, d] contiguous and k [bsz*heads, S, d] with packed rows (any batch stride that is
    a multiple of 16), d a multiple of 16 up to 128 and S a multiple of 16 up to 4096;
    mask None or fp32 [bsz, 1, T, S] contiguous."""
    if not (_ok(q, torch.int8) and type(k) is torch.Tensor and k.dtype is torch.int8 and k.is_cuda and q.dim() == 3
            and k.dim() == 3 and q.shape[0] == k.shape[0] == bsz * heads and q.shape[2] == k.shape[2]
            and k.device == q.device and q.numel() > 0):
        return False
    T, S, d = q.shape[1], k.shape[1], q.shape[2]
    if not _lib.ti_attn_qk_softmax_q_supported(T, S, d):
        return False
    if k.stride(2) != 1 or k.stride(1) != d or k.stride(0) < S * d or k.stride(0) % 16 or q.data_ptr() % 16 or \
            k.data_ptr() % 16:
        return False
    return mask is None or (_ok(mask, torch.float32) and mask.shape == (bsz, 1, T, S) and mask.device == q.device
                            and mask.data_ptr() % 16 == 0)


_mask_classes_cache = {}  # id(mask) -> (weak reference, version counter, classes tensor)


def mask_classes(mask):
    """The class array of an additive fp32 mask [bsz, 1, T, S] for the long-prefill attention kernel (which tiles of
    64 rows x 256 keys are all zero / all one masked value / mixed), or None when the shape takes none.  Made once per
    mask tensor and version: every head and every layer of a forward pass adds the same mask."""
    import weakref
    key = id(mask)
    hit = _mask_classes_cache.get(key)
    if hit is not None and hit[0]() is mask and hit[1] == mask._version:
        return hit[2]
    bsz, _, T, S = mask.shape
    n = _lib.ti_attn_mask_classes_bytes(bsz, T, S)
    if n <= 0:
        return None
    cls = torch.empty(n, dtype=torch.uint8, device=mask.device)
    with _on(mask.device):
        rc = _lib.ti_attn_mask_classes(mask.data_ptr(), cls.data_ptr(), bsz, T, S, _raw_stream(mask.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.mask_classes: {_lib.ti_last_error().decode()} (status {rc})")
    if len(_mask_classes_cache) >= 64:
        _mask_classes_cache.clear()
    _mask_classes_cache[key] = (weakref.ref(mask, lambda _r, k=key: _mask_classes_cache.pop(k, None)), mask._version, cls)
    return cls


def _classes_ptr(mask, S):
    """Pointer to the mask's class array where the kernel that will run reads one (more than 576 keys), else None."""
    if mask is None or S <= 576:
        return None
    cls = mask_classes(mask)
    return cls.data_ptr() if cls is not None else None


def attn_qk_softmax_q(q, k, mask, alpha, heads, checked=False):
    """int8 round(127 softmax(alpha q k^T + mask)) [bsz*heads, T, S] in one launch: the values of
    ``attn_softmax_q(bmm_s8t_s8n_f32t(q, k, alpha), mask, heads)`` without the fp32 scores in memory."""
    if not checked and not can_attn_qk_softmax_q(q, k, mask, q.shape[0] // heads, heads):
        raise RuntimeError("torch_int._hip_ext.attn_qk_softmax_q: needs int8 HIP q [B*H,T,d] / k [B*H,S,d] (d a multiple of 16 up to 128, "
                           "S a multiple of 16 up to 4096) and an fp32 mask [B,1,T,S] or None")
    BH, T, d = q.shape
    S = k.shape[1]
    dev = q.device
    probs = torch.empty((BH, T, S), dtype=torch.int8, device=dev)
    with _on(dev):
        rc = _lib.ti_attn_qk_softmax_q_mc(q.data_ptr(), k.data_ptr(), mask.data_ptr() if mask is not None else None,
                                          _classes_ptr(mask, S), probs.data_ptr(), BH, T, S, d, T * d, k.stride(0), heads,
                                          alpha, _raw_stream(dev.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.attn_qk_softmax_q: {_lib.ti_last_error().decode()} (status {rc})")
    return probs


def can_attn_prefill(q, k, vt, mask, bsz, heads):
    """``can_attn_qk_softmax_q`` plus: vt = V transposed, int8 [bsz*heads, d, S] contiguous, and a shape the form
    that multiplies on with V takes (``ti_attn_prefill_supported``)."""
    return (can_attn_qk_softmax_q(q, k, mask, bsz, heads) and _ok(vt, torch.int8)
            and vt.shape == (q.shape[0], q.shape[2], k.shape[1]) and vt.device == q.device and vt.data_ptr() % 16 == 0
            and bool(_lib.ti_attn_prefill_supported(q.shape[1], k.shape[1], q.shape[2])))


def attn_prefill_shape_ok(T, S, d):
    """Whether ``attn_prefill`` takes T query rows over S keys at head size d (cheap: before V is transposed)."""
    return bool(_lib.ti_attn_prefill_supported(int(T), int(S), int(d)))


def attn_prefill(q, k, vt, mask, alpha_qk, alpha_pv, heads, checked=False):
    """Prefill attention in one launch: int8 context [bsz, T, heads*128] =
    merge_heads(bmm_s8t_s8n_s8t(attn_qk_softmax_q(q, k, mask, alpha_qk), vt, alpha_pv)), the same bits, without the
    score and probability tensors."""
    if not checked and not can_attn_prefill(q, k, vt, mask, q.shape[0] // heads, heads):
        raise RuntimeError("torch_int._hip_ext.attn_prefill: needs int8 HIP q [B*H,T,d], k [B*H,S,d], vt [B*H,d,S] "
                           "(d a multiple of 16 up to 128, S a multiple of 16 up to 4096) and an fp32 mask [B,1,T,S] or None")
    BH, T, d = q.shape
    S = k.shape[1]
    dev = q.device
    ctx = torch.empty((BH // heads, T, heads * d), dtype=torch.int8, device=dev)
    with _on(dev):
        rc = _lib.ti_attn_prefill_s8_mc(q.data_ptr(), k.data_ptr(), vt.data_ptr(),
                                        mask.data_ptr() if mask is not None else None, _classes_ptr(mask, S),
                                        ctx.data_ptr(), BH, T, S, d, T * d, k.stride(0), heads, alpha_qk, alpha_pv,
                                        _raw_stream(dev.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.attn_prefill: {_lib.ti_last_error().decode()} (status {rc})")
    return ctx


def decode_attention_shape_ok(T, S, d):
    """Whether ``decode_attention`` takes T query rows over S cache positions of head size d."""
    return bool(_lib.ti_decode_attn_supported(T, S, d))


def can_decode_attention(q, k_new, v_new, k_buf, v_buf, filled, mask):
    """int8 HIP tensors on one device: q / k_new / v_new [B, H, T, d] contiguous with 1 <= T <= 4 and d a multiple of 16 up to 128,
    cache buffers [B, H, cap, d] contiguous holding ``filled`` positions with room for T more; mask None or fp32
    [B, 1, T, filled + T] contiguous; and scores that fit the LDS."""
    if not (_ok(q, torch.int8) and q.dim() == 4 and can_kv_append(k_new, v_new, k_buf, v_buf)
            and q.shape == k_new.shape and q.device == k_new.device and q.numel() > 0):
        return False
    B, H, T, d = q.shape
    S = filled + T
    if S > k_buf.shape[2] or not _lib.ti_decode_attn_supported(T, S, d):
        return False
    if any(t.data_ptr() % 16 for t in (q, k_new, v_new, k_buf, v_buf)):
        return False
    return mask is None or (_ok(mask, torch.float32) and mask.shape == (B, 1, T, S) and mask.device == q.device)


def decode_attention(q, k_new, v_new, k_buf, v_buf, filled, mask, alpha_qk, alpha_pv, want_probs=False,
                     checked=False):
    """The attention of a decode step in one launch: writes k_new / v_new behind the ``filled`` positions of the
    cache buffers and returns (ctx int8 [B*H, T, d], probs int8 [B*H, T, filled+T] or None) with
    ctx = bmm_s8t_s8t_s8t(round(127 softmax(alpha_qk q k^T + mask)), v, alpha_pv), bit for bit what the separate
    Q.K^T, softmax and P.V kernels return."""
    if not checked and not can_decode_attention(q, k_new, v_new, k_buf, v_buf, filled, mask):
        raise RuntimeError("torch_int._hip_ext.decode_attention: needs contiguous int8 HIP q/k_new/v_new [B,H,T,d] "
                           "(T <= 4, d a multiple of 16 up to 128), cache buffers [B,H,cap,d] with room, and an fp32 mask [B,1,T,S] or None")
    B, H, T, d = q.shape
    S = filled + T
    dev = q.device
    ctx = torch.empty((B * H, T, d), dtype=torch.int8, device=dev)
    probs = torch.empty((B * H, T, S), dtype=torch.int8, device=dev) if want_probs else None
    with _on(dev):
        stream = _raw_stream(dev.index)
        if _fast_decode_attn is not None:
            rc = _fast_decode_attn(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_buf.data_ptr(), v_buf.data_ptr(),
                                   mask.data_ptr() if mask is not None else 0, ctx.data_ptr(),
                                   probs.data_ptr() if probs is not None else 0, B * H, T, d, k_buf.shape[2], S, H,
                                   alpha_qk, alpha_pv, stream)
        else:
            rc = _lib.ti_decode_attn_s8(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_buf.data_ptr(),
                                        v_buf.data_ptr(), mask.data_ptr() if mask is not None else None, ctx.data_ptr(),
                                        probs.data_ptr() if probs is not None else None, B * H, T, d, k_buf.shape[2],
                                        S, H, alpha_qk, alpha_pv, stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.decode_attention: {_lib.ti_last_error().decode()} (status {rc})")
    return ctx, probs


_decode_attn_ok = {}


def decode_attention_shape_ok_cached(T, S, d):
    """``decode_attention_shape_ok`` remembered per shape (a decode loop asks once per layer and step)."""
    key = (T, S, d)
    ok = _decode_attn_ok.get(key)
    if ok is None:
        if len(_decode_attn_ok) > 65536:
            _decode_attn_ok.clear()
        ok = _decode_attn_ok[key] = bool(_lib.ti_decode_attn_supported(T, S, d))
    return ok


_attn_prefill_ok = {}


def attn_prefill_shape_ok_cached(T, S, d):
    """``attn_prefill_shape_ok`` remembered per shape."""
    key = (T, S, d)
    ok = _attn_prefill_ok.get(key)
    if ok is None:
        if len(_attn_prefill_ok) > 65536:
            _attn_prefill_ok.clear()
        ok = _attn_prefill_ok[key] = bool(_lib.ti_attn_prefill_supported(T, S, d))
    return ok


_layer_scratch = {}   # (device, stream) -> uint8 tensor: the intermediate tensors of a layer issued from one C call


def _scratch_for(dev, stream, nbytes):
    """One buffer per device and stream, grown on demand and shared by every layer (calls on one stream run one
    after the other).  Memory allocated while the stream is capturing belongs to that graph's pool and is not kept."""
    key = (dev.index, stream)
    buf = _layer_scratch.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(int(nbytes), dtype=torch.uint8, device=dev)
        if not torch.cuda.is_current_stream_capturing():
            if len(_layer_scratch) >= 64:
                _layer_scratch.clear()
            _layer_scratch[key] = buf
    return buf


_layer_scratch_need = {}


def opt_layer_decode(plan, hidden, mask, k_buf, v_buf, S):
    """One decode step of one decoder layer from one C call (``ti_opt_decoder_layer_decode``): ``hidden`` [B, 1, embed]
    (fp32, or fp16 when the plan says half) is updated in place, the new key and value rows are appended to the cache
    buffers, which hold S - 1 positions before the call.  ``plan`` carries ``addr`` (the address of an ``OptDecodeLayer``
    that the caller filled from tensors it keeps alive), ``embed`` and ``ffn``; the caller has checked shapes, dtypes,
    devices and contiguity (the decoder layer does).  The scratch memory is one buffer per device, stream and size,
    shared by every layer."""
    dev = hidden.device
    B = hidden.shape[0]
    with _on(dev):
        stream = _raw_stream(dev.index)
        key = (0, B, plan.embed, plan.ffn)
        need = _layer_scratch_need.get(key)
        if need is None:
            need = _layer_scratch_need[key] = _lib.ti_opt_decoder_layer_decode_scratch_bytes(B, plan.embed, plan.ffn)
        scratch = _scratch_for(dev, stream, need)
        if _fast_opt_layer_decode is not None:
            rc = _fast_opt_layer_decode(plan.addr, hidden.data_ptr(),
                                        mask.data_ptr() if mask is not None else 0, k_buf.data_ptr(), v_buf.data_ptr(),
                                        B, k_buf.shape[2], S, scratch.data_ptr(), scratch.numel(), stream)
        else:
            rc = _lib.ti_opt_decoder_layer_decode(plan.addr, hidden.data_ptr(),
                                                  mask.data_ptr() if mask is not None else None, k_buf.data_ptr(),
                                                  v_buf.data_ptr(), B, k_buf.shape[2], S, scratch.data_ptr(),
                                                  scratch.numel(), stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.opt_layer_decode: {_lib.ti_last_error().decode()} (status {rc})")
    return hidden


def opt_layer_prefill(plan, hidden, mask, k_out, v_out):
    """A prefill through one decoder layer from one C call (``ti_opt_decoder_layer_prefill``): ``hidden`` [B, T, embed]
    is updated in place, ``k_out`` / ``v_out`` (int8 [B, heads, T, head_dim], contiguous) receive the layer's key and
    value rows.  ``plan`` as for ``opt_layer_decode``; the caller has checked shapes, dtypes, devices and contiguity."""
    dev = hidden.device
    B, T = hidden.shape[0], hidden.shape[1]
    M, E, F = B * T, plan.embed, plan.ffn
    with _on(dev):
        stream = _raw_stream(dev.index)
        key = (1, M, E, F)
        need = _layer_scratch_need.get(key)
        if need is None:
            if len(_layer_scratch_need) > 4096:
                _layer_scratch_need.clear()
            need = _layer_scratch_need[key] = (
                _lib.ti_opt_decoder_layer_prefill_scratch_bytes(M, E, F),
                max(_CUDA._ws_bytes(M, E, E), _CUDA._ws_bytes(M, F, E), _CUDA._ws_bytes(M, E, F)))
        scratch = _scratch_for(dev, stream, need[0])
        ws_ptr, ws_bytes = _CUDA._workspace(dev.index, stream, need[1])
        cls = _classes_ptr(mask, T) if mask is not None else None
        if _fast_opt_layer_prefill is not None:
            rc = _fast_opt_layer_prefill(plan.addr, hidden.data_ptr(), mask.data_ptr() if mask is not None else 0,
                                         cls or 0, k_out.data_ptr(), v_out.data_ptr(), B, T, scratch.data_ptr(),
                                         scratch.numel(), ws_ptr, ws_bytes, stream)
        else:
            rc = _lib.ti_opt_decoder_layer_prefill(plan.addr, hidden.data_ptr(),
                                                   mask.data_ptr() if mask is not None else None, cls, k_out.data_ptr(),
                                                   v_out.data_ptr(), B, T, scratch.data_ptr(), scratch.numel(),
                                                   ws_ptr or None, ws_bytes, stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.opt_layer_prefill: {_lib.ti_last_error().decode()} (status {rc})")
    return hidden


def decode_attention_devlen(q, k_new, v_new, k_buf, v_buf, length, max_length, alpha_qk, alpha_pv):
    """``decode_attention`` without a mask for a launch that is captured into a HIP graph and replayed while the cache
    grows: the number of positions after the append is read from ``length`` (int32 HIP tensor of one element, set
    by the caller before every replay; T <= length <= max_length <= capacity) when the kernel runs.  Returns ctx
    int8 [B*H, T, d]."""
    if not (can_decode_attention(q, k_new, v_new, k_buf, v_buf, max_length - q.shape[2], None)
            and _ok(length, torch.int32) and length.numel() == 1 and length.device == q.device):
        raise RuntimeError("torch_int._hip_ext.decode_attention_devlen: needs contiguous int8 HIP q/k_new/v_new "
                           "[B,H,T,d] (T <= 4, d a multiple of 16 up to 128), cache buffers [B,H,cap,d] with cap >= max_length, and an "
                           "int32 HIP tensor holding the length")
    B, H, T, d = q.shape
    dev = q.device
    ctx = torch.empty((B * H, T, d), dtype=torch.int8, device=dev)
    with _on(dev):
        rc = _lib.ti_decode_attn_s8_devlen(q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), k_buf.data_ptr(),
                                           v_buf.data_ptr(), ctx.data_ptr(), B * H, T, d, k_buf.shape[2],
                                           int(max_length), length.data_ptr(), H, alpha_qk, alpha_pv,
                                           _raw_stream(dev.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.decode_attention_devlen: {_lib.ti_last_error().decode()} (status {rc})")
    return ctx


def can_linear_group(x, weights, biases):
    """One int8 HIP activation matrix [M, K] (contiguous) and up to four contiguous int8 weights [N, K] of one
    shape with int8 biases of N elements, all on one device."""
    if not (_ok(x, torch.int8) and x.dim() == 2 and 1 <= len(weights) == len(biases) <= 4 and x.numel() > 0):
        return False
    N, K = weights[0].shape[0], x.shape[1]
    for w, b in zip(weights, biases):
        if not (_ok(w, torch.int8) and _ok(b, torch.int8) and w.dim() == 2 and w.shape[0] == N and w.shape[1] == K
                and b.numel() == N and w.device == x.device and b.device == x.device):
            return False
    return True


def linear_a8_w8_b8_o8_group(x, weights, biases, alphas, betas, checked=False):
    """``[_CUDA.linear_a8_w8_b8_o8(x, w, b, a, be) for ...]`` as one call: a tuple of int8 [M, N] outputs (views
    of one allocation).  For decode-sized M the weights are streamed by a single kernel launch."""
    if not checked and not can_linear_group(x, weights, biases):
        raise RuntimeError("torch_int._hip_ext.linear_a8_w8_b8_o8_group: needs a contiguous int8 HIP input [M,K] and "
                           "1-4 contiguous int8 weights [N,K] / biases [N] of one shape on the same device")
    n = len(weights)
    M, K = x.shape
    N = weights[0].shape[0]
    out = torch.empty((n, M, N), dtype=torch.int8, device=x.device)
    step = M * N
    base = out.data_ptr()
    with _on(x.device):
        stream = _raw_stream(x.device.index)
        if n == 3 and _fast_group3 is not None:
            rc = _fast_group3(x.data_ptr(), weights[0].data_ptr(), weights[1].data_ptr(), weights[2].data_ptr(),
                              biases[0].data_ptr(), biases[1].data_ptr(), biases[2].data_ptr(), base, base + step,
                              base + 2 * step, M, N, K, float(alphas[0]), float(alphas[1]), float(alphas[2]),
                              float(betas[0]), float(betas[1]), float(betas[2]), stream)
        else:
            arr = ctypes.c_void_p * n
            farr = _f32 * n
            rc = _lib.ti_linear_a8_w8_b8_o8_group(
                x.data_ptr(), arr(*[w.data_ptr() for w in weights]), arr(*[b.data_ptr() for b in biases]),
                arr(*[base + i * step for i in range(n)]), farr(*[float(a) for a in alphas]),
                farr(*[float(b) for b in betas]), n, M, N, K, stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.linear_a8_w8_b8_o8_group: {_lib.ti_last_error().decode()} (status {rc})")
    return out.unbind(0)


def linear_group_is_one_launch(M, N, K, count=3):
    """Whether the library runs a group of [M,K] x [N,K] linears as ONE launch (otherwise it loops over the
    problems, without the split-K workspace that separate calls would get).  The library's own decision
    (``ti_linear_group_is_one_launch``), cached per shape."""
    key = (int(M), int(N), int(K), int(count))
    hit = _group_one_launch.get(key)
    if hit is None:
        hit = _group_one_launch[key] = bool(_lib.ti_linear_group_is_one_launch(*key))
    return hit


def linear_a8_w8_b8_o8_group_heads(x, weights, biases, alphas, betas, bsz, seq_len, heads, head_dim, checked=False):
    """``[linear_a8_w8_b8_o8_heads(x, w, b, a, be, bsz, seq_len, heads, head_dim) for ...]`` as one call: a tuple
    of int8 [bsz, heads, seq, head_dim] outputs (views of one allocation).  The q/k/v projections of a prefill:
    widths the 256x160, 256x288 or (see ``linear_group_is_one_launch``) 256x128 tiles divide run as one persistent
    launch over all the problems."""
    if not checked and not (can_linear_group(x, weights, biases)
                            and all(can_linear_heads(x, w, b, bsz, seq_len, heads, head_dim)
                                    for w, b in zip(weights, biases))):
        raise RuntimeError("torch_int._hip_ext.linear_a8_w8_b8_o8_group_heads: needs a contiguous int8 HIP input "
                           "[bsz*seq,K] and 1-4 contiguous int8 weights [heads*d,K] / biases [heads*d] of one shape "
                           "on the same device, d a multiple of 16")
    n = len(weights)
    M, K = x.shape
    N = weights[0].shape[0]
    out = torch.empty((n, bsz, heads, seq_len, head_dim), dtype=torch.int8, device=x.device)
    step = M * N
    base = out.data_ptr()
    arr = ctypes.c_void_p * n
    farr = _f32 * n
    with _on(x.device):
        stream = _raw_stream(x.device.index)
        rc = _lib.ti_linear_a8_w8_b8_o8_group_heads(
            x.data_ptr(), arr(*[w.data_ptr() for w in weights]), arr(*[b.data_ptr() for b in biases]),
            arr(*[base + i * step for i in range(n)]), farr(*[float(a) for a in alphas]),
            farr(*[float(b) for b in betas]), n, M, N, K, seq_len, head_dim, stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.linear_a8_w8_b8_o8_group_heads: {_lib.ti_last_error().decode()} "
                           f"(status {rc})")
    return out.unbind(0)


def can_linear_heads(x, w, bias, bsz, seq_len, heads, head_dim):
    return (_ok(x, torch.int8) and _ok(w, torch.int8) and _ok(bias, torch.int8) and x.dim() == 2 and w.dim() == 2
            and x.shape[1] == w.shape[1] and x.shape[0] == bsz * seq_len and w.shape[0] == heads * head_dim
            and bias.numel() == w.shape[0] and head_dim % 16 == 0 and x.numel() > 0
            and w.device == x.device and bias.device == x.device)


def linear_a8_w8_b8_o8_heads(x, w, bias, alpha, beta, bsz, seq_len, heads, head_dim, checked=False):
    """``_CUDA.linear_a8_w8_b8_o8(x, w, bias, alpha, beta).view(bsz, seq, heads, d).transpose(1, 2).contiguous()``
    with the permutation done by the GEMM's stores: int8 [bsz, heads, seq, head_dim]."""
    if not checked and not can_linear_heads(x, w, bias, bsz, seq_len, heads, head_dim):
        raise RuntimeError("torch_int._hip_ext.linear_a8_w8_b8_o8_heads: needs contiguous int8 HIP tensors x [bsz*seq,K], "
                           "w [heads*d,K], bias [heads*d] with d a multiple of 16")
    M, K = x.shape
    N = w.shape[0]
    out = torch.empty((bsz, heads, seq_len, head_dim), dtype=torch.int8, device=x.device)
    idx = x.device.index
    with _on(x.device):
        stream = _raw_stream(idx)
        ws_ptr, ws_bytes = _CUDA._workspace(idx, stream, _CUDA._ws_bytes(M, N, K)) if M > 16 else (0, 0)
        rc = _lib.ti_linear_a8_w8_b8_o8_heads(x.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), M, N, K,
                                              float(alpha), float(beta), seq_len, head_dim, ws_ptr or None, ws_bytes,
                                              stream or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.linear_a8_w8_b8_o8_heads: {_lib.ti_last_error().decode()} (status {rc})")
    return out


def diag_mfma_loop(mode, data, iters, sink):
    """Diagnostic launch (computes nothing): the mainloop's instruction mix ``iters`` times per wave on the bytes of
    ``data`` (uint8 / int8 HIP tensor of at least 1 MiB); mode 0 = MFMA only, 1 = + LDS fragment reads, 2 = + global->LDS
    copies and a barrier per step.  ``sink`` is an int32 HIP tensor of one element.  Returns the integer operations
    the launch performs."""
    if not (isinstance(data, torch.Tensor) and data.is_cuda and data.is_contiguous() and data.element_size() == 1):
        raise RuntimeError("torch_int._hip_ext.diag_mfma_loop: data must be a contiguous one-byte HIP tensor")
    if not (_ok(sink, torch.int32) and sink.numel() >= 1 and sink.device == data.device):
        raise RuntimeError("torch_int._hip_ext.diag_mfma_loop: sink must be an int32 HIP tensor on the same device")
    with _on(data.device):
        rc = _lib.ti_diag_mfma_loop(int(mode), data.data_ptr(), data.numel(), int(iters), sink.data_ptr(),
                                    _raw_stream(data.device.index) or None)
        ops = int(_lib.ti_diag_mfma_loop_ops(int(iters)))
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.diag_mfma_loop: {_lib.ti_last_error().decode()} (status {rc})")
    return ops


def diag_store_loop(out, workgroups, reps=1):
    """Diagnostic launch: ``workgroups`` workgroups fill the fp32 HIP matrix ``out`` ([M, N] contiguous, M a multiple of
    256, N of 160) with 1.0, ``reps`` times, using the store pattern of the 256x160 GEMM kernel's 32-bit epilogue.
    Returns the bytes the launch writes."""
    if not (_ok(out, torch.float32) and out.dim() == 2):
        raise RuntimeError("torch_int._hip_ext.diag_store_loop: out must be a contiguous fp32 HIP matrix")
    with _on(out.device):
        rc = _lib.ti_diag_store_loop(out.data_ptr(), out.shape[0], out.shape[1], int(workgroups), int(reps),
                                     _raw_stream(out.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.diag_store_loop: {_lib.ti_last_error().decode()} (status {rc})")
    return out.numel() * 4 * int(reps)


def diag_read_loop(mode, data, sink):
    """One read-only pass over the int8 matrix ``data`` [N, K] (``ti_diag_read_loop``): mode 0 flat, 1 flat
    non-temporal, 2 the streaming GEMM's copy pipeline (non-temporal), 3 the same with the default cache policy.
    Returns the bytes read."""
    if not (_ok(data, torch.int8) and data.dim() == 2):
        raise RuntimeError("torch_int._hip_ext.diag_read_loop: data must be a contiguous int8 HIP matrix")
    if not (_ok(sink, torch.int32) and sink.device == data.device and sink.numel() >= 1):
        raise RuntimeError("torch_int._hip_ext.diag_read_loop: sink must be an int32 HIP tensor on the same device")
    with _on(data.device):
        rc = _lib.ti_diag_read_loop(int(mode), data.data_ptr(), data.shape[0], data.shape[1], sink.data_ptr(),
                                    _raw_stream(data.device.index) or None)
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.diag_read_loop: {_lib.ti_last_error().decode()} (status {rc})")
    return data.numel()


def diag_copy_loop(mode, data, iters, sink):
    """Diagnostic launch (computes nothing): every CU fetches 48 KiB per step, ``iters`` steps, from the first 2 MiB of
    ``data`` (one-byte HIP tensor) with the GEMM mainloop's access pattern; mode 0 = global->LDS copies, 1 = loads into
    registers.  Returns the bytes the launch fetches."""
    if not (isinstance(data, torch.Tensor) and data.is_cuda and data.is_contiguous() and data.element_size() == 1):
        raise RuntimeError("torch_int._hip_ext.diag_copy_loop: data must be a contiguous one-byte HIP tensor")
    if not (_ok(sink, torch.int32) and sink.numel() >= 1 and sink.device == data.device):
        raise RuntimeError("torch_int._hip_ext.diag_copy_loop: sink must be an int32 HIP tensor on the same device")
    with _on(data.device):
        rc = _lib.ti_diag_copy_loop(int(mode), data.data_ptr(), data.numel(), int(iters), sink.data_ptr(),
                                    _raw_stream(data.device.index) or None)
        nbytes = int(_lib.ti_diag_copy_loop_bytes(int(iters)))
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.diag_copy_loop: {_lib.ti_last_error().decode()} (status {rc})")
    return nbytes


def diag_mix_loop(shape, parts, data, iters, sink):
    """Diagnostic launch (computes nothing): ``iters`` K steps of the instruction mix of the 256x160 (``shape`` 0) or
    128x80 (``shape`` 1) GEMM tile; ``parts`` bit set: 1 MFMAs, 2 LDS fragment reads, 4 global->LDS copies, 8 barrier.
    ``data``: one-byte HIP tensor of at least 3 MiB.  Returns the integer operations of the MFMAs of one launch."""
    if not (isinstance(data, torch.Tensor) and data.is_cuda and data.is_contiguous() and data.element_size() == 1):
        raise RuntimeError("torch_int._hip_ext.diag_mix_loop: data must be a contiguous one-byte HIP tensor")
    if not (_ok(sink, torch.int32) and sink.numel() >= 1 and sink.device == data.device):
        raise RuntimeError("torch_int._hip_ext.diag_mix_loop: sink must be an int32 HIP tensor on the same device")
    with _on(data.device):
        rc = _lib.ti_diag_mix_loop(int(shape), int(parts), data.data_ptr(), data.numel(), int(iters), sink.data_ptr(),
                                   _raw_stream(data.device.index) or None)
        ops = int(_lib.ti_diag_mix_loop_ops(int(shape), int(iters)))
    if rc:
        raise RuntimeError(f"torch_int._hip_ext.diag_mix_loop: {_lib.ti_last_error().decode()} (status {rc})")
    return ops


def measure_mfma_ceiling(window_ms=250.0, iters=20000, window=None):
    """What the int8 matrix pipe of the current device sustains, in TOP/s, for the three loop modes of
    ``diag_mfma_loop`` and for the K step of the 256x160 GEMM tile as a bare instruction mix (``diag_mix_loop``), each
    on constant and on uniformly random operand bytes: back-to-back launches between two HIP
    events for at least ``window_ms`` per figure (after the same again as warm-up, so the clocks have settled under
    the board's power limit).  ``window(label)``, when given, returns a context manager that is entered around the
    timed window of each figure (a benchmark samples clocks and board power there)."""
    import contextlib
    dev = torch.device("cuda", torch.cuda.current_device())
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    patterns = {"constant": torch.full((1 << 20,), 1, dtype=torch.int8, device=dev),
                "random": torch.randint(-127, 128, (1 << 20,), dtype=torch.int8, device=dev)}
    out = {}
    for mode, label in ((0, "mfma_only"), (1, "lds_reads"), (2, "lds_fed")):
        for pname, data in patterns.items():
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            ops = diag_mfma_loop(mode, data, iters, sink)
            end.record()
            torch.cuda.synchronize()
            n = max(2, int(window_ms / max(start.elapsed_time(end), 1e-3)) + 1)
            for timed in (False, True):
                with (window(f"{label}_{pname}") if timed and window is not None else contextlib.nullcontext()):
                    start.record()
                    for _ in range(n):
                        diag_mfma_loop(mode, data, iters, sink)
                    end.record()
                    torch.cuda.synchronize()
            out[f"{label}_{pname}"] = ops * n / start.elapsed_time(end) / 1e9
    # the K step of the 256x160 GEMM tile as a bare instruction mix (16x16x64 MFMAs, fragment reads, copies, barrier)
    big = {"constant": torch.full((3 << 20,), 1, dtype=torch.int8, device=dev),
           "random": torch.randint(-127, 128, (3 << 20,), dtype=torch.int8, device=dev)}
    for pname, data in big.items():
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        ops = diag_mix_loop(0, 15, data, iters, sink)
        end.record()
        torch.cuda.synchronize()
        n = max(2, int(window_ms / max(start.elapsed_time(end), 1e-3)) + 1)
        for timed in (False, True):
            with (window(f"step_mix_256x160_{pname}") if timed and window is not None else contextlib.nullcontext()):
                start.record()
                for _ in range(n):
                    diag_mix_loop(0, 15, data, iters, sink)
                end.record()
                torch.cuda.synchronize()
        out[f"step_mix_256x160_{pname}"] = ops * n / start.elapsed_time(end) / 1e9
    return out

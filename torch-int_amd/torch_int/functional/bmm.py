"""Functional aliases of the batched INT8 products (upstream
``torch_int/functional/bmm.py:5-17``)."""
from .._CUDA import bmm_s8t_s8n_s8t, bmm_s8t_s8n_s32t


def bmm_i8_o8(a, b, scale):
    """int8 [B,M,N] = sat_s8(round(scale * a[B,M,K] . b[B,N,K]^T))."""
    return bmm_s8t_s8n_s8t(a, b, scale)


def bmm_i8_o32(a, b):
    """int32 [B,M,N] = a[B,M,K] . b[B,N,K]^T."""
    return bmm_s8t_s8n_s32t(a, b)

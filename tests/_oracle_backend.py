"""Test helper: run the torch_int modules on CPU tensors by swapping the nine
``torch_int._CUDA`` entry points for the CPU oracle.  Only tests use this; the
package itself has no CPU path."""
import contextlib

import torch

from oracle import oracle as orc

NAMES = ["linear_a8_w8_b32_o32", "linear_a8_w8_b32_o32_with_scaling", "linear_a8_w8_bfp32_ofp32",
         "linear_a8_w8_b8_o8", "linear_relu_a8_w8_b8_o8", "bmm_s8t_s8n_f32t", "bmm_s8t_s8n_s8t",
         "bmm_s8t_s8n_s32t", "dq_add_layernorm_q"]


def _wrap(fn, big_acc):
    def call(*args):
        if big_acc and fn.__name__ != "dq_add_layernorm_q":
            return fn(*args, acc_fn=orc.gemm_acc_torch)
        return fn(*args)
    return call


@contextlib.contextmanager
def oracle_backend(fast_matmul=False):
    """``fast_matmul`` accumulates with torch's CPU int32 matmul (same integers, faster on big shapes)."""
    import torch_int._CUDA as C
    import torch_int.functional.bmm as fbmm
    import torch_int.functional.fused as ffused
    saved = {n: getattr(C, n) for n in NAMES}
    saved_f = (ffused.dq_add_layernorm_q, fbmm.bmm_s8t_s8n_s8t, fbmm.bmm_s8t_s8n_s32t)
    try:
        for n in NAMES:
            setattr(C, n, _wrap(getattr(orc, n), fast_matmul))
        ffused.dq_add_layernorm_q = C.dq_add_layernorm_q
        fbmm.bmm_s8t_s8n_s8t, fbmm.bmm_s8t_s8n_s32t = C.bmm_s8t_s8n_s8t, C.bmm_s8t_s8n_s32t
        yield
    finally:
        for n, f in saved.items():
            setattr(C, n, f)
        ffused.dq_add_layernorm_q, fbmm.bmm_s8t_s8n_s8t, fbmm.bmm_s8t_s8n_s32t = saved_f


def randomize_int8_layer(layer, gen, scale_lo=1e-4, scale_hi=1e-2):
    """Decoder-layer benchmark initialisation of an Int8OPTDecoderLayer: int8 weights and biases
    uniform in [-127,127], fp32 biases ~N(0,1), per-tensor scales ~U(lo,hi), LayerNorm
    gamma ~N(1,0.02), beta ~N(0,0.02)."""
    def u():
        return float(torch.empty(1).uniform_(scale_lo, scale_hi, generator=gen))
    attn = layer.self_attn
    for lin in (attn.q_proj, attn.k_proj, attn.v_proj, layer.fc1):
        lin.weight = torch.randint(-127, 128, lin.weight.shape, dtype=torch.int8, generator=gen)
        lin.bias = torch.randint(-127, 128, (1, lin.out_features), dtype=torch.int8, generator=gen)
        lin.a = torch.tensor(u())
        lin.b = torch.tensor(u())
    for lin in (attn.out_proj, layer.fc2):
        lin.weight = torch.randint(-127, 128, lin.weight.shape, dtype=torch.int8, generator=gen)
        lin.bias = torch.randn(1, lin.out_features, generator=gen)
        lin.a = torch.tensor(u())
    attn.qk_bmm.a = torch.tensor(u())
    attn.pv_bmm.a = torch.tensor(u())
    for ln in (layer.self_attn_layer_norm, layer.final_layer_norm):
        ln.weight = 1 + 0.02 * torch.randn(ln.weight.shape, generator=gen)
        ln.bias = 0.02 * torch.randn(ln.bias.shape, generator=gen)
    return layer


def causal_mask(bsz, tgt, src, dtype=torch.float32, device="cpu"):
    neg = torch.finfo(dtype).min
    m = torch.zeros(tgt, src, dtype=dtype, device=device)
    q = torch.arange(src - tgt, src, device=device)[:, None]
    k = torch.arange(src, device=device)[None, :]
    m = m.masked_fill(k > q, neg)
    return m[None, None].expand(bsz, 1, tgt, src).contiguous()

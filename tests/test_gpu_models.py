"""The modules and OPT blocks on the GPU kernels against the same modules run on CPU
with the oracle behind them (tests/_oracle_backend.py).

Integer results are compared exactly.  Across the fp32 softmax / LayerNorm inside a
decoder layer the CPU and GPU use different library reductions; the bar there is
<= 1e-3 max relative error on fp32 tensors, and int8 tensors derived from them may
differ by one LSB on a small fraction of elements.
"""
import copy
import sys

import pytest
import torch

from _oracle_backend import causal_mask, oracle_backend, randomize_int8_layer
from torch_int.models.opt import Int8OPTDecoderLayer, Int8OPTForCausalLM, OPTConfigLite
from torch_int.nn import (BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T, DQ_Add_LayerNorm_Q, W8A8B8O8Linear,
                          W8A8B8O8LinearReLU, W8A8B32O32Linear, W8A8B32O32LinearWithoutScaling,
                          W8A8BFP32OFP32Linear)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _rel_err(a, b):
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


@torch.no_grad()
def test_linear_and_bmm_modules_on_gpu():
    g = torch.Generator().manual_seed(0)
    x = torch.randint(-127, 128, (4, 512, 768), dtype=torch.int8, generator=g)  # BASELINE config 1 input
    for cls in (W8A8B8O8Linear, W8A8B8O8LinearReLU, W8A8B32O32Linear, W8A8B32O32LinearWithoutScaling,
                W8A8BFP32OFP32Linear):
        _say("module", cls.__name__)
        m = cls(768, 768) if cls is W8A8B32O32LinearWithoutScaling else cls(768, 768, 0.001, 0.01)
        m.weight = torch.randint(-127, 128, (768, 768), dtype=torch.int8, generator=g)
        if m.bias.dtype == torch.float32:
            m.bias = torch.randn(1, 768, generator=g)
        else:
            m.bias = torch.randint(-127, 128, (1, 768), generator=g).to(m.bias.dtype)
        with oracle_backend():
            ref = m(x)
        out = copy.deepcopy(m).to(DEV)(x.to(DEV))
        assert out.shape == (4, 512, 768) and out.dtype == ref.dtype
        assert torch.equal(out.cpu(), ref), cls.__name__
    a = torch.randint(-127, 128, (6, 40, 64), dtype=torch.int8, generator=g)
    b = torch.randint(-127, 128, (6, 56, 64), dtype=torch.int8, generator=g)
    for m in (BMM_S8T_S8N_S8T(0.0007), BMM_S8T_S8N_F32T(0.003)):
        with oracle_backend():
            ref = m(a, b)
        assert torch.equal(copy.deepcopy(m).to(DEV)(a.to(DEV), b.to(DEV)).cpu(), ref)
    d = DQ_Add_LayerNorm_Q(768)
    d.input_scale = 0.004
    d.weight = torch.ones(768) * 30
    inp = torch.randint(-65536, 65536, (4, 16, 768), dtype=torch.int32, generator=g)
    res = torch.randn(4, 16, 768, generator=g)
    with oracle_backend():
        r_ref, q_ref = d(res, inp)
    r, q = copy.deepcopy(d).to(DEV)(res.to(DEV), inp.to(DEV))
    assert torch.equal(r.cpu(), r_ref) and torch.equal(q.cpu(), q_ref)


def _compare_layer(D, H, F, B, T, seed, fast):
    g = torch.Generator().manual_seed(seed)
    layer = randomize_int8_layer(Int8OPTDecoderLayer(D, H, F), g)
    hidden = torch.randn(B, T, D, generator=g)
    mask = causal_mask(B, T, T)
    with oracle_backend(fast_matmul=fast):
        ref = layer(hidden.clone(), attention_mask=mask, use_cache=True)
    gl = copy.deepcopy(layer).to(DEV)
    out = gl(hidden.to(DEV), attention_mask=mask.to(DEV), use_cache=True)
    # K and V caches are pure int8 GEMM outputs of an int8 LayerNorm output
    k_bad = (out[1][0].cpu() != ref[1][0]).float().mean().item()
    v_bad = (out[1][1].cpu() != ref[1][1]).float().mean().item()
    assert (out[1][0].cpu().int() - ref[1][0].int()).abs().max() <= 1 and k_bad < 1e-3, k_bad
    assert (out[1][1].cpu().int() - ref[1][1].int()).abs().max() <= 1 and v_bad < 1e-3, v_bad
    err = _rel_err(out[0].cpu(), ref[0])
    return err


@torch.no_grad()
def test_decoder_layer_small():
    _say("decoder layer D=256")
    err = _compare_layer(256, 4, 1024, 2, 48, seed=1, fast=False)
    assert err <= 1e-3, err


@torch.no_grad()
def test_decoder_layer_opt13b_shape():
    # BASELINE config 4: hidden 5120, 40 heads, FFN 20480, batch 4, seq 512, causal mask
    _say("decoder layer OPT-13B shape (CPU emulation takes a while)")
    err = _compare_layer(5120, 40, 20480, 4, 512, seed=2, fast=True)
    assert err <= 1e-3, err


@torch.no_grad()
def test_causal_lm_prefill_and_decode_on_gpu():
    cfg = OPTConfigLite(hidden_size=256, num_hidden_layers=3, ffn_dim=1024, num_attention_heads=4, vocab_size=512,
                        max_position_embeddings=128)
    torch.manual_seed(0)
    lm = Int8OPTForCausalLM(cfg)
    g = torch.Generator().manual_seed(3)
    for layer in lm.model.decoder.layers:
        randomize_int8_layer(layer, g)
    ids = torch.randint(2, 512, (2, 37), generator=g)  # 37 -> padded to 48 inside the decoder
    with oracle_backend():
        ref = lm(ids, use_cache=True)
        ref_step = lm(ids[:, -1:], past_key_values=ref.past_key_values, use_cache=True)
    glm = copy.deepcopy(lm).to(DEV)
    _say("causal LM prefill")
    out = glm(ids.to(DEV), use_cache=True)
    assert out.logits.shape == (2, 37, 512)
    assert _rel_err(out.logits.cpu(), ref.logits) <= 2e-3
    _say("causal LM decode step (src_len 49: not a multiple of 16)")
    step = glm(ids[:, -1:].to(DEV), past_key_values=out.past_key_values, use_cache=True)
    assert step.past_key_values[0][0].shape[2] == 49
    assert _rel_err(step.logits.cpu(), ref_step.logits) <= 2e-3

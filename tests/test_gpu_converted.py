"""Modules made by ``from_float`` and models loaded from a state dict, on the HIP kernels.

This is how the reference is used (``Int8OPTForCausalLM.from_pretrained`` of an exported int8 checkpoint, upstream
tests/test_opt.py:49-54; ``from_float`` of fp modules with absmax-calibrated scales, tests/test_opt_decoder_layer.py:33-41,
tests/test_linear_modules.py).  Bars: integer GEMM outputs bit-exact against the same module on the oracle backend;
across the fp32 LayerNorm / softmax of a decoder layer one LSB on a small fraction of int8 values and <= 1e-3
relative error on fp32 tensors; relative mean squared error against the fp32 module <= 1e-2.
"""
import copy
import io
import sys

import pytest
import torch
from torch import nn

from _float_opt import FloatOPTDecoderLayer, clone_linear
from _oracle_backend import causal_mask, oracle_backend, randomize_int8_layer
from torch_int.models.opt import Int8OPTDecoderLayer, Int8OPTForCausalLM, OPTConfigLite
from torch_int.nn import (W8A8B8O8Linear, W8A8B8O8LinearReLU, W8A8B32O32Linear, W8A8BFP32OFP32Linear, W8A16Linear,
                          W8FakeA8Linear)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def _rmse2(ref, got):
    return (((ref - got) ** 2).mean() / (ref ** 2).mean()).item()


@torch.no_grad()
def test_from_float_linears_on_gpu():
    # upstream tests/test_linear_modules.py: x ~ N(0,1) [128,512], Linear(512,1024), absmax scales
    torch.manual_seed(0)
    lin = nn.Linear(512, 1024)
    x = torch.randn(128, 512)
    y_gt = lin(x)
    x_scale = x.abs().max() / 127
    q_x = (x / x_scale).round().to(torch.int8)
    cases = [(W8A8B8O8Linear, y_gt, (x_scale, y_gt.abs().max() / 127)),
             (W8A8B8O8LinearReLU, y_gt.clamp(min=0), (x_scale, y_gt.clamp(min=0).abs().max() / 127)),
             (W8A8BFP32OFP32Linear, y_gt, (x_scale,)),
             (W8A8B32O32Linear, y_gt, (x_scale, y_gt.abs().max() / (2 ** 31 - 1)))]
    for cls, ref, scales in cases:
        _say("from_float", cls.__name__)
        m = cls.from_float(clone_linear(lin), *scales)
        with oracle_backend():
            y_cpu = m(q_x)
        y_gpu = copy.deepcopy(m).to(DEV)(q_x.to(DEV))
        assert y_gpu.dtype == y_cpu.dtype and torch.equal(y_gpu.cpu(), y_cpu), cls.__name__
        y = y_gpu.cpu().float() * (scales[1] if len(scales) == 2 else 1.0)
        assert _rmse2(ref, y) < 2e-3, (cls.__name__, _rmse2(ref, y))


@torch.no_grad()
def test_from_float_decoder_layer_on_gpu():
    torch.manual_seed(0)
    D, H, F, B, T = 256, 4, 1024, 2, 64
    fp = FloatOPTDecoderLayer(D, H, F).requires_grad_(False)
    x = torch.randn(B, T, D)
    mask = causal_mask(B, T, T)
    scales = {}
    y_gt = fp(x, mask, record=scales)
    int8 = Int8OPTDecoderLayer.from_float(fp, **scales)
    _say("from_float decoder layer: oracle backend")
    with oracle_backend():
        ref = int8(x.clone(), attention_mask=mask, use_cache=True)
    _say("from_float decoder layer: GPU")
    gl = copy.deepcopy(int8).to(DEV)
    h = x.to(DEV)
    out = gl(h, attention_mask=mask.to(DEV), use_cache=True)
    assert out[0] is h
    for got, want in zip(out[1], ref[1]):   # int8 K / V caches: GEMM outputs of the int8 LayerNorm output
        d = (got.cpu().int() - want.int()).abs()
        assert d.max() <= 1 and (d != 0).float().mean() < 1e-3
    err = ((out[0].cpu() - ref[0]).abs().max() / ref[0].abs().max()).item()
    assert err <= 1e-3, err
    assert _rmse2(y_gt, out[0].cpu()) < 1e-2, _rmse2(y_gt, out[0].cpu())
    # a decode step of the converted layer on the in-place cache
    x1 = torch.randn(B, 1, D)
    m1 = torch.zeros(B, 1, 1, T + 1)
    with oracle_backend():
        ref1 = int8(x1.clone(), attention_mask=m1, use_cache=True, past_key_value=ref[1])
    out1 = gl(x1.to(DEV), attention_mask=m1.to(DEV), use_cache=True, past_key_value=out[1])
    assert out1[1][0].shape == (B, H, T + 1, D // H)
    err = ((out1[0].cpu() - ref1[0]).abs().max() / ref1[0].abs().max()).item()
    assert err <= 2e-3, err


# buffer names of one decoder layer in an exported int8 OPT checkpoint (upstream nn/linear.py:23-28, nn/bmm.py,
# nn/fused.py:8-11, models/opt.py:36-46,207-216)
LAYER_KEYS = {"self_attn.qk_bmm.a", "self_attn.pv_bmm.a",
              "self_attn.k_proj.weight", "self_attn.k_proj.bias", "self_attn.k_proj.a", "self_attn.k_proj.b",
              "self_attn.v_proj.weight", "self_attn.v_proj.bias", "self_attn.v_proj.a", "self_attn.v_proj.b",
              "self_attn.q_proj.weight", "self_attn.q_proj.bias", "self_attn.q_proj.a", "self_attn.q_proj.b",
              "self_attn.out_proj.weight", "self_attn.out_proj.bias", "self_attn.out_proj.a",
              "self_attn_layer_norm.weight", "self_attn_layer_norm.bias",
              "fc1.weight", "fc1.bias", "fc1.a", "fc1.b", "fc2.weight", "fc2.bias", "fc2.a",
              "final_layer_norm.weight", "final_layer_norm.bias"}


@torch.no_grad()
def test_state_dict_round_trip_runs_on_gpu():
    cfg = OPTConfigLite(hidden_size=256, num_hidden_layers=2, ffn_dim=1024, num_attention_heads=4, vocab_size=512,
                        max_position_embeddings=128)
    torch.manual_seed(0)
    lm = Int8OPTForCausalLM(cfg)
    g = torch.Generator().manual_seed(3)
    for layer in lm.model.decoder.layers:
        randomize_int8_layer(layer, g, 2e-4, 2e-3)
    sd = lm.state_dict()
    keys = {k[len("model.decoder.layers.0."):] for k in sd if k.startswith("model.decoder.layers.0.")}
    assert keys == LAYER_KEYS, keys ^ LAYER_KEYS
    assert sd["model.decoder.layers.0.self_attn.q_proj.weight"].dtype == torch.int8
    assert sd["model.decoder.layers.0.self_attn.q_proj.bias"].shape == (1, 256)
    assert sd["model.decoder.layers.0.fc2.bias"].dtype == torch.float32 and sd["model.decoder.layers.0.fc1.a"].dim() == 0
    assert sd["lm_head.weight"].data_ptr() == sd["model.decoder.embed_tokens.weight"].data_ptr()   # tied
    # what an exported checkpoint holds: tied weights stored once; through a file and the safe loader
    sd = {k: v for k, v in sd.items() if k != "lm_head.weight"}
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    loaded = torch.load(buf, weights_only=True)
    torch.manual_seed(1)
    fresh = Int8OPTForCausalLM(cfg)
    missing = fresh.load_state_dict(loaded, strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys
    assert fresh.lm_head.weight.data_ptr() == fresh.model.decoder.embed_tokens.weight.data_ptr()
    ids = torch.randint(2, 512, (2, 37), generator=g)
    _say("state dict: original on GPU")
    a = copy.deepcopy(lm).to(DEV)(ids.to(DEV), use_cache=True)
    _say("state dict: loaded copy on GPU")
    glm = fresh.to(DEV)
    b = glm(ids.to(DEV), use_cache=True)
    assert torch.equal(a.logits, b.logits)
    with oracle_backend():
        ref = lm(ids, use_cache=True)
    assert ((b.logits.cpu() - ref.logits).abs().max() / ref.logits.abs().max()).item() <= 2e-3
    step_a = glm(ids[:, -1:].to(DEV), past_key_values=b.past_key_values, use_cache=True)
    with oracle_backend():
        step_ref = lm(ids[:, -1:], past_key_values=ref.past_key_values, use_cache=True)
    assert ((step_a.logits.cpu() - step_ref.logits).abs().max() / step_ref.logits.abs().max()).item() <= 2e-3


@torch.no_grad()
def test_weight_only_layers_on_gpu():
    # W8A16Linear / W8FakeA8Linear: int8 weights, floating-point activations (torch ops only; no INT8 kernel)
    torch.manual_seed(0)
    lin = nn.Linear(512, 768)
    x = torch.randn(4, 33, 512)
    y_gt = lin(x)
    for make in (lambda: W8A16Linear.from_float(clone_linear(lin)),
                 lambda: W8A16Linear.from_float(clone_linear(lin), weight_quant="per_tensor"),
                 lambda: W8FakeA8Linear.from_float(clone_linear(lin), act_quant="per_token"),
                 lambda: W8FakeA8Linear.from_float(clone_linear(lin), act_quant="per_tensor")):
        m = make()
        _say("weight-only layer", type(m).__name__)
        y_cpu = m(x.clone())
        mg = copy.deepcopy(m).to(DEV)
        assert mg.weight.is_cuda and mg.weight.dtype == torch.int8
        y32 = mg(x.clone().to(DEV))
        assert y32.dtype == torch.float32 and _rmse2(y_cpu, y32.cpu()) < 1e-6
        assert _rmse2(y_gt, y32.cpu()) < 2e-3
        y16 = mg.half()(x.clone().to(DEV).half())      # the int8 weight survives .half()
        assert y16.dtype == torch.float16 and mg.weight.dtype == torch.int8
        assert _rmse2(y_gt, y16.float().cpu()) < 3e-3

"""Host-side logic of torch_int.nn and torch_int.models.opt, on CPU, with the nine native
entry points swapped for the oracle (tests/_oracle_backend.py).  What is pinned here:
buffer names / shapes / dtypes (state-dict compatibility with upstream), from_float
algebra, flatten/unflatten, the attention/decoder wiring against an independent per-head
computation, pad-to-16 and the KV-cache path."""
import math

import pytest
import torch
from torch import nn

from _float_opt import FloatOPTAttention as _FloatOPTAttention
from _float_opt import FloatOPTDecoderLayer as _FloatOPTDecoderLayer
from _float_opt import clone_linear as _clone_linear
from _oracle_backend import causal_mask, oracle_backend, randomize_int8_layer
from oracle import oracle as orc
from torch_int.models.opt import (Int8OPTAttention, Int8OPTDecoder, Int8OPTDecoderLayer, Int8OPTForCausalLM,
                                  Int8OPTModel, OPTConfigLite, OPTLearnedPositionalEmbedding)
from torch_int.nn import (BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T, BMM_S8T_S8N_S32T, DQ_Add_LayerNorm_Q, LayerNormQ,
                          W8A8B8O8Linear, W8A8B8O8LinearReLU, W8A8B32O32Linear, W8A8B32O32LinearWithoutScaling,
                          W8A8BFP32OFP32Linear)


def _s8(g, *shape):
    return torch.randint(-127, 128, shape, dtype=torch.int8, generator=g)


# ------------------------------------------------------------------ buffers / state dict

def test_linear_buffers_match_upstream_layout():
    # upstream nn/linear.py:23-28,116-119,139-144,189-193
    expect = {
        W8A8B8O8Linear: {"weight": torch.int8, "bias": torch.int8, "a": torch.float32, "b": torch.float32},
        W8A8B8O8LinearReLU: {"weight": torch.int8, "bias": torch.int8, "a": torch.float32, "b": torch.float32},
        W8A8B32O32LinearWithoutScaling: {"weight": torch.int8, "bias": torch.int32},
        W8A8B32O32Linear: {"weight": torch.int8, "bias": torch.int32, "a": torch.float32, "b": torch.float32},
        W8A8BFP32OFP32Linear: {"weight": torch.int8, "bias": torch.float32, "a": torch.float32},
    }
    for cls, keys in expect.items():
        m = cls(48, 32)
        sd = m.state_dict()
        assert {k: v.dtype for k, v in sd.items()} == keys, cls.__name__
        assert sd["weight"].shape == (32, 48) and sd["bias"].shape == (1, 32)
        assert all(sd[k].dim() == 0 for k in keys if k in ("a", "b"))
        assert int(sd["weight"].min()) >= -127 and int(sd["weight"].max()) <= 126  # randint(-127, 127)
        m2 = cls(48, 32)
        m2.load_state_dict(sd)
        assert all(torch.equal(a, b) for a, b in zip(m2.state_dict().values(), sd.values()))
    assert list(BMM_S8T_S8N_S8T(0.5).state_dict()) == ["a"] and list(BMM_S8T_S8N_F32T(0.5).state_dict()) == ["a"]
    assert list(BMM_S8T_S8N_S32T().state_dict()) == []
    assert {k: v.dtype for k, v in LayerNormQ(16).state_dict().items()} == \
        {"weight": torch.float32, "bias": torch.float32}


def test_fp32_bias_survives_half_and_int_buffers_survive_dtype_casts():
    m = W8A8BFP32OFP32Linear(16, 8).half()
    assert m.bias.dtype == torch.float32 and m.weight.dtype == torch.int8 and m.a.dtype == torch.float16
    m = W8A8BFP32OFP32Linear(16, 8).to(torch.float16)
    assert m.bias.dtype == torch.float32 and m.weight.dtype == torch.int8
    m = W8A8B8O8Linear(16, 8).to(torch.float16)
    assert m.weight.dtype == torch.int8 and m.bias.dtype == torch.int8


def test_opt_state_dict_keys():
    cfg = OPTConfigLite(hidden_size=32, num_hidden_layers=2, ffn_dim=64, num_attention_heads=4, vocab_size=50,
                        max_position_embeddings=40)
    keys = set(Int8OPTForCausalLM(cfg).state_dict())
    for k in ["model.decoder.embed_tokens.weight", "model.decoder.embed_positions.weight",
              "model.decoder.final_layer_norm.weight", "lm_head.weight",
              "model.decoder.layers.1.self_attn.q_proj.weight", "model.decoder.layers.1.self_attn.q_proj.a",
              "model.decoder.layers.1.self_attn.q_proj.b", "model.decoder.layers.0.self_attn.out_proj.a",
              "model.decoder.layers.0.self_attn.qk_bmm.a", "model.decoder.layers.0.self_attn.pv_bmm.a",
              "model.decoder.layers.0.self_attn_layer_norm.weight", "model.decoder.layers.0.final_layer_norm.bias",
              "model.decoder.layers.0.fc1.bias", "model.decoder.layers.0.fc2.a"]:
        assert k in keys, k
    assert "model.decoder.layers.0.self_attn.out_proj.b" not in keys  # upstream nn/linear.py:189-193
    assert Int8OPTForCausalLM(cfg).model.decoder.embed_positions.weight.shape == (42, 32)  # +2 offset rows


# ------------------------------------------------------------------ forward = one entry point

@pytest.mark.parametrize("cls,ref", [(W8A8B8O8Linear, orc.linear_a8_w8_b8_o8),
                                     (W8A8B8O8LinearReLU, orc.linear_relu_a8_w8_b8_o8),
                                     (W8A8B32O32Linear, orc.linear_a8_w8_b32_o32_with_scaling)])
def test_scaled_linear_modules_flatten_and_pass_scales(cls, ref):
    g = torch.Generator().manual_seed(1)
    m = cls(64, 48, alpha=0.003, beta=0.02)
    m.weight = _s8(g, 48, 64)
    m.bias = (_s8(g, 1, 48) if m.bias.dtype == torch.int8 else
              torch.randint(-10 ** 6, 10 ** 6, (1, 48), dtype=torch.int32, generator=g))
    x = _s8(g, 2, 5, 64)
    with oracle_backend():
        y = m(x)
        assert y.shape == (2, 5, 48)
        assert torch.equal(y.view(10, 48), ref(x.view(10, 64), m.weight, m.bias, 0.003, 0.02))
        m.a = torch.tensor(0.001)  # replacing the buffer must invalidate the cached scalar
        assert torch.equal(m(x).view(10, 48), ref(x.view(10, 64), m.weight, m.bias, 0.001, 0.02))
        m.b.fill_(0.5)             # so must an in-place update
        assert torch.equal(m(x).view(10, 48), ref(x.view(10, 64), m.weight, m.bias, 0.001, 0.5))


def test_unscaled_and_fp32_linear_modules():
    g = torch.Generator().manual_seed(2)
    x = _s8(g, 3, 4, 32)
    m = W8A8B32O32LinearWithoutScaling(32, 16)
    m.bias = torch.randint(-1000, 1000, (1, 16), dtype=torch.int32, generator=g)
    f = W8A8BFP32OFP32Linear(32, 16, alpha=0.004)
    f.bias = torch.randn(1, 16, generator=g)
    with oracle_backend():
        assert torch.equal(m(x).view(12, 16), orc.linear_a8_w8_b32_o32(x.view(12, 32), m.weight, m.bias))
        # beta is always 1 (upstream nn/linear.py:213-214)
        assert torch.equal(f(x).view(12, 16), orc.linear_a8_w8_bfp32_ofp32(x.view(12, 32), f.weight, f.bias, 0.004, 1))


def test_weight_only_linear_modules():
    # W8A16Linear / W8FakeA8Linear (upstream nn/linear.py:232-337): pure torch, no INT8 kernel involved
    from torch_int.nn.linear import W8A16Linear, W8FakeA8Linear
    torch.manual_seed(0)
    lin = torch.nn.Linear(64, 48)
    x = torch.randn(5, 7, 64)
    y_gt = lin(x)
    for quant in ("per_channel", "per_tensor"):
        m = W8A16Linear.from_float(_clone_linear(lin), weight_quant=quant)
        assert m.weight.dtype == torch.int8 and m.bias.dtype == torch.float16 and m.bias.shape == (48,)
        assert set(m.state_dict()) == {"weight", "bias", "weight_scales"}
        y = m(x.clone())
        assert y.shape == y_gt.shape
        assert ((y - y_gt) ** 2).mean() / (y_gt ** 2).mean() < 1e-3, quant
    with pytest.raises(ValueError):
        W8A16Linear.from_float(_clone_linear(lin), weight_quant="per_row")
    for act in ("per_token", "per_tensor"):
        m = W8FakeA8Linear.from_float(_clone_linear(lin), act_quant=act)
        y = m(x.clone())
        assert ((y - y_gt) ** 2).mean() / (y_gt ** 2).mean() < 2e-3, act
    with pytest.raises(ValueError):
        W8FakeA8Linear(8, 8, act_quant="per_block")
    m = W8A16Linear(16, 8, bias=False)
    assert m.bias is None and m(torch.randn(3, 16)).shape == (3, 8)
    # the fake-quantised activations lie on the int8 grid of their row scale
    t = torch.randn(4, 64)
    scale = t.abs().max(dim=-1, keepdim=True)[0] / 127
    q = W8FakeA8Linear(64, 8).activation_fake_quantizer(t.clone()) / scale
    assert torch.allclose(q, q.round(), atol=1e-4) and q.abs().max() <= 127.001


def test_bmm_modules_and_from_scale():
    g = torch.Generator().manual_seed(3)
    a, b = _s8(g, 2, 5, 16), _s8(g, 2, 7, 16)
    with oracle_backend():
        m = BMM_S8T_S8N_S8T.from_scale(0.1, 0.2, 0.5)
        assert math.isclose(m.a.item(), 0.1 * 0.2 / 0.5, rel_tol=1e-6)
        assert torch.equal(m(a, b), orc.bmm_s8t_s8n_s8t(a, b, m.a.item()))
        m = BMM_S8T_S8N_F32T.from_scale(torch.tensor(0.1), 0.2)
        assert math.isclose(m.a.item(), 0.02, rel_tol=1e-6)
        assert torch.equal(m(a, b), orc.bmm_s8t_s8n_f32t(a, b, m.a.item()))
        assert torch.equal(BMM_S8T_S8N_S32T()(a, b), orc.bmm_s8t_s8n_s32t(a, b))


def test_layernorm_modules():
    g = torch.Generator().manual_seed(4)
    ln = nn.LayerNorm(64)
    ln.weight.data = 1 + 0.1 * torch.randn(64, generator=g)
    ln.bias.data = 0.1 * torch.randn(64, generator=g)
    q = LayerNormQ.from_float(ln, 0.05)
    assert torch.allclose(q.weight, ln.weight / 0.05) and torch.allclose(q.bias, ln.bias / 0.05) and q.eps == ln.eps
    x = torch.randn(3, 7, 64, generator=g)
    y = q(x)
    assert y.dtype == torch.int8 and y.shape == x.shape
    assert torch.equal(y, (ln(x) / 0.05).round().clamp(-128, 127).to(torch.int8)) or \
        (y.int() - (ln(x) / 0.05).round().clamp(-128, 127).int()).abs().max() <= 1
    assert torch.equal(q(x.half()), q(x.half().float()))  # input is promoted to fp32 first
    d = DQ_Add_LayerNorm_Q(64)
    d.input_scale = 0.01
    d.weight, d.bias = q.weight, q.bias
    inp = torch.randint(-65536, 65536, (3, 7, 64), dtype=torch.int32, generator=g)
    with oracle_backend():
        r, yq = d(x, inp)  # residual first, int32 second (upstream nn/fused.py:37-43)
    r_ref, q_ref = orc.dq_add_layernorm_q(inp, 0.01, x, q.weight.detach(), q.bias.detach(), 1e-5)
    assert torch.equal(r, r_ref) and torch.equal(yq, q_ref)


# ------------------------------------------------------------------ from_float

def test_linear_from_float_algebra_and_accuracy():
    # upstream tests/test_linear_modules.py: x ~ N(0,1) [128,512], Linear(512,1024), absmax scales
    torch.manual_seed(0)
    lin = nn.Linear(512, 1024)
    x = torch.randn(128, 512)
    y_gt = lin(x).detach()
    x_scale = x.abs().max() / 127
    q_x = (x / x_scale).round().to(torch.int8)
    w_scale = (lin.weight.abs().max() / 127).item()
    with oracle_backend():
        for cls in (W8A8B8O8Linear, W8A8B8O8LinearReLU):
            ref = y_gt.clamp(min=0) if cls is W8A8B8O8LinearReLU else y_gt
            y_scale = ref.abs().max() / 127
            m = cls.from_float(_clone_linear(lin), x_scale, y_scale)
            assert math.isclose(m.a.item(), x_scale.item() * w_scale / y_scale.item(), rel_tol=1e-5)
            assert m.weight.dtype == torch.int8 and m.bias.dtype == torch.int8
            y = m(q_x).float() * y_scale
            r2 = ((ref - y) ** 2).mean() / (ref ** 2).mean()
            assert r2 < 2e-3, (cls.__name__, r2.item())
        m = W8A8BFP32OFP32Linear.from_float(_clone_linear(lin), x_scale)
        assert math.isclose(m.a.item(), x_scale.item() * w_scale, rel_tol=1e-5) and m.bias.dtype == torch.float32
        r2 = ((y_gt - m(q_x)) ** 2).mean() / (y_gt ** 2).mean()
        assert r2 < 1e-3, r2.item()
        y_scale = y_gt.abs().max() / (2 ** 31 - 1)
        m = W8A8B32O32Linear.from_float(_clone_linear(lin), x_scale, y_scale)
        assert m.bias.dtype == torch.int32
        r2 = ((y_gt - m(q_x).float() * y_scale) ** 2).mean() / (y_gt ** 2).mean()
        assert r2 < 1e-3, r2.item()


@torch.no_grad()
def test_attention_from_float_tracks_the_float_module():
    # upstream tests/test_opt_attention.py (B,L,D,H = 1,16,16,1), plus a multi-head case
    for (B, L, D, H) in [(1, 16, 16, 1), (2, 32, 64, 4)]:
        torch.manual_seed(0)
        fp = _FloatOPTAttention(D, H).requires_grad_(False)
        x = torch.randn(B, L, D)
        x_scale = x.abs().max().item() / 127
        y_gt = fp(x)
        rec = {}
        h = x
        rec["q"] = fp.q_proj(h).abs().max().item() / 127
        rec["k"] = fp.k_proj(h).abs().max().item() / 127
        rec["v"] = fp.v_proj(h).abs().max().item() / 127
        q = (fp.q_proj(h) * fp.scaling).view(B, L, H, D // H).transpose(1, 2)
        k = fp.k_proj(h).view(B, L, H, D // H).transpose(1, 2)
        v = fp.v_proj(h).view(B, L, H, D // H).transpose(1, 2)
        ctx = (torch.softmax(q @ k.transpose(-1, -2), -1) @ v).transpose(1, 2).reshape(B, L, D)
        rec["o"] = ctx.abs().max().item() / 127
        # note: like upstream, the converter folds 1/sqrt(d) into fp.q_proj and then quantises the
        # fp weights in place, so `fp` is consumed by this call
        int8 = Int8OPTAttention.from_float(fp, x_scale, rec["q"], rec["k"], rec["v"], rec["o"])
        assert math.isclose(int8.qk_bmm.a.item(), rec["q"] * (D // H) ** -0.5 * rec["k"], rel_tol=1e-5)
        assert math.isclose(int8.pv_bmm.a.item(), rec["v"] / 127 / rec["o"], rel_tol=1e-5)
        q_x = (x / x_scale).round().to(torch.int8)
        with oracle_backend():
            y, probs, (k_c, v_c) = int8(q_x)
        assert y.dtype == torch.float32 and probs is None
        assert k_c.shape == (B, H, L, D // H) and k_c.dtype == torch.int8 and v_c.shape == k_c.shape
        r2 = ((y_gt - y) ** 2).mean() / (y_gt ** 2).mean()
        assert r2 < 5e-3, r2.item()


@torch.no_grad()
def test_decoder_layer_from_float_tracks_the_float_module():
    torch.manual_seed(0)
    D, H, F, B, T = 64, 4, 256, 2, 48
    fp = _FloatOPTDecoderLayer(D, H, F).requires_grad_(False)
    x = torch.randn(B, T, D)
    mask = causal_mask(B, T, T)
    scales = {}
    y_gt = fp(x, mask, record=scales)
    int8 = Int8OPTDecoderLayer.from_float(fp, **scales)
    hidden = x.clone()
    with oracle_backend():
        out = int8(hidden, attention_mask=mask)
    assert out[0] is hidden  # the residual stream is updated in place (upstream models/opt.py:281,289)
    r2 = ((y_gt - out[0]) ** 2).mean() / (y_gt ** 2).mean()
    assert r2 < 5e-3, r2.item()


# ------------------------------------------------------------------ wiring against an independent computation

@torch.no_grad()
def _attention_per_head(layer, x_q, mask):
    """Int8OPTAttention restated head by head with explicit int64 matmuls and the oracle's
    epilogues; shares no reshape/transpose code with the module."""
    B, T, D = x_q.shape
    a = layer
    H, d = a.num_heads, a.head_dim

    def proj(lin, x2d):
        acc = (x2d.long() @ lin.weight.long().T).to(torch.int32)
        return orc.epi_b8_o8(acc, lin.bias.reshape(-1), lin.a.item(), lin.b.item())

    out_ctx = torch.empty(B, T, D, dtype=torch.int8)
    for b in range(B):
        q, k, v = (proj(l, x_q[b]) for l in (a.q_proj, a.k_proj, a.v_proj))
        for h in range(H):
            sl = slice(h * d, (h + 1) * d)
            s = orc.epi_f32t((q[:, sl].long() @ k[:, sl].long().T).to(torch.int32), a.qk_bmm.a.item())
            s = torch.clamp_min(s + mask[b, 0], torch.finfo(torch.float32).min)
            p = (torch.softmax(s, -1) * 127).round().to(torch.int8)
            out_ctx[b, :, sl] = orc.epi_s8t((p.long() @ v[:, sl].long()).to(torch.int32), a.pv_bmm.a.item())
    acc = (out_ctx.view(B * T, D).long() @ a.out_proj.weight.long().T).to(torch.int32)
    return orc.epi_bfp32_ofp32(acc, a.out_proj.bias.reshape(-1), a.out_proj.a.item(), 1.0).view(B, T, D)


@torch.no_grad()
def test_attention_and_layer_wiring():
    g = torch.Generator().manual_seed(5)
    D, H, F, B, T = 64, 4, 128, 2, 24
    layer = randomize_int8_layer(Int8OPTDecoderLayer(D, H, F), g, 2e-4, 2e-3)
    x_q = _s8(g, B, T, D)
    mask = causal_mask(B, T, T)
    with oracle_backend():
        y, probs, (k_c, v_c) = layer.self_attn(x_q, attention_mask=mask, output_attentions=True)
    ref = _attention_per_head(layer.self_attn, x_q, mask)
    assert torch.equal(y, ref)
    # upstream returns the probabilities after its in-place *127 and round (models/opt.py:166-178)
    assert probs.shape == (B, H, T, T) and probs.max() <= 127 and torch.equal(probs, probs.round())
    assert torch.equal(probs.triu(1), torch.zeros_like(probs))  # causal
    # whole layer: residual stream algebra
    hidden = torch.randn(B, T, D, generator=g)
    h0 = hidden.clone()
    with oracle_backend():
        out, = layer(hidden, attention_mask=mask)
        a_in = layer.self_attn_layer_norm(h0)
        r1 = h0 + _attention_per_head(layer.self_attn, a_in, mask)
        f_in = layer.final_layer_norm(r1)
        r2 = r1 + layer.fc2(layer.fc1(f_in))
    assert torch.equal(out, r2)


@torch.no_grad()
def test_kv_cache_decode_matches_full_prefill():
    g = torch.Generator().manual_seed(6)
    D, H, F, B, T = 64, 4, 128, 2, 21  # src_len is not a multiple of 16: beyond what upstream's kernels accept
    layer = randomize_int8_layer(Int8OPTDecoderLayer(D, H, F), g, 2e-4, 2e-3)
    hidden = torch.randn(B, T + 1, D, generator=g)
    with oracle_backend():
        full, = layer(hidden.clone(), attention_mask=causal_mask(B, T + 1, T + 1))
        pre = layer(hidden[:, :T].clone(), attention_mask=causal_mask(B, T, T), use_cache=True)
        assert pre[1][0].shape == (B, H, T, D // H)
        step = layer(hidden[:, T:].clone(), attention_mask=causal_mask(B, 1, T + 1), use_cache=True,
                     past_key_value=pre[1])
    assert step[1][0].shape == (B, H, T + 1, D // H)
    assert torch.equal(pre[0], full[:, :T])
    assert torch.allclose(step[0], full[:, T:], rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------ decoder / model scaffolding

def test_learned_positions_and_decoder_padding():
    emb = OPTLearnedPositionalEmbedding(32, 8)
    mask = torch.tensor([[1, 1, 1, 0], [0, 1, 1, 1]])
    pos = emb(mask)
    assert torch.equal(pos[0, 1], emb.weight[3]) and torch.equal(pos[1, 1], emb.weight[2])  # +2 offset
    assert torch.equal(pos[0, 3], emb.weight[1])  # padded slot -> index -1 + 2
    assert torch.equal(emb(mask, 2)[0, 0], emb.weight[4])

    cfg = OPTConfigLite(hidden_size=32, num_hidden_layers=2, ffn_dim=64, num_attention_heads=4, vocab_size=60,
                        max_position_embeddings=64)
    torch.manual_seed(0)
    dec = Int8OPTDecoder(cfg)
    g = torch.Generator().manual_seed(7)
    for layer in dec.layers:
        randomize_int8_layer(layer, g, 2e-4, 2e-3)
    ids = torch.randint(2, 60, (2, 23), generator=g)  # 23 -> padded to 32 (upstream models/opt.py:375-383)
    with oracle_backend():
        out = dec(ids)
        assert out.last_hidden_state.shape == (2, 23, 32)
        out_c = dec(ids, use_cache=True)
        assert out_c.past_key_values[0][0].shape == (2, 4, 32, 8)  # the cache holds the padded length
        # padding sits after the real tokens and is causally invisible to them
        ids32 = torch.cat([ids, torch.full((2, 9), 1)], dim=1)
        m32 = torch.cat([torch.ones(2, 23), torch.zeros(2, 9)], dim=1)
        out32 = dec(ids32, attention_mask=m32)
    assert torch.equal(out32.last_hidden_state[:, :23], out.last_hidden_state)


@torch.no_grad()
def test_causal_lm_prefill_then_decode():
    cfg = OPTConfigLite(hidden_size=32, num_hidden_layers=2, ffn_dim=64, num_attention_heads=4, vocab_size=60,
                        max_position_embeddings=64)
    torch.manual_seed(0)
    lm = Int8OPTForCausalLM(cfg)
    assert isinstance(lm.model, Int8OPTModel) and lm.get_decoder() is lm.model.decoder
    g = torch.Generator().manual_seed(8)
    for layer in lm.model.decoder.layers:
        randomize_int8_layer(layer, g, 2e-4, 2e-3)
    ids = torch.randint(2, 60, (2, 16), generator=g)
    with oracle_backend():
        out = lm(ids, use_cache=True)
        assert out.logits.shape == (2, 16, 60) and len(out.past_key_values) == 2
        nxt = out.logits[:, -1].argmax(-1, keepdim=True)
        step = lm(nxt, past_key_values=out.past_key_values, use_cache=True)
        assert step.logits.shape == (2, 1, 60) and step.past_key_values[0][0].shape[2] == 17
        full = lm(torch.cat([ids, nxt], dim=1))
        loss = lm(ids, labels=ids).loss
    assert torch.allclose(step.logits[:, 0], full.logits[:, 16], rtol=1e-4, atol=1e-4)
    assert loss.dim() == 0 and torch.isfinite(loss)


def test_kv_cache_append_in_place_semantics():
    # _kv_append must behave like torch.cat for every caller, however the cache tensors are reused
    from torch_int.models.opt import _kv_append
    g = torch.Generator().manual_seed(5)

    def rnd(*shape):
        return torch.randint(-127, 128, shape, dtype=torch.int8, generator=g)
    past, t1, t2, t3 = rnd(2, 3, 10, 8), rnd(2, 3, 1, 8), rnd(2, 3, 1, 8), rnd(2, 3, 2, 8)
    a = _kv_append(past, t1)                       # no buffer yet: copies into one with spare room
    assert torch.equal(a, torch.cat([past, t1], 2)) and not a.is_contiguous() and a._ti_kv.buf.shape[2] >= 11 + 64
    b = _kv_append(a, t2)                          # appended behind a, same storage
    assert b.data_ptr() == a.data_ptr() and torch.equal(b, torch.cat([past, t1, t2], 2))
    assert torch.equal(a, torch.cat([past, t1], 2))
    c = _kv_append(a, t3)                          # a second continuation of a: must not disturb b
    assert c.data_ptr() != b.data_ptr()
    assert torch.equal(c, torch.cat([past, t1, t3], 2)) and torch.equal(b, torch.cat([past, t1, t2], 2))
    d = _kv_append(b[:, :, :11], t3)               # a slice made by the caller carries no buffer: plain copy
    assert torch.equal(d, torch.cat([past, t1, t3], 2)) and torch.equal(b, torch.cat([past, t1, t2], 2))
    e = b
    for _ in range(200):                           # growth beyond the spare room re-allocates, values survive
        e = _kv_append(e, t1)
    assert e.shape[2] == 212 and torch.equal(e[:, :, :12], b) and torch.equal(e[:, :, -1:], t1)
    f = _kv_append(b.index_select(0, torch.tensor([1, 0])), t2)   # beam-search style re-ordering
    assert torch.equal(f, torch.cat([b.index_select(0, torch.tensor([1, 0])), t2], 2))


def test_decode_with_in_place_cache_matches_concatenation():
    from torch_int.models.opt import Int8OPTAttention
    cfg = OPTConfigLite(hidden_size=64, num_hidden_layers=2, ffn_dim=128, num_attention_heads=4, vocab_size=97,
                        max_position_embeddings=64)
    torch.manual_seed(3)
    lm = Int8OPTForCausalLM(cfg).eval()
    g = torch.Generator().manual_seed(4)
    for layer in lm.model.decoder.layers:
        randomize_int8_layer(layer, g, 2e-3, 8e-3)
    ids = torch.randint(2, 97, (2, 9), generator=g)
    outs = {}
    with oracle_backend():
        for mode in (True, False):
            Int8OPTAttention.kv_cache_in_place = mode
            try:
                o = lm(ids[:, :5], use_cache=True)
                steps = [o.logits]
                for t in range(5, 9):
                    o = lm(ids[:, t:t + 1], past_key_values=o.past_key_values, use_cache=True)
                    steps.append(o.logits)
                outs[mode] = (steps, o.past_key_values)
            finally:
                Int8OPTAttention.kv_cache_in_place = True
    for x, y in zip(outs[True][0], outs[False][0]):
        assert torch.equal(x, y)
    for (k1, v1), (k2, v2) in zip(outs[True][1], outs[False][1]):
        assert k1.shape[2] == 20 and torch.equal(k1, k2) and torch.equal(v1, v2)  # 5 tokens padded to 16, then 4 steps
        assert not k1.is_contiguous() and k2.is_contiguous()


def test_causal_lm_ties_lm_head_and_loads_a_checkpoint_without_it():
    # upstream's post_init ties lm_head to the token embedding; exported checkpoints store the tensor once
    cfg = OPTConfigLite(hidden_size=32, num_hidden_layers=1, ffn_dim=64, num_attention_heads=4, vocab_size=60,
                        max_position_embeddings=64)
    torch.manual_seed(0)
    lm = Int8OPTForCausalLM(cfg)
    assert lm.lm_head.weight is lm.model.decoder.embed_tokens.weight
    sd = {k: v.clone() for k, v in lm.state_dict().items() if k != "lm_head.weight"}
    torch.manual_seed(1)
    other = Int8OPTForCausalLM(cfg)
    res = other.load_state_dict(sd, strict=True)
    assert not res.missing_keys and not res.unexpected_keys
    assert torch.equal(other.lm_head.weight, lm.model.decoder.embed_tokens.weight)
    assert other.lm_head.weight is other.model.decoder.embed_tokens.weight
    # a checkpoint that does carry an untied head keeps it apart when the config says so
    cfg2 = OPTConfigLite(hidden_size=32, num_hidden_layers=1, ffn_dim=64, num_attention_heads=4, vocab_size=60,
                         max_position_embeddings=64)
    cfg2.tie_word_embeddings = False
    untied = Int8OPTForCausalLM(cfg2)
    assert untied.lm_head.weight is not untied.model.decoder.embed_tokens.weight

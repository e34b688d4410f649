"""Test helper: plain fp32 OPT blocks with the attribute names the int8 converters read (``from_float``), and the
absmax calibration upstream's tests use (tests/test_opt_decoder_layer.py:33-41)."""
import torch
from torch import nn


def clone_linear(lin):
    c = nn.Linear(lin.in_features, lin.out_features)
    c.load_state_dict(lin.state_dict())
    return c.requires_grad_(False)


class FloatOPTAttention(nn.Module):
    """Plain fp32 OPT self-attention (attribute names the int8 converter reads)."""

    def __init__(self, embed_dim, num_heads):
        super().__init__()
        self.embed_dim, self.num_heads, self.head_dim = embed_dim, num_heads, embed_dim // num_heads
        self.scaling = self.head_dim ** -0.5
        self.q_proj, self.k_proj = nn.Linear(embed_dim, embed_dim), nn.Linear(embed_dim, embed_dim)
        self.v_proj, self.out_proj = nn.Linear(embed_dim, embed_dim), nn.Linear(embed_dim, embed_dim)

    def forward(self, x, mask=None):
        B, T, D = x.shape
        H, d = self.num_heads, self.head_dim
        q = (self.q_proj(x) * self.scaling).view(B, T, H, d).transpose(1, 2)
        k = self.k_proj(x).view(B, T, H, d).transpose(1, 2)
        v = self.v_proj(x).view(B, T, H, d).transpose(1, 2)
        s = q @ k.transpose(-1, -2)
        if mask is not None:
            s = s + mask
        p = torch.softmax(s, -1)
        return self.out_proj((p @ v).transpose(1, 2).reshape(B, T, D))


class FloatOPTDecoderLayer(nn.Module):
    def __init__(self, embed_dim, num_heads, ffn_dim):
        super().__init__()
        self.embed_dim = embed_dim
        self.self_attn = FloatOPTAttention(embed_dim, num_heads)
        self.self_attn_layer_norm, self.final_layer_norm = nn.LayerNorm(embed_dim), nn.LayerNorm(embed_dim)
        self.fc1, self.fc2 = nn.Linear(embed_dim, ffn_dim), nn.Linear(ffn_dim, embed_dim)

    def forward(self, x, mask=None, record=None):
        h = self.self_attn_layer_norm(x)
        if record is not None:
            record["attn_input_scale"] = h.abs().max().item() / 127
            a = self.self_attn
            record["q_output_scale"] = a.q_proj(h).abs().max().item() / 127
            record["k_output_scale"] = a.k_proj(h).abs().max().item() / 127
            record["v_output_scale"] = a.v_proj(h).abs().max().item() / 127
            B, T, D = h.shape
            q = (a.q_proj(h) * a.scaling).view(B, T, a.num_heads, a.head_dim).transpose(1, 2)
            k = a.k_proj(h).view(B, T, a.num_heads, a.head_dim).transpose(1, 2)
            v = a.v_proj(h).view(B, T, a.num_heads, a.head_dim).transpose(1, 2)
            s = q @ k.transpose(-1, -2) + (mask if mask is not None else 0)
            ctx = (torch.softmax(s, -1) @ v).transpose(1, 2).reshape(B, T, D)
            record["out_input_scale"] = ctx.abs().max().item() / 127
        x = x + self.self_attn(h, mask)
        h = self.final_layer_norm(x)
        if record is not None:
            record["fc1_input_scale"] = h.abs().max().item() / 127
            record["fc2_input_scale"] = torch.relu(self.fc1(h)).abs().max().item() / 127
        return x + self.fc2(torch.relu(self.fc1(h)))

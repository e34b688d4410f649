"""INT8 OPT blocks on the MI355X kernels (upstream ``torch_int/models/opt.py``).

``Int8OPTAttention`` and ``Int8OPTDecoderLayer`` keep upstream's constructor
signatures, sub-module names, scale algebra and forward semantics.  The
decoder / model / causal-LM wrappers carry their own small OPT scaffolding
(token + learned position embeddings with the +2 offset, additive causal
mask, final LayerNorm, fp ``lm_head``) instead of borrowing methods from a
particular ``transformers`` release; any object with OPTConfig's field names
works as ``config``.
"""
import ctypes
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch
from torch import nn

from .. import _hip_ext
from ..nn.bmm import BMM_S8T_S8N_F32T, BMM_S8T_S8N_S8T
from ..nn.fused import LayerNormQ
from ..nn.linear import W8A8B8O8Linear, W8A8B8O8LinearReLU, W8A8BFP32OFP32Linear


class _KVBuffer:
    """Backing store of one growing K or V cache tensor: ``buf`` is [bsz, heads, capacity, head_dim] and the
    first ``filled`` positions hold tokens.  The tensors handed out as ``past_key_value`` are views
    ``buf[:, :, :n]`` that carry a reference to this object."""
    __slots__ = ("buf", "filled")

    def __init__(self, buf, filled):
        self.buf, self.filled = buf, filled


def _kv_room(past, new):
    """The buffer behind ``past`` when ``new`` can be written right after it, else None."""
    kv = getattr(past, "_ti_kv", None)
    S, T = past.shape[2], new.shape[2]
    if (kv is not None and kv.filled == S and S + T <= kv.buf.shape[2] and past.data_ptr() == kv.buf.data_ptr()
            and past.stride() == kv.buf.stride() and past.shape[:2] == new.shape[:2] and past.shape[3] == new.shape[3]
            and past.dtype == new.dtype and past.device == new.device):
        return kv
    return None


def _kv_room_for(past, T):
    """``_kv_room`` for T new positions that will be written by a kernel (there is no tensor to compare with)."""
    kv = getattr(past, "_ti_kv", None)
    S = past.shape[2]
    if (kv is not None and kv.filled == S and S + T <= kv.buf.shape[2] and past.data_ptr() == kv.buf.data_ptr()
            and past.stride() == kv.buf.stride()):
        return kv
    return None


def _kv_fresh(past, T):
    """A new buffer holding ``past`` with room for T + max(64, a quarter of the length) further positions."""
    S = past.shape[2]
    cap = -(-(S + T + max(64, (S + T) // 4)) // 16) * 16
    buf = torch.empty((past.shape[0], past.shape[1], cap, past.shape[3]), dtype=past.dtype, device=past.device)
    buf[:, :, :S].copy_(past)
    return _KVBuffer(buf, S)


def _kv_view(kv, n):
    out = kv.buf[:, :, :n]
    out._ti_kv = kv
    return out


def _kv_append(past, new):
    """``torch.cat([past, new], dim=2)`` for [bsz, heads, len, head_dim] cache tensors without re-copying the
    past: when ``past`` is a view handed out by an earlier call and nothing was appended after it, ``new`` is
    written into the spare room behind it and a longer view of the same buffer is returned; the values
    ``past`` shows never change.  Otherwise (first decode step, a cache that was re-indexed or sliced by the
    caller, a second continuation of the same past, no room left) the result is built in a fresh buffer."""
    S, T = past.shape[2], new.shape[2]
    kv = _kv_room(past, new) or _kv_fresh(past, T)
    kv.buf[:, :, S:S + T].copy_(new)
    kv.filled = S + T
    return _kv_view(kv, S + T)


def _kv_append_pair(past_k, past_v, new_k, new_v):
    """``_kv_append`` for the key and the value cache of one layer, with a single copy kernel when both live
    in HIP buffers of the same shape."""
    S, T = past_k.shape[2], new_k.shape[2]
    if past_v.shape[2] != S or new_v.shape[2] != T:
        return _kv_append(past_k, new_k), _kv_append(past_v, new_v)
    kk = _kv_room(past_k, new_k) or _kv_fresh(past_k, T)
    vv = _kv_room(past_v, new_v) or _kv_fresh(past_v, T)
    if _hip_ext.can_kv_append(new_k, new_v, kk.buf, vv.buf):
        _hip_ext.kv_append(new_k, new_v, kk.buf, vv.buf, S, checked=True)
    else:
        kk.buf[:, :, S:S + T].copy_(new_k)
        vv.buf[:, :, S:S + T].copy_(new_v)
    kk.filled = vv.filled = S + T
    return _kv_view(kk, S + T), _kv_view(vv, S + T)


class Int8OPTAttention(nn.Module):
    """Multi-head self-attention with int8 projections and int8 Q.K^T / P.V products.

    upstream: ``torch_int/models/opt.py:22-199``.

    ``kv_cache_in_place`` (class attribute, default True): the (key, value) tensors returned for
    ``past_key_value`` reuse one buffer with spare room, so a decode step appends its token instead of
    re-copying the whole cache (see ``_kv_append``).  They are then views that are packed per head but not
    across heads; set it to False to get upstream's freshly concatenated contiguous tensors.
    """
    kv_cache_in_place = True
    # False: the probabilities come from upstream's own chain of torch ops between the two products (mask add,
    # clamp, softmax, * 127, round, int8 cast; models/opt.py:144-178) instead of the fused kernels, whose
    # e * (127 / sum) differs from (e / sum) * 127 by one LSB on a small fraction of the probabilities.
    fused_softmax = True

    def __init__(self, embed_dim: int, num_heads: int):
        super().__init__()
        self.embed_dim = embed_dim
        self.num_heads = num_heads
        self.head_dim = embed_dim // num_heads
        if self.head_dim * num_heads != embed_dim:
            raise ValueError(f"embed_dim must be divisible by num_heads (got `embed_dim`: {embed_dim}"
                             f" and `num_heads`: {num_heads}).")
        self.attention_weight_scale = 1.0
        self.qk_bmm = BMM_S8T_S8N_F32T(1.0)
        self.pv_bmm = BMM_S8T_S8N_S8T(1.0)
        self.k_proj = W8A8B8O8Linear(embed_dim, embed_dim)
        self.v_proj = W8A8B8O8Linear(embed_dim, embed_dim)
        self.q_proj = W8A8B8O8Linear(embed_dim, embed_dim)
        self.out_proj = W8A8BFP32OFP32Linear(embed_dim, embed_dim)

    @staticmethod
    @torch.no_grad()
    def from_float(module, input_scale: float, q_output_scale: float, k_output_scale: float,
                   v_output_scale: float, out_input_scale: float):
        """``module`` is an fp OPT attention (attributes embed_dim, num_heads, scaling,
        q/k/v/out_proj).  The 1/sqrt(d) factor is folded into q_proj, in place on ``module``."""
        q = Int8OPTAttention(module.embed_dim, module.num_heads)
        q_output_scale = q_output_scale * module.scaling
        module.q_proj.weight *= module.scaling
        module.q_proj.bias *= module.scaling
        q.q_proj = W8A8B8O8Linear.from_float(module.q_proj, input_scale, q_output_scale)
        q.k_proj = W8A8B8O8Linear.from_float(module.k_proj, input_scale, k_output_scale)
        q.v_proj = W8A8B8O8Linear.from_float(module.v_proj, input_scale, v_output_scale)
        q.out_proj = W8A8BFP32OFP32Linear.from_float(module.out_proj, out_input_scale)
        q.qk_bmm = BMM_S8T_S8N_F32T.from_scale(q_output_scale, k_output_scale)
        # probabilities are quantised with scale 1/127
        q.pv_bmm = BMM_S8T_S8N_S8T.from_scale(1.0 / 127, v_output_scale, out_input_scale)
        return q

    def _qkv_grouped(self, hidden_states):
        """(q, k, v) projections [bsz, tgt, embed] from one grouped call, or None when the three layers are not
        plain W8A8B8O8Linear of one shape on contiguous HIP tensors."""
        q, k, v = self.q_proj, self.k_proj, self.v_proj
        if not (type(q) is W8A8B8O8Linear and type(k) is W8A8B8O8Linear and type(v) is W8A8B8O8Linear):
            return None
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        (wq, bq), (wk, bk), (wv, bv) = q._wb(), k._wb(), v._wb()
        weights, biases = (wq, wk, wv), (bq.reshape(-1), bk.reshape(-1), bv.reshape(-1))
        if not _hip_ext.can_linear_group(x, weights, biases):
            return None
        outs = _hip_ext.linear_a8_w8_b8_o8_group(
            x, weights, biases, (q._scalar("a"), k._scalar("a"), v._scalar("a")),
            (q._scalar("b"), k._scalar("b"), v._scalar("b")), checked=True)
        lead = hidden_states.shape[:-1]
        return tuple(o.view(*lead, -1) for o in outs)

    def _qkv_head_major(self, hidden_states, bsz, tgt_len):
        """(q, k, v), each int8 [bsz, heads, tgt, head_dim] written in that layout by the projection GEMMs
        themselves, or None when the layers or tensors do not qualify."""
        q, k, v = self.q_proj, self.k_proj, self.v_proj
        if not (type(q) is W8A8B8O8Linear and type(k) is W8A8B8O8Linear and type(v) is W8A8B8O8Linear):
            return None
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        H, d = self.num_heads, self.head_dim
        wb = [lin._wb() for lin in (q, k, v)]
        weights, biases = [w for w, _ in wb], [b.reshape(-1) for _, b in wb]
        if not all(_hip_ext.can_linear_heads(x, w, b, bsz, tgt_len, H, d) for w, b in zip(weights, biases)):
            return None
        if (_hip_ext.can_linear_group(x, weights, biases)
                and _hip_ext.linear_group_is_one_launch(x.shape[0], weights[0].shape[0], x.shape[1], len(weights))):
            # one call; widths the 16x16-block tiles divide run as a single persistent launch
            return _hip_ext.linear_a8_w8_b8_o8_group_heads(
                x, weights, biases, [lin._scalar("a") for lin in (q, k, v)], [lin._scalar("b") for lin in (q, k, v)],
                bsz, tgt_len, H, d, checked=True)
        return tuple(_hip_ext.linear_a8_w8_b8_o8_heads(x, w, b, lin._scalar("a"), lin._scalar("b"), bsz, tgt_len, H, d,
                                                       checked=True)
                     for lin, w, b in zip((q, k, v), weights, biases))

    def _shape(self, tensor: torch.Tensor, seq_len: int, bsz: int):
        """[bsz, seq, embed] -> contiguous [bsz, heads, seq, head_dim]."""
        if seq_len < 0:
            seq_len = tensor.numel() // (bsz * self.embed_dim)
        return _hip_ext.split_heads(tensor, bsz, seq_len, self.num_heads, self.head_dim)

    @torch.no_grad()
    def _decode_fused(self, query4, key, value, past_key_value, attention_mask, output_attentions):
        """The whole attention of a decode step (cache append, Q.K^T, softmax-quant, P.V) as one kernel launch,
        or None when the shapes, the cache or the product modules do not allow it; same values as the separate
        steps of ``forward``."""
        past_k, past_v = past_key_value
        if not (type(self.qk_bmm) is BMM_S8T_S8N_F32T and type(self.pv_bmm) is BMM_S8T_S8N_S8T
                and past_k.dim() == 4 and past_v.shape == past_k.shape):
            return None
        bsz, H, T, d = query4.shape
        S0 = past_k.shape[2]
        if not _hip_ext.decode_attention_shape_ok(T, S0 + T, d):
            return None
        kk = _kv_room(past_k, key) or _kv_fresh(past_k, T)
        vv = _kv_room(past_v, value) or _kv_fresh(past_v, T)
        if not _hip_ext.can_decode_attention(query4, key, value, kk.buf, vv.buf, S0, attention_mask):
            return None   # (a buffer made above is simply dropped; the caller builds its own)
        ctx, probs = _hip_ext.decode_attention(query4, key, value, kk.buf, vv.buf, S0, attention_mask,
                                               self.qk_bmm._scalar("a"), self.pv_bmm._scalar("a"),
                                               want_probs=output_attentions, checked=True)
        kk.filled = vv.filled = S0 + T
        present = (_kv_view(kk, S0 + T), _kv_view(vv, S0 + T))
        probs_out = probs.view(bsz, H, T, S0 + T).float() if output_attentions else None
        ctx = _hip_ext.merge_heads(ctx, bsz, H, T, d)
        return self.out_proj(ctx), probs_out, present

    def decode_step_devlen(self, hidden_states, k_buf, v_buf, length, max_length):
        """Self-attention of one new token per sequence (int8 [bsz, 1, embed]) over cache buffers [bsz, heads, cap,
        head_dim] whose length after the append is read from the int32 HIP tensor ``length`` when the kernels run
        (``Int8OPTGraphDecoder`` records this once and replays it).  No mask, no head mask; the values of
        ``forward`` with a cache of ``length - 1`` positions.  Returns the fp32 output of ``out_proj``."""
        bsz, tgt_len, _ = hidden_states.shape
        flat = self._qkv_grouped(hidden_states)
        if flat is None or not (type(self.qk_bmm) is BMM_S8T_S8N_F32T and type(self.pv_bmm) is BMM_S8T_S8N_S8T):
            raise RuntimeError("Int8OPTAttention.decode_step_devlen: needs the stock int8 projections and products "
                               "on contiguous HIP tensors")
        query4, key, value = (self._shape(t, tgt_len, bsz) for t in flat)
        ctx = _hip_ext.decode_attention_devlen(query4, key, value, k_buf, v_buf, length, max_length,
                                               self.qk_bmm._scalar("a"), self.pv_bmm._scalar("a"))
        ctx = _hip_ext.merge_heads(ctx, bsz, self.num_heads, tgt_len, self.head_dim)
        return self.out_proj(ctx)

    def forward(self, hidden_states: torch.Tensor, key_value_states: Optional[torch.Tensor] = None,
                past_key_value: Optional[Tuple[torch.Tensor]] = None,
                attention_mask: Optional[torch.Tensor] = None,
                layer_head_mask: Optional[torch.Tensor] = None, output_attentions: bool = False,
                ) -> Tuple[torch.Tensor, Optional[torch.Tensor], Optional[Tuple[torch.Tensor]]]:
        """hidden_states: int8 [batch, time, channel] -> (fp32 output, probs or None, (k, v) int8 cache)."""
        cross = key_value_states is not None
        bsz, tgt_len, _ = hidden_states.size()
        H, d = self.num_heads, self.head_dim
        if attention_mask is not None and attention_mask.is_cuda and attention_mask.dtype in (torch.float16, torch.bfloat16):
            # the mask of an fp16 model: it is only ever added to the fp32 scores, where type promotion turns it into
            # these same fp32 values; the fused kernels read fp32
            attention_mask = attention_mask.float()

        # Self-attention on HIP tensors takes the q/k/v projections from one of two fused forms: a single
        # grouped launch for decode-sized inputs, or projections whose stores already produce the
        # [bsz, heads, seq, head_dim] layout; both give the values of the plain layers.
        proj = None  # (q, k, v), each [bsz, H, tgt, d]
        if not cross and hidden_states.is_cuda:
            if bsz * tgt_len <= 16:
                flat = self._qkv_grouped(hidden_states)
                if flat is not None:
                    proj = tuple(self._shape(t, tgt_len, bsz) for t in flat)
            else:
                proj = self._qkv_head_major(hidden_states, bsz, tgt_len)
        if proj is not None:
            query4, key, value = proj
        else:
            query4 = self._shape(self.q_proj(hidden_states), tgt_len, bsz)
        if cross and past_key_value is not None:
            key, value = past_key_value
        else:
            if proj is None:
                kv_src = key_value_states if cross else hidden_states
                key = self._shape(self.k_proj(kv_src), -1, bsz)
                value = self._shape(self.v_proj(kv_src), -1, bsz)
            if not cross and past_key_value is not None:
                if (self.kv_cache_in_place and self.fused_softmax and proj is not None and tgt_len <= 4
                        and layer_head_mask is None):
                    fused = self._decode_fused(query4, key, value, past_key_value, attention_mask, output_attentions)
                    if fused is not None:
                        return fused
                if self.kv_cache_in_place:
                    key, value = _kv_append_pair(past_key_value[0], past_key_value[1], key, value)
                else:
                    key = torch.cat([past_key_value[0], key], dim=2)
                    value = torch.cat([past_key_value[1], value], dim=2)
        present = (key, value)

        query = query4.view(bsz * H, -1, d)
        # cache views are packed per head; [bsz, H] merges into one batch dimension either way
        key = key.view(bsz * H, -1, d) if key.is_contiguous() else key.reshape(bsz * H, key.shape[2], d)
        value = value.view(bsz * H, -1, d) if value.is_contiguous() else value.reshape(bsz * H, value.shape[2], d)
        src_len = key.size(1)

        # Beyond 576 keys the fused kernels sweep the keys three times and win through the key tiles a causal mask
        # kills (160 x 2048 x 2048: 0.99 ms against 1.34 ms for the separate kernels; without a mask they are slower), so
        # they are taken for a plain prefill (tgt_len == src_len) only.
        long_ok = src_len <= 576 or tgt_len == src_len
        if (self.fused_softmax and long_ok and layer_head_mask is None and not output_attentions and tgt_len > 16
                and type(self.qk_bmm) is BMM_S8T_S8N_F32T and type(self.pv_bmm) is BMM_S8T_S8N_S8T
                and _hip_ext.can_attn_qk_softmax_q(query, key, attention_mask, bsz, H) and value.is_cuda
                and _hip_ext.attn_prefill_shape_ok(tgt_len, src_len, d)):
            # the whole attention (Q.K^T, softmax-quant, P.V, head merge) in one kernel on V transposed
            vt = _hip_ext.transpose_last2(value.contiguous())
            if _hip_ext.can_attn_prefill(query, key, vt, attention_mask, bsz, H):
                ctx = _hip_ext.attn_prefill(query, key, vt, attention_mask, self.qk_bmm._scalar("a"),
                                            self.pv_bmm._scalar("a"), H, checked=True)
                return self.out_proj(ctx), None, present
        probs_q = None
        if (self.fused_softmax and long_ok and layer_head_mask is None and tgt_len > 16
                and type(self.qk_bmm) is BMM_S8T_S8N_F32T and _hip_ext.can_attn_qk_softmax_q(query, key, attention_mask, bsz, H)):
            # Q.K^T, mask, clamp, softmax, *127, round and int8 cast in one kernel: the fp32 scores stay in registers
            probs_q = _hip_ext.attn_qk_softmax_q(query, key, attention_mask, self.qk_bmm._scalar("a"), H, checked=True)
            probs_out = probs_q.view(bsz, H, tgt_len, src_len).float() if output_attentions else None
        elif (not key.is_contiguous() and type(self.qk_bmm) is BMM_S8T_S8N_F32T
                and _hip_ext.can_bmm_strided(query, key)):
            scores = _hip_ext.bmm_s8t_s8n_f32t_strided(query, key, self.qk_bmm._scalar("a"), checked=True)
        else:
            scores = self.qk_bmm(query, key.contiguous())  # fp32 [bsz*H, tgt, src]
        if probs_q is None and scores.size() != (bsz * H, tgt_len, src_len):
            raise ValueError(f"Attention weights should be of size {(bsz * H, tgt_len, src_len)}, but is"
                             f" {scores.size()}")
        if attention_mask is not None and attention_mask.size() != (bsz, 1, tgt_len, src_len):
            raise ValueError(f"Attention mask should be of size {(bsz, 1, tgt_len, src_len)}, but is"
                             f" {attention_mask.size()}")
        if layer_head_mask is not None and layer_head_mask.size() != (H,):
            raise ValueError(f"Head mask for a single layer should be of size {(H,)}, but is"
                             f" {layer_head_mask.size()}")
        if probs_q is not None:
            pass
        elif self.fused_softmax and layer_head_mask is None and _hip_ext.can_fuse_softmax(scores, attention_mask, bsz, H):
            # mask add, clamp, softmax, *127, round and int8 cast in one kernel
            probs_q = _hip_ext.attn_softmax_q(scores, attention_mask, H, checked=True)
            probs_out = probs_q.view(bsz, H, tgt_len, src_len).float() if output_attentions else None
        else:
            if attention_mask is not None:
                scores = scores.view(bsz, H, tgt_len, src_len) + attention_mask
                scores = torch.clamp_min(scores, torch.finfo(scores.dtype).min)
                scores = scores.view(bsz * H, tgt_len, src_len)
            probs = nn.functional.softmax(scores, dim=-1)
            if layer_head_mask is not None:
                probs = (layer_head_mask.view(1, -1, 1, 1) * probs.view(bsz, H, tgt_len, src_len)
                         ).view(bsz * H, tgt_len, src_len)
            probs_out = probs.view(bsz, H, tgt_len, src_len) if output_attentions else None
            # The probabilities are scaled and rounded in place, so with output_attentions the
            # returned view holds round(127 p), which is what upstream returns too
            # (models/opt.py:166-178).
            probs_q = probs.mul_(127).round_().to(torch.int8)
        if tgt_len <= 16 and type(self.pv_bmm) is BMM_S8T_S8N_S8T and _hip_ext.can_bmm_rowmajor(probs_q, value):
            # few query rows (incremental decoding): stream V once, as the cache stores it
            ctx = _hip_ext.bmm_s8t_s8t_s8t(probs_q, value, self.pv_bmm._scalar("a"), checked=True)
        else:
            # P.V with V transposed to [bsz*H, d, src]: (P V) = P . (V^T)^T
            ctx = self.pv_bmm(probs_q, _hip_ext.transpose_last2(value.contiguous()))  # int8 [bsz*H, tgt, d]
        if ctx.size() != (bsz * H, tgt_len, d):
            raise ValueError(f"`attn_output` should be of size {(bsz, H, tgt_len, d)}, but is {ctx.size()}")
        ctx = _hip_ext.merge_heads(ctx, bsz, H, tgt_len, d)
        return self.out_proj(ctx), probs_out, present


class _DecodePlan:
    """``Int8OPTDecoderLayer`` flattened into the structure ``ti_opt_decoder_layer_decode`` reads, plus what it was
    built from: (dict that holds the tensor, its name, the tensor, its version) for every buffer, so that a replaced
    or rewritten buffer is noticed."""
    __slots__ = ("ok", "half", "device", "struct", "addr", "sources", "modules", "embed", "heads", "head_dim", "ffn")

    @staticmethod
    def build(layer, half, device):
        plan = _DecodePlan()
        plan.ok, plan.half, plan.device, plan.sources = False, half, device, []
        at = layer.self_attn
        plan.modules = (at, at.q_proj, at.k_proj, at.v_proj, at.out_proj, at.qk_bmm, at.pv_bmm, layer.fc1, layer.fc2,
                        layer.self_attn_layer_norm, layer.final_layer_norm)
        stock = (type(at.q_proj) is W8A8B8O8Linear and type(at.k_proj) is W8A8B8O8Linear
                 and type(at.v_proj) is W8A8B8O8Linear and type(at.out_proj) is W8A8BFP32OFP32Linear
                 and type(layer.fc1) is W8A8B8O8LinearReLU and type(layer.fc2) is W8A8BFP32OFP32Linear
                 and type(at.qk_bmm) is BMM_S8T_S8N_F32T and type(at.pv_bmm) is BMM_S8T_S8N_S8T
                 and type(layer.self_attn_layer_norm) is LayerNormQ and type(layer.final_layer_norm) is LayerNormQ)
        if not stock:
            return plan
        E, H, d, F = at.embed_dim, at.num_heads, at.head_dim, layer.fc1.out_features
        fdt = torch.float16 if half else torch.float32

        def tensor(mod, name, dtype, numel):
            holder = mod._buffers if mod._buffers.get(name) is not None else mod._parameters
            t = holder.get(name)
            if not (isinstance(t, torch.Tensor) and t.device == device and t.dtype is dtype and t.is_contiguous()
                    and t.numel() == numel and t.data_ptr() % 16 == 0):
                raise _NotStock
            plan.sources.append((holder, name, t, t._version))
            return t.data_ptr()

        def scalar(mod, name):
            value = mod._scalar(name)
            t = mod._buffers.get(name)
            if isinstance(t, torch.Tensor):
                plan.sources.append((mod._buffers, name, t, t._version))
            else:
                raise _NotStock   # a scale that is not a registered buffer cannot be watched
            return value

        try:
            for lin in (at.out_proj, layer.fc2):   # their fp32 bias may still be in the dtype a cast left (see _run)
                _, bias = lin._wb()
                if bias.dtype is not torch.float32:
                    lin.bias = bias.to(torch.float32)
            st = _hip_ext.OptDecodeLayer()
            st.embed, st.heads, st.head_dim, st.ffn, st.half = E, H, d, F, int(half)
            ln1, ln2 = layer.self_attn_layer_norm, layer.final_layer_norm
            st.ln1_eps, st.ln2_eps = float(ln1.eps), float(ln2.eps)
            st.ln1_gamma, st.ln1_beta = tensor(ln1, "weight", fdt, E), tensor(ln1, "bias", fdt, E)
            st.ln2_gamma, st.ln2_beta = tensor(ln2, "weight", fdt, E), tensor(ln2, "bias", fdt, E)
            st.wq, st.wk, st.wv = (tensor(m, "weight", torch.int8, E * E) for m in (at.q_proj, at.k_proj, at.v_proj))
            st.bq, st.bk, st.bv = (tensor(m, "bias", torch.int8, E) for m in (at.q_proj, at.k_proj, at.v_proj))
            st.alpha_q, st.alpha_k, st.alpha_v = (scalar(m, "a") for m in (at.q_proj, at.k_proj, at.v_proj))
            st.beta_q, st.beta_k, st.beta_v = (scalar(m, "b") for m in (at.q_proj, at.k_proj, at.v_proj))
            st.alpha_qk, st.alpha_pv = scalar(at.qk_bmm, "a"), scalar(at.pv_bmm, "a")
            st.wo, st.bo = tensor(at.out_proj, "weight", torch.int8, E * E), tensor(at.out_proj, "bias", torch.float32, E)
            st.alpha_o = scalar(at.out_proj, "a")
            st.w1, st.b1 = tensor(layer.fc1, "weight", torch.int8, F * E), tensor(layer.fc1, "bias", torch.int8, F)
            st.alpha_1, st.beta_1 = scalar(layer.fc1, "a"), scalar(layer.fc1, "b")
            st.w2, st.b2 = tensor(layer.fc2, "weight", torch.int8, E * F), tensor(layer.fc2, "bias", torch.float32, E)
            st.alpha_2 = scalar(layer.fc2, "a")
        except _NotStock:
            return plan
        if H * d != E or at.q_proj.in_features != E or layer.fc2.in_features != F:
            return plan
        plan.struct, plan.addr = st, ctypes.addressof(st)
        plan.embed, plan.heads, plan.head_dim, plan.ffn = E, H, d, F
        plan.ok = True
        return plan


class _NotStock(Exception):
    pass


def _mask_as_fp32(mask):
    """The additive mask as the fused kernels read it: fp32 on the device (None when it is neither that nor an fp16 /
    bf16 HIP tensor).  The mask of an fp16 model is only ever added to fp32 scores (see ``Int8OPTAttention.forward``);
    it is converted once per mask tensor and version, not once per layer."""
    if not mask.is_cuda:
        return None
    if mask.dtype is torch.float32:
        return mask
    if mask.dtype is torch.float16 or mask.dtype is torch.bfloat16:
        m32 = getattr(mask, "_ti_f32", None)
        if m32 is None or m32[0] != mask._version:
            m32 = (mask._version, mask.float())
            mask._ti_f32 = m32
        return m32[1]
    return None


_GLOBAL_FORWARD_HOOKS = torch.nn.modules.module._global_forward_hooks
_GLOBAL_FORWARD_PRE_HOOKS = torch.nn.modules.module._global_forward_pre_hooks


class Int8OPTDecoderLayer(nn.Module):
    """Pre-LN OPT block on an fp residual stream: LayerNormQ -> int8 attention -> add ->
    LayerNormQ -> fc1 (ReLU, int8) -> fc2 (fp32) -> add.  The input tensor is updated in
    place, as upstream does (``torch_int/models/opt.py:202-299``)."""

    def __init__(self, embed_dim, num_attention_heads, ffn_dim):
        super().__init__()
        self.embed_dim = embed_dim
        self.self_attn = Int8OPTAttention(embed_dim=embed_dim, num_heads=num_attention_heads)
        self.self_attn_layer_norm = LayerNormQ(embed_dim)
        self.fc1 = W8A8B8O8LinearReLU(embed_dim, ffn_dim)
        self.fc2 = W8A8BFP32OFP32Linear(ffn_dim, embed_dim)
        self.final_layer_norm = LayerNormQ(embed_dim)

    @staticmethod
    def from_float(module, attn_input_scale: float, q_output_scale: float, k_output_scale: float,
                   v_output_scale: float, out_input_scale: float, fc1_input_scale: float,
                   fc2_input_scale: float):
        q = Int8OPTDecoderLayer(module.embed_dim, module.self_attn.num_heads, module.fc1.out_features)
        q.self_attn_layer_norm = LayerNormQ.from_float(module.self_attn_layer_norm, attn_input_scale)
        q.self_attn = Int8OPTAttention.from_float(module.self_attn, attn_input_scale, q_output_scale,
                                                  k_output_scale, v_output_scale, out_input_scale)
        q.final_layer_norm = LayerNormQ.from_float(module.final_layer_norm, fc1_input_scale)
        q.fc1 = W8A8B8O8LinearReLU.from_float(module.fc1, fc1_input_scale, fc2_input_scale)
        q.fc2 = W8A8BFP32OFP32Linear.from_float(module.fc2, fc2_input_scale)
        return q

    #: one new token per sequence with a KV cache: the layer's kernels are issued from one C call
    #: (``ti_opt_decoder_layer_decode``: the same entry points with the same arguments, so the same values) instead of
    #: one Python call per module; set to False to go through the modules
    decode_in_one_call = True

    def _decode_plan(self, half, device):
        """The layer as ``ti_opt_decoder_layer_decode`` reads it, built once and rebuilt when a tensor it was built from
        has been replaced or written to; None when the layer is not the stock int8 block on ``device``."""
        plan = self.__dict__.get("_ti_decode_plan")
        if plan is not None and plan.half == half and plan.device == device:
            for holder, name, tensor, version in plan.sources:
                if holder.get(name) is not tensor or tensor._version != version:
                    plan = None
                    break
        else:
            plan = None
        if plan is None:
            plan = self.__dict__["_ti_decode_plan"] = _DecodePlan.build(self, half, device)
        if not plan.ok or _GLOBAL_FORWARD_HOOKS or _GLOBAL_FORWARD_PRE_HOOKS:
            return None
        for mod in plan.modules:   # a hook on a sub-module wants to see that module's call
            if mod._forward_hooks or mod._forward_pre_hooks:
                return None
        return plan

    def _decode_in_one_call(self, hidden_states, attention_mask, past_key_value, use_cache):
        """``forward`` for one new token per sequence over a KV cache, or None when the tensors do not qualify."""
        hs = hidden_states
        dtype = hs.dtype
        if not (hs.is_cuda and hs.is_contiguous() and hs.shape[0] <= 16
                and (dtype is torch.float32 or dtype is torch.float16)):
            return None
        past_k, past_v = past_key_value
        bsz = hs.shape[0]
        if not (past_k.dim() == 4 and past_v.shape == past_k.shape and past_k.dtype is torch.int8
                and past_v.dtype is torch.int8 and past_k.device == hs.device and past_v.device == hs.device
                and past_k.shape[0] == bsz):
            return None
        plan = self._decode_plan(dtype is torch.float16, hs.device)
        if plan is None or past_k.shape[1] != plan.heads or past_k.shape[3] != plan.head_dim or hs.shape[2] != plan.embed:
            return None
        S = past_k.shape[2] + 1
        if not _hip_ext.decode_attention_shape_ok_cached(1, S, plan.head_dim):
            return None
        mask = attention_mask
        if mask is not None:
            mask = _mask_as_fp32(mask)
            if not (mask is not None and mask.is_contiguous() and mask.shape == (bsz, 1, 1, S) and mask.device == hs.device):
                return None
        kk = _kv_room_for(past_k, 1) or _kv_fresh(past_k, 1)
        vv = _kv_room_for(past_v, 1) or _kv_fresh(past_v, 1)
        if kk.buf.data_ptr() % 16 or vv.buf.data_ptr() % 16 or not (kk.buf.is_contiguous() and vv.buf.is_contiguous()
                                                                    and kk.buf.shape == vv.buf.shape):
            return None
        _hip_ext.opt_layer_decode(plan, hs, mask, kk.buf, vv.buf, S)
        kk.filled = vv.filled = S
        if use_cache:
            return hs, (_kv_view(kk, S), _kv_view(vv, S))
        return (hs,)

    #: a prefill of up to 4096 tokens in all (more than 16 per sequence, a multiple of 16): likewise one C call
    #: (``ti_opt_decoder_layer_prefill``); at those sizes a layer's kernels take less time than eight trips through Python
    prefill_in_one_call = True

    def _prefill_in_one_call(self, hidden_states, attention_mask, use_cache):
        """``forward`` without a cache on T > 16 tokens per sequence, or None when the tensors do not qualify."""
        hs = hidden_states
        dtype = hs.dtype
        bsz, T = hs.shape[0], hs.shape[1]
        if not (hs.is_cuda and hs.is_contiguous() and T % 16 == 0 and 0 < bsz * T <= 4096
                and (dtype is torch.float32 or dtype is torch.float16)):
            return None
        plan = self._decode_plan(dtype is torch.float16, hs.device)
        if plan is None or hs.shape[2] != plan.embed or not _hip_ext.attn_prefill_shape_ok_cached(T, T, plan.head_dim):
            return None
        mask = attention_mask
        if mask is not None:
            mask = _mask_as_fp32(mask)
            if not (mask is not None and mask.is_contiguous() and mask.shape == (bsz, 1, T, T) and mask.device == hs.device
                    and mask.data_ptr() % 16 == 0):
                return None
        key = torch.empty((bsz, plan.heads, T, plan.head_dim), dtype=torch.int8, device=hs.device)
        value = torch.empty((bsz, plan.heads, T, plan.head_dim), dtype=torch.int8, device=hs.device)
        _hip_ext.opt_layer_prefill(plan, hs, mask, key, value)
        if use_cache:
            return hs, (key, value)
        return (hs,)

    def decode_step_devlen(self, hidden_states, k_buf, v_buf, length, max_length):
        """``forward`` for one new token per sequence with the cache length read on the device (see
        ``Int8OPTAttention.decode_step_devlen``): updates ``hidden_states`` in place and appends to the cache."""
        residual = hidden_states
        x = self.self_attn_layer_norm(hidden_states)
        x = self.self_attn.decode_step_devlen(x, k_buf, v_buf, length, max_length)
        x = self.final_layer_norm(residual, add=x)
        x = self.fc1(x)
        if type(self.fc2) is W8A8BFP32OFP32Linear:
            self.fc2(x, add_to=residual)
        else:
            residual.add_(self.fc2(x).to(residual.dtype))
        return residual

    def forward(self, hidden_states: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
                layer_head_mask: Optional[torch.Tensor] = None, output_attentions: Optional[bool] = False,
                use_cache: Optional[bool] = False, past_key_value: Optional[Tuple[torch.Tensor]] = None):
        """hidden_states: fp [batch, time, embed_dim] residual stream -> tuple starting with it."""
        if (past_key_value is not None and self.decode_in_one_call and hidden_states.dim() == 3
                and hidden_states.shape[1] == 1 and layer_head_mask is None and not output_attentions
                and self.self_attn.kv_cache_in_place and self.self_attn.fused_softmax):
            out = self._decode_in_one_call(hidden_states, attention_mask, past_key_value, use_cache)
            if out is not None:
                return out
        elif (past_key_value is None and self.prefill_in_one_call and hidden_states.dim() == 3
                and 16 < hidden_states.shape[1] and layer_head_mask is None and not output_attentions
                and self.self_attn.fused_softmax):
            out = self._prefill_in_one_call(hidden_states, attention_mask, use_cache)
            if out is not None:
                return out
        residual = hidden_states
        x = self.self_attn_layer_norm(hidden_states)
        x, attn_weights, present = self.self_attn(
            hidden_states=x, past_key_value=past_key_value, attention_mask=attention_mask,
            layer_head_mask=layer_head_mask, output_attentions=output_attentions)
        x = self.final_layer_norm(residual, add=x)  # residual += x, then LayerNormQ
        x = self.fc1(x)
        if type(self.fc2) is W8A8BFP32OFP32Linear:
            self.fc2(x, add_to=residual)  # residual += fc2(x), added in the GEMM epilogue when residual is fp32
        else:
            residual.add_(self.fc2(x).to(residual.dtype))
        outputs = (residual,)
        if output_attentions:
            outputs += (attn_weights,)
        if use_cache:
            outputs += (present,)
        return outputs


# --------------------------------------------------------------------------------------
# OPT scaffolding around the int8 blocks
# --------------------------------------------------------------------------------------

@dataclass
class OPTConfigLite:
    """The OPTConfig fields the int8 model reads, with OPT-125m defaults."""
    vocab_size: int = 50272
    hidden_size: int = 768
    num_hidden_layers: int = 12
    ffn_dim: int = 3072
    num_attention_heads: int = 12
    max_position_embeddings: int = 2048
    word_embed_proj_dim: Optional[int] = None
    pad_token_id: int = 1
    do_layer_norm_before: bool = True
    _remove_final_layer_norm: bool = False
    use_cache: bool = True

    def __post_init__(self):
        if self.word_embed_proj_dim is None:
            self.word_embed_proj_dim = self.hidden_size


@dataclass
class BaseModelOutputWithPast:
    last_hidden_state: torch.Tensor = None
    past_key_values: Optional[tuple] = None
    hidden_states: Optional[tuple] = None
    attentions: Optional[tuple] = None


@dataclass
class CausalLMOutputWithPast:
    loss: Optional[torch.Tensor] = None
    logits: torch.Tensor = None
    past_key_values: Optional[tuple] = None
    hidden_states: Optional[tuple] = None
    attentions: Optional[tuple] = None


class OPTLearnedPositionalEmbedding(nn.Embedding):
    """Learned absolute positions; OPT reserves the first two rows, so indices are offset by 2."""
    offset = 2

    def __init__(self, num_embeddings: int, embedding_dim: int):
        super().__init__(num_embeddings + self.offset, embedding_dim)

    def forward(self, attention_mask: torch.Tensor, past_key_values_length: int = 0):
        mask = attention_mask.long()
        positions = torch.cumsum(mask, dim=1) * mask - 1  # padded slots get -1
        return super().forward(positions[:, past_key_values_length:] + self.offset)


def _additive_decoder_mask(attention_mask, tgt_len, past_len, dtype, device):
    """[bsz, 1, tgt, past+tgt] mask: 0 where attention is allowed, finfo.min where the
    key is in the future or is padding (both conditions add up)."""
    bsz, src_len = attention_mask.shape
    neg = torch.finfo(dtype).min
    keep = attention_mask[:, None, None, :].to(dtype)
    pad = (1.0 - keep).masked_fill((1.0 - keep).bool(), neg).expand(bsz, 1, tgt_len, src_len)
    if tgt_len <= 1:
        return pad.contiguous()
    q_pos = torch.arange(past_len, past_len + tgt_len, device=device)[:, None]
    k_pos = torch.arange(src_len, device=device)[None, :]
    causal = torch.zeros((tgt_len, src_len), dtype=dtype, device=device).masked_fill(k_pos > q_pos, neg)
    return pad + causal[None, None]


class Int8OPTDecoder(nn.Module):
    """Stack of ``Int8OPTDecoderLayer`` with fp embeddings and final LayerNorm
    (upstream ``torch_int/models/opt.py:302-398``).  Without a KV cache the token dimension
    is padded to a multiple of 16 with <pad> (id 1, masked out) and the result sliced back,
    exactly as upstream; with a cache the new tokens are used as they are."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.padding_idx = config.pad_token_id
        self.max_target_positions = config.max_position_embeddings
        self.vocab_size = config.vocab_size
        D, E = config.hidden_size, config.word_embed_proj_dim
        self.embed_tokens = nn.Embedding(config.vocab_size, E, self.padding_idx)
        self.embed_positions = OPTLearnedPositionalEmbedding(config.max_position_embeddings, D)
        self.project_out = nn.Linear(D, E, bias=False) if E != D else None
        self.project_in = nn.Linear(E, D, bias=False) if E != D else None
        if config.do_layer_norm_before and not getattr(config, "_remove_final_layer_norm", False):
            self.final_layer_norm = nn.LayerNorm(D)
        else:
            self.final_layer_norm = None
        self.layers = nn.ModuleList(
            [Int8OPTDecoderLayer(D, config.num_attention_heads, config.ffn_dim)
             for _ in range(config.num_hidden_layers)])

    def get_input_embeddings(self):
        return self.embed_tokens

    def set_input_embeddings(self, value):
        self.embed_tokens = value

    @staticmethod
    def from_float(module, decoder_layer_scales):
        q = Int8OPTDecoder(module.config)
        q.embed_tokens = module.embed_tokens
        q.embed_positions = module.embed_positions
        q.project_out = module.project_out
        q.project_in = getattr(module, "project_in", None)
        q.final_layer_norm = module.final_layer_norm
        for i, layer in enumerate(module.layers):
            q.layers[i] = Int8OPTDecoderLayer.from_float(layer, **decoder_layer_scales[i])
        return q

    @torch.no_grad()
    def forward(self, input_ids: torch.LongTensor = None, attention_mask: Optional[torch.Tensor] = None,
                head_mask: Optional[torch.Tensor] = None,
                past_key_values: Optional[List[Tuple[torch.Tensor]]] = None,
                inputs_embeds: Optional[torch.Tensor] = None, use_cache: Optional[bool] = None,
                output_attentions: Optional[bool] = None, output_hidden_states: Optional[bool] = None,
                return_dict: Optional[bool] = None):
        use_cache = bool(use_cache) if use_cache is not None else False
        if inputs_embeds is None:
            input_ids = input_ids.view(-1, input_ids.shape[-1])
        input_len = (input_ids if input_ids is not None else inputs_embeds).shape[1]
        past_len = past_key_values[0][0].shape[2] if past_key_values else 0

        pad_len = (-input_len) % 16 if (past_len == 0 and inputs_embeds is None) else 0
        if pad_len:
            input_ids = nn.functional.pad(input_ids, (0, pad_len), value=1)
            if attention_mask is not None:
                attention_mask = nn.functional.pad(attention_mask, (0, pad_len), value=0)
        if inputs_embeds is None:
            inputs_embeds = self.embed_tokens(input_ids)
        bsz, tgt_len = inputs_embeds.shape[:2]
        if attention_mask is None:
            attention_mask = torch.ones((bsz, past_len + tgt_len), dtype=torch.bool, device=inputs_embeds.device)
        pos = self.embed_positions(attention_mask, past_len)
        mask = _additive_decoder_mask(attention_mask, tgt_len, past_len, inputs_embeds.dtype,
                                      inputs_embeds.device)
        if mask.is_cuda and mask.dtype in (torch.float16, torch.bfloat16):
            mask = mask.float()  # once here instead of once per layer (see Int8OPTAttention.forward)
        if self.project_in is not None:
            inputs_embeds = self.project_in(inputs_embeds)
        hidden = inputs_embeds + pos  # a fresh tensor: the layers update it in place

        all_hidden = () if output_hidden_states else None
        all_attn = () if output_attentions else None
        cache = () if use_cache else None
        for i, layer in enumerate(self.layers):
            if output_hidden_states:
                all_hidden += (hidden.clone(),)
            out = layer(hidden, attention_mask=mask,
                        layer_head_mask=head_mask[i] if head_mask is not None else None,
                        output_attentions=bool(output_attentions), use_cache=use_cache,
                        past_key_value=past_key_values[i] if past_key_values else None)
            hidden = out[0]
            if output_attentions:
                all_attn += (out[1],)
            if use_cache:
                cache += (out[-1],)
        if self.final_layer_norm is not None:
            hidden = self.final_layer_norm(hidden)
        if self.project_out is not None:
            hidden = self.project_out(hidden)
        if output_hidden_states:
            all_hidden += (hidden,)
        if pad_len:
            hidden = hidden[:, :input_len, :]
        return BaseModelOutputWithPast(last_hidden_state=hidden, past_key_values=cache,
                                       hidden_states=all_hidden, attentions=all_attn)


class Int8OPTModel(nn.Module):
    """upstream ``torch_int/models/opt.py:401-417``."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.decoder = Int8OPTDecoder(config)

    def get_input_embeddings(self):
        return self.decoder.embed_tokens

    def set_input_embeddings(self, value):
        self.decoder.embed_tokens = value

    def get_decoder(self):
        return self.decoder

    @staticmethod
    def from_float(module, decoder_layer_scales):
        q = Int8OPTModel(module.config)
        q.decoder = Int8OPTDecoder.from_float(module.decoder, decoder_layer_scales)
        return q

    def forward(self, *args, **kwargs):
        return self.decoder(*args, **kwargs)


class Int8OPTForCausalLM(nn.Module):
    """Int8 decoder + fp ``lm_head`` (not quantised; upstream ``torch_int/models/opt.py:420-450``)."""
    _keys_to_ignore_on_load_missing = [r"lm_head.weight"]

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.model = Int8OPTModel(config)
        self.lm_head = nn.Linear(config.word_embed_proj_dim, config.vocab_size, bias=False)
        # Upstream's post_init ties the output projection to the token embedding (OPTConfig.tie_word_embeddings
        # defaults to True), and exported checkpoints then carry no ``lm_head.weight``.
        if getattr(config, "tie_word_embeddings", True):
            self.lm_head.weight = self.model.decoder.embed_tokens.weight
        self._register_load_state_dict_pre_hook(self._fill_tied_lm_head)

    def _fill_tied_lm_head(self, state_dict, prefix, *unused):
        """A state dict without ``lm_head.weight`` (tied weights are stored once) loads the embedding there."""
        head, emb = prefix + "lm_head.weight", prefix + "model.decoder.embed_tokens.weight"
        if head not in state_dict and emb in state_dict and self.lm_head.weight.shape == state_dict[emb].shape:
            state_dict[head] = state_dict[emb]

    @staticmethod
    def from_float(module, decoder_layer_scales):
        q = Int8OPTForCausalLM(module.config)
        q.model = Int8OPTModel.from_float(module.model, decoder_layer_scales)
        q.lm_head = module.lm_head
        return q

    def get_input_embeddings(self):
        return self.model.decoder.embed_tokens

    def set_input_embeddings(self, value):
        self.model.decoder.embed_tokens = value

    def get_output_embeddings(self):
        return self.lm_head

    def set_output_embeddings(self, new_embeddings):
        self.lm_head = new_embeddings

    def set_decoder(self, decoder):
        self.model.decoder = decoder

    def get_decoder(self):
        return self.model.decoder

    @torch.no_grad()
    def forward(self, input_ids: torch.LongTensor = None, attention_mask: Optional[torch.Tensor] = None,
                head_mask: Optional[torch.Tensor] = None, past_key_values=None,
                inputs_embeds: Optional[torch.Tensor] = None, labels: Optional[torch.LongTensor] = None,
                use_cache: Optional[bool] = None, output_attentions: Optional[bool] = None,
                output_hidden_states: Optional[bool] = None, return_dict: Optional[bool] = None):
        out = self.model.decoder(input_ids=input_ids, attention_mask=attention_mask, head_mask=head_mask,
                                 past_key_values=past_key_values, inputs_embeds=inputs_embeds,
                                 use_cache=use_cache, output_attentions=output_attentions,
                                 output_hidden_states=output_hidden_states)
        logits = self.lm_head(out.last_hidden_state.to(self.lm_head.weight.dtype)).contiguous()
        loss = None
        if labels is not None:
            shift = logits[..., :-1, :].contiguous()
            loss = nn.functional.cross_entropy(shift.view(-1, shift.size(-1)),
                                               labels[..., 1:].contiguous().view(-1).to(logits.device))
        return CausalLMOutputWithPast(loss=loss, logits=logits, past_key_values=out.past_key_values,
                                      hidden_states=out.hidden_states, attentions=out.attentions)

    def prepare_inputs_for_generation(self, input_ids, past_key_values=None, attention_mask=None, **kwargs):
        if past_key_values:
            input_ids = input_ids[:, -1:]
        return {"input_ids": input_ids, "attention_mask": attention_mask,
                "past_key_values": past_key_values, "use_cache": kwargs.get("use_cache")}

    @staticmethod
    def _reorder_cache(past, beam_idx):
        return tuple(tuple(s.index_select(0, beam_idx) for s in layer) for layer in past)


class Int8OPTGraphDecoder:
    """Token-by-token decoding of an ``Int8OPTForCausalLM`` on HIP with the decoder layers of a step replayed from
    one HIP graph (no counterpart upstream, whose ``generate`` re-issues every launch from Python).

    A decode step of a small or medium model is bound by the host: seven launches per layer and the Python around
    them.  Here the layers are recorded once, on fixed buffers: the residual stream of the new token, the key /
    value caches (buffers with room for ``max_new_tokens`` more positions) and an int32 tensor holding the cache
    length, which the attention kernel reads when it runs, so the same recording serves every step.  Embeddings,
    the final LayerNorm and ``lm_head`` stay ordinary torch calls around the replay.  No padding inside the batch
    (every sequence has the same length) and no head mask.  Values are those of ``lm(ids, past_key_values=...)``.

        out = lm(prompt_ids, use_cache=True)
        dec = Int8OPTGraphDecoder(lm, out.past_key_values, max_new_tokens=128)
        tok = out.logits[:, -1].argmax(-1, keepdim=True)
        for _ in range(128):
            tok = dec.step(tok)[:, -1].argmax(-1, keepdim=True)
    """

    @torch.no_grad()
    def __init__(self, lm, past_key_values, max_new_tokens):
        dec = lm.model.decoder
        k0 = past_key_values[0][0]
        if not (k0.is_cuda and k0.dtype is torch.int8 and k0.dim() == 4 and len(past_key_values) == len(dec.layers)):
            raise RuntimeError("Int8OPTGraphDecoder: needs the int8 HIP key/value caches of every decoder layer")
        bsz, H, S0, d = k0.shape
        self.lm, self.filled, self.max_length = lm, S0, S0 + int(max_new_tokens)
        if max_new_tokens < 1 or self.max_length > dec.max_target_positions:
            raise RuntimeError(f"Int8OPTGraphDecoder: {S0} cached + {max_new_tokens} new positions exceed the model's "
                               f"{dec.max_target_positions}")
        if not _hip_ext.decode_attention_shape_ok(1, self.max_length, d):
            raise RuntimeError(f"Int8OPTGraphDecoder: the decode attention kernel does not take {self.max_length} "
                               f"positions of head size {d}")
        cap = -(-self.max_length // 16) * 16
        self.caches = []
        for k, v in past_key_values:
            kb = torch.empty((bsz, H, cap, d), dtype=torch.int8, device=k0.device)
            vb = torch.empty_like(kb)
            kb[:, :, :S0].copy_(k)
            vb[:, :, :S0].copy_(v)
            self.caches.append((kb, vb))
        stream_dtype = dec.embed_positions.weight.dtype
        self.hidden = torch.zeros((bsz, 1, dec.embed_positions.weight.shape[1]), dtype=stream_dtype, device=k0.device)
        self.length = torch.full((1,), S0 + 1, dtype=torch.int32, device=k0.device)
        self._ones = torch.ones((bsz, self.max_length), dtype=torch.bool, device=k0.device)

        def layers():
            for layer, (kb, vb) in zip(dec.layers, self.caches):
                layer.decode_step_devlen(self.hidden, kb, vb, self.length, self.max_length)
        # one eager pass first: scalar caches, kernel attributes and the allocator's pools are then warm, and nothing
        # in the recording synchronises.  It writes position S0 of the caches, which the first real step overwrites.
        side = torch.cuda.Stream(device=k0.device)
        side.wait_stream(torch.cuda.current_stream(k0.device))
        with torch.cuda.stream(side):
            layers()
        torch.cuda.current_stream(k0.device).wait_stream(side)
        # recorded on the stream of the eager pass: the library's per-stream state (split-K workspace and arrival
        # counters, placement probe) is then ready, and nothing in the recording has to fall back or synchronise
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            layers()

    @torch.no_grad()
    def step(self, input_ids):
        """Logits [bsz, 1, vocab] for one new token per sequence (``input_ids`` [bsz, 1]); the caches grow by one."""
        if self.filled >= self.max_length:
            raise RuntimeError("Int8OPTGraphDecoder: max_new_tokens steps have been taken")
        dec = self.lm.model.decoder
        embeds = dec.embed_tokens(input_ids)
        pos = dec.embed_positions(self._ones[:, :self.filled + 1], self.filled)
        if dec.project_in is not None:
            embeds = dec.project_in(embeds)
        self.hidden.copy_(embeds + pos)
        self.length.fill_(self.filled + 1)
        self.graph.replay()
        self.filled += 1
        hidden = self.hidden
        if dec.final_layer_norm is not None:
            hidden = dec.final_layer_norm(hidden)
        if dec.project_out is not None:
            hidden = dec.project_out(hidden)
        return self.lm.lm_head(hidden.to(self.lm.lm_head.weight.dtype)).contiguous()

    @property
    def past_key_values(self):
        """The caches as ``forward`` would return them: per layer (key, value) int8 [bsz, heads, filled, head_dim]."""
        return tuple((kb[:, :, :self.filled], vb[:, :, :self.filled]) for kb, vb in self.caches)


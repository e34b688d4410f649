#!/usr/bin/env python3
"""One Int8OPTDecoderLayer, or its Int8OPTAttention alone, at a given size on one GPU.

Mirrors upstream benchmark/bench_opt_decoder_layer.py and benchmark/bench_opt_attention.py (defaults: a
GPT-3-175B-sized layer, hidden 12288, FFN 49152, 96 heads, batch 8 x 512 tokens; benchmark/utils.py:32-55 times 100
forwards after 10 warm-ups): random int8 weights, per-tensor scales ~U(1e-4, 1e-2), an fp32 (or fp16) residual stream
and a causal mask; back-to-back forwards between two HIP events for at least --window-ms.

  python torch-int_amd/benchmark/bench_decoder_layer.py
  python torch-int_amd/benchmark/bench_decoder_layer.py --hidden-size 5120 --ffn-dim 20480 --num-attention-heads 40 --batch-size 4
  python torch-int_amd/benchmark/bench_decoder_layer.py --module attention
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import torch  # noqa: E402
from torch_int.models.opt import Int8OPTDecoderLayer  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch-size", type=int, default=8)
    ap.add_argument("--seq-len", type=int, default=512)
    ap.add_argument("--hidden-size", type=int, default=12288)
    ap.add_argument("--ffn-dim", type=int, default=12288 * 4)
    ap.add_argument("--num-attention-heads", type=int, default=96)
    ap.add_argument("--module", choices=["layer", "attention"], default="layer")
    ap.add_argument("--dtype", choices=["fp32", "fp16"], default="fp32", help="residual stream and LayerNorm parameters")
    ap.add_argument("--window-ms", type=float, default=200.0)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    B, T, D, F, H = args.batch_size, args.seq_len, args.hidden_size, args.ffn_dim, args.num_attention_heads
    g = torch.Generator(device=dev).manual_seed(0)

    def u():
        return float(torch.empty(1, device=dev).uniform_(1e-4, 1e-2, generator=g))
    with torch.device(dev):
        layer = Int8OPTDecoderLayer(D, H, F)
        a = layer.self_attn
        for lin in (a.q_proj, a.k_proj, a.v_proj, layer.fc1):
            lin.weight.random_(-127, 128, generator=g)
            lin.bias = torch.randint(-127, 128, (1, lin.out_features), dtype=torch.int8, device=dev, generator=g)
            lin.a.fill_(u())
            lin.b.fill_(u())
        for lin in (a.out_proj, layer.fc2):
            lin.weight.random_(-127, 128, generator=g)
            lin.bias = torch.randn(1, lin.out_features, device=dev, generator=g)
            lin.a.fill_(u())
        a.qk_bmm.a.fill_(u())
        a.pv_bmm.a.fill_(u())
    if args.dtype == "fp16":
        layer = layer.half()
    layer.eval()
    mask = torch.zeros(T, T, device=dev).masked_fill(
        torch.triu(torch.ones(T, T, dtype=torch.bool, device=dev), 1), torch.finfo(torch.float32).min)
    mask = mask[None, None].expand(B, 1, T, T).contiguous()
    if args.dtype == "fp16":
        mask = mask.half()
    if args.module == "layer":
        # the layer updates its input in place, as upstream's does; LayerNorm keeps the growing residual in range
        x = torch.randn(B, T, D, device=dev, dtype=torch.float16 if args.dtype == "fp16" else torch.float32)
        fn = lambda: layer(x, attention_mask=mask)  # noqa: E731
        ops = 2.0 * B * T * (4 * D * D + 2 * D * F)
    else:
        x = torch.randint(-127, 128, (B, T, D), dtype=torch.int8, device=dev, generator=g)
        fn = lambda: a(x, attention_mask=mask)  # noqa: E731
        ops = 2.0 * B * T * 4 * D * D
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.no_grad():
        for _ in range(10):
            fn()
        start.record()
        fn()
        end.record()
        torch.cuda.synchronize()
        n = max(5, int(args.window_ms / max(start.elapsed_time(end), 1e-3)))
        start.record()
        for _ in range(n):
            fn()
        end.record()
        torch.cuda.synchronize()
    ms = start.elapsed_time(end) / n
    print(json.dumps({"module": args.module, "batch_size": B, "seq_len": T, "hidden_size": D, "ffn_dim": F, "heads": H,
                      "dtype": args.dtype, "ms": round(ms, 4), "linear_TOPS": round(ops / ms / 1e9, 1), "forwards": n,
                      "memory_MB": round(torch.cuda.max_memory_allocated() / 2 ** 20, 1)}), flush=True)


if __name__ == "__main__":
    main()

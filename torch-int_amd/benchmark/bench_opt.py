#!/usr/bin/env python3
"""Random-weight Int8OPTForCausalLM on one GPU: prefill latency and per-token decode latency.

Mirrors upstream benchmark/bench_opt.py / profiling/profile_opt.py (which also build random-init
models), without checkpoints: weights are generated on the device, so the 65 GB of int8 weights of
OPT-66B never pass through host memory.

  python torch-int_amd/benchmark/bench_opt.py --model opt-66b --batch 4 --seq 512 --decode-steps 32
  python torch-int_amd/benchmark/bench_opt.py --model opt-13b --layers 4 --batch 1 --seq 128
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import torch  # noqa: E402
from torch_int.models.opt import Int8OPTForCausalLM, OPTConfigLite  # noqa: E402

# hidden, heads, ffn, layers (facebook/opt-* configurations; vocab 50272, 2048 positions)
MODELS = {
    "opt-125m": (768, 12, 3072, 12), "opt-1.3b": (2048, 32, 8192, 24), "opt-2.7b": (2560, 32, 10240, 32),
    "opt-6.7b": (4096, 32, 16384, 32),
    "opt-13b": (5120, 40, 20480, 40), "opt-30b": (7168, 56, 28672, 48), "opt-66b": (9216, 72, 36864, 64),
}


def build(name, layers, dev, seed=0):
    D, H, F, L = MODELS[name]
    cfg = OPTConfigLite(hidden_size=D, num_attention_heads=H, ffn_dim=F, num_hidden_layers=layers or L)
    torch.manual_seed(seed)
    with torch.device(dev):
        model = Int8OPTForCausalLM(cfg)
        g = torch.Generator(device=dev).manual_seed(seed)

        def u():
            return float(torch.empty(1, device=dev).uniform_(1e-4, 1e-2, generator=g))
        for layer in model.model.decoder.layers:
            a = layer.self_attn
            for lin in (a.q_proj, a.k_proj, a.v_proj, layer.fc1):
                lin.bias = torch.randint(-127, 128, (1, lin.out_features), dtype=torch.int8, device=dev, generator=g)
                lin.a.fill_(u())
                lin.b.fill_(u())
            for lin in (a.out_proj, layer.fc2):
                lin.bias = torch.randn(1, lin.out_features, device=dev, generator=g)
                lin.a.fill_(u())
            a.qk_bmm.a.fill_(u())
            a.pv_bmm.a.fill_(u())
    return model.eval(), cfg


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="opt-13b", choices=list(MODELS))
    ap.add_argument("--layers", type=int, default=0, help="override the number of decoder layers")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--seq", type=int, default=512)
    ap.add_argument("--decode-steps", type=int, default=32)
    ap.add_argument("--iters", type=int, default=3)
    ap.add_argument("--dtype", default="fp32", choices=["fp32", "fp16"],
                    help="dtype of the embeddings, the residual stream, the LayerNorm parameters and lm_head "
                         "(upstream serves its SmoothQuant checkpoints in fp16)")
    ap.add_argument("--graph-decode", action="store_true",
                    help="also time the decode steps with the decoder layers replayed from a HIP graph "
                         "(Int8OPTGraphDecoder)")
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    t0 = time.perf_counter()
    model, cfg = build(args.model, args.layers, dev)
    if args.dtype == "fp16":
        model = model.half()
    torch.cuda.synchronize()
    int8_bytes = sum(b.numel() for n, b in model.named_buffers() if b.dtype == torch.int8)
    build_s = time.perf_counter() - t0
    g = torch.Generator(device=dev).manual_seed(1)
    ids = torch.randint(2, cfg.vocab_size, (args.batch, args.seq), device=dev, generator=g)

    def prefill():
        return model(ids, use_cache=True)

    with torch.no_grad():
        out = prefill()  # warm-up
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(args.iters):
            out = prefill()
        torch.cuda.synchronize()
        prefill_ms = (time.perf_counter() - t) * 1e3 / args.iters
        # the decoder stack alone (upstream's benchmark/bench_opt.py times Int8OPTModel, which has no lm_head;
        # the fp32 logits of every prompt position are a torch GEMM outside this library)
        model.model(ids, use_cache=True)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(args.iters):
            model.model(ids, use_cache=True)
        torch.cuda.synchronize()
        prefill_decoder_ms = (time.perf_counter() - t) * 1e3 / args.iters
        past = out.past_key_values
        tok = out.logits[:, -1].argmax(-1, keepdim=True)
        step_ms = []
        for _ in range(args.decode_steps):
            torch.cuda.synchronize()
            t = time.perf_counter()
            o = model(tok, past_key_values=past, use_cache=True)
            torch.cuda.synchronize()
            step_ms.append((time.perf_counter() - t) * 1e3)
            past = o.past_key_values
            tok = o.logits[:, -1].argmax(-1, keepdim=True)
        graph_ms = None
        if args.graph_decode:
            from torch_int.models.opt import Int8OPTGraphDecoder
            dec = Int8OPTGraphDecoder(model, out.past_key_values, max_new_tokens=args.decode_steps)
            tok = out.logits[:, -1].argmax(-1, keepdim=True)
            times = []
            for _ in range(args.decode_steps):
                torch.cuda.synchronize()
                t = time.perf_counter()
                logits = dec.step(tok)
                torch.cuda.synchronize()
                times.append((time.perf_counter() - t) * 1e3)
                tok = logits[:, -1].argmax(-1, keepdim=True)
            graph_ms = sorted(times)[len(times) // 2]
    finite = bool(torch.isfinite(o.logits).all())
    steady = sorted(step_ms)[len(step_ms) // 2] if step_ms else None
    tokens = args.batch * args.seq
    D, H, F, L = MODELS[args.model]
    L = args.layers or L
    gemm_ops = 2.0 * tokens * L * (4 * D * D + 2 * D * F)
    print(json.dumps({
        "model": args.model, "dtype": args.dtype, "layers": L, "batch": args.batch, "seq": args.seq, "int8_weight_GB": int8_bytes / 1e9,
        "build_s": build_s, "prefill_ms": prefill_ms, "prefill_decoder_ms": prefill_decoder_ms,
        "prefill_linear_TOPS": gemm_ops / prefill_decoder_ms / 1e9,
        "decode_steps": args.decode_steps, "decode_ms_per_token_median": steady,
        "decode_weight_GBps": (int8_bytes / 1e9) / (steady / 1e3) if steady else None,
        "graph_decode_ms_per_token_median": graph_ms,
        "final_src_len": int(past[0][0].shape[2]), "logits_finite": finite,
        "peak_mem_GB": torch.cuda.max_memory_allocated() / 1e9}), flush=True)


if __name__ == "__main__":
    main()

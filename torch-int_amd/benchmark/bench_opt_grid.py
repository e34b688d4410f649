#!/usr/bin/env python3
"""The reference's model-latency grid on one MI355X, in one process.

Upstream scripts/bench_opt.sh:1-4 + benchmark/bench_opt.py: Int8OPTModel (decoder stack, no lm_head) in its
"int8-fp16" precision (fp16 embeddings, residual stream and LayerNorm parameters), one forward over
[batch, seq_len] token ids, models opt-125m ... opt-13b (opt-30b commented out there), batch in {1, 2, 4, 8, 16, 32},
seq_len in {128, 256, 512, 1024}; it prints the average latency (benchmark/utils.py:32-55: 10 warm-up forwards, then
100) and torch.cuda.max_memory_allocated.  Here the weights are random and generated on the device (no checkpoints),
each model is built once, and a row runs 3 warm-up forwards and then enough of them to fill a window.

  python torch-int_amd/benchmark/bench_opt_grid.py                       # upstream's five models, one JSON line per row
  python torch-int_amd/benchmark/bench_opt_grid.py --models opt-30b opt-66b --batches 1 4 --seqs 512
"""
import argparse
import gc
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import torch  # noqa: E402
from bench_opt import MODELS, build  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--models", nargs="+", default=["opt-125m", "opt-1.3b", "opt-2.7b", "opt-6.7b", "opt-13b"],
                    choices=list(MODELS))
    ap.add_argument("--batches", type=int, nargs="+", default=[1, 2, 4, 8, 16, 32])
    ap.add_argument("--seqs", type=int, nargs="+", default=[128, 256, 512, 1024])
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "fp32"])
    ap.add_argument("--window-ms", type=float, default=150.0)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    for name in args.models:
        model, cfg = build(name, 0, dev)
        if args.dtype == "fp16":
            model = model.half()
        stack = model.model
        D, H, F, L = MODELS[name]
        weights_gb = sum(b.numel() for _, b in model.named_buffers() if b.dtype == torch.int8) / 1e9
        g = torch.Generator(device=dev).manual_seed(1)
        for seq in args.seqs:
            for batch in args.batches:
                ids = torch.randint(2, cfg.vocab_size, (batch, seq), device=dev, generator=g)
                torch.cuda.empty_cache()
                torch.cuda.reset_peak_memory_stats()
                with torch.no_grad():
                    for _ in range(3):
                        stack(ids)
                    torch.cuda.synchronize()
                    t = time.perf_counter()
                    stack(ids)
                    torch.cuda.synchronize()
                    n = max(3, int(args.window_ms / max((time.perf_counter() - t) * 1e3, 1e-3)))
                    t = time.perf_counter()
                    for _ in range(n):
                        stack(ids)
                    torch.cuda.synchronize()
                    ms = (time.perf_counter() - t) * 1e3 / n
                tokens = batch * seq
                ops = 2.0 * tokens * L * (4 * D * D + 2 * D * F)
                print(json.dumps({"model": name, "precision": "int8-" + args.dtype, "batch_size": batch, "seq_len": seq,
                                  "latency_ms": round(ms, 3), "memory_MB": round(torch.cuda.max_memory_allocated() / 2 ** 20, 1),
                                  "linear_TOPS": round(ops / ms / 1e9, 1), "tokens_per_s": round(tokens / ms * 1e3),
                                  "int8_weight_GB": round(weights_gb, 2)}), flush=True)
        del model, stack
        gc.collect()  # the modules hold reference cycles: without this the next model's peak includes this one's weights
        torch.cuda.empty_cache()


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""The reference's own kernel-latency grids on one MI355X, in one process.

Linears (upstream scripts/bench_linear_kernels.sh:23-26 + benchmark/bench_linear_kernels.py): GPT-3-175B widths,
seq_len in {128, 256, 512, 1024} rows:
    fc1  linear_relu_a8_w8_b8_o8   [seq, 12288] x [49152, 12288]^T
    fc2  linear_a8_w8_b32_o32      [seq, 49152] x [12288, 49152]^T
    qkv  linear_a8_w8_b8_o8        [seq, 12288] x [12288, 12288]^T
    out  linear_a8_w8_b32_o32      [seq, 12288] x [12288, 12288]^T
Batched products (upstream scripts/bench_bmm.sh:1-4 + benchmark/bench_bmm.py:9-15): bmm_s8t_s8n_s8t of
[batch, seq, 12288] x [batch, seq, 12288]^T, batch in {1, 4, 8, 16}, seq in {256, 512, 1024}.

Protocol of upstream benchmark/utils.py:81-96: 100 warm-up calls, then back-to-back calls between two events on the
launch stream (here enough of them to fill a window, instead of a fixed 2000 / 5000).  Upstream repeats one weight
tensor, so a 151 MB weight is served by the 256 MB last-level cache after the first call; `--cold` rotates weight
copies so that every call streams them from HBM, which is how a model's layers find theirs.  Each row carries the
fraction of its binding roofline (5.0 POP/s dense INT8 or 8 TB/s HBM, by arithmetic intensity) and the kernel family.

  python torch-int_amd/benchmark/bench_grid.py            # both grids, one JSON line per row
  python torch-int_amd/benchmark/bench_grid.py --cold --grid linear
"""
import argparse
import ctypes
import json
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import torch  # noqa: E402
import torch_int._CUDA as C  # noqa: E402

PEAK_TOPS, PEAK_GBS = 5000.0, 8000.0
LINEAR_SETTINGS = [("fc1", 12288, 49152, "linear_relu_a8_w8_b8_o8"), ("fc2", 49152, 12288, "linear_a8_w8_b32_o32"),
                   ("qkv", 12288, 12288, "linear_a8_w8_b8_o8"), ("out", 12288, 12288, "linear_a8_w8_b32_o32")]
SEQ_LENS = [128, 256, 512, 1024]
BMM_BATCHES, BMM_SEQS, BMM_HIDDEN = [1, 4, 8, 16], [256, 512, 1024], 12288


def timed_ms(fns, window_ms, warm=100):
    n = len(fns)
    for i in range(warm):
        fns[i % n]()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(8):
        fns[i % n]()
    end.record()
    torch.cuda.synchronize()
    iters = max(16, int(window_ms / max(start.elapsed_time(end) / 8, 1e-3)) + 1)
    start.record()
    for i in range(iters):
        fns[i % n]()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def roofline(ops, nbytes, ms):
    tops, gbs = ops / ms / 1e9, nbytes / ms / 1e6
    bound = "mfma" if ops / nbytes >= PEAK_TOPS * 1e3 / PEAK_GBS else "hbm"
    return {"us": round(ms * 1e3, 2), "TOPS": round(tops, 1), "GBps": round(gbs, 1), "bound": bound,
            "frac": round(tops / PEAK_TOPS if bound == "mfma" else gbs / PEAK_GBS, 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--grid", choices=["linear", "bmm", "both"], default="both")
    ap.add_argument("--cold", action="store_true", help="rotate weight copies (> 256 MB in total) between calls")
    ap.add_argument("--window-ms", type=float, default=60.0)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    lib = C._lib
    lib.ti_last_kernel.restype = ctypes.c_char_p
    g = torch.Generator(device=dev).manual_seed(0)

    def s8(*shape):
        return torch.randint(-127, 127, shape, dtype=torch.int8, device=dev, generator=g)

    if args.grid in ("linear", "both"):
        for name, c1, c2, fn_name in LINEAR_SETTINGS:
            copies = max(1, -(-320 * 2 ** 20 // (c1 * c2))) if args.cold else 1
            ws = [s8(c2, c1) for _ in range(copies)]
            if fn_name == "linear_a8_w8_b32_o32":
                bias = torch.randint(-65535, 65535, (c2,), dtype=torch.int32, device=dev, generator=g)
                ob = 4
            else:
                bias = s8(c2)
                ob = 1
            for seq in SEQ_LENS:
                x = s8(seq, c1)
                if fn_name == "linear_a8_w8_b32_o32":
                    fns = [lambda w=w: C.linear_a8_w8_b32_o32(x, w, bias) for w in ws]
                elif fn_name == "linear_a8_w8_b8_o8":
                    fns = [lambda w=w: C.linear_a8_w8_b8_o8(x, w, bias, 0.001, 0.01) for w in ws]
                else:
                    fns = [lambda w=w: C.linear_relu_a8_w8_b8_o8(x, w, bias, 0.001, 0.01) for w in ws]
                fns[0]()
                family = lib.ti_last_kernel().decode()
                ms = timed_ms(fns, args.window_ms)
                row = {"grid": "linear", "name": name, "fn": fn_name, "seq_len": seq, "C1": c1, "C2": c2,
                       "weights": "cold" if args.cold else "repeated", "kernel": family}
                row.update(roofline(2.0 * seq * c1 * c2, seq * c1 + c1 * c2 + c2 * ob + seq * c2 * ob, ms))
                print(json.dumps(row), flush=True)
            del ws
            torch.cuda.empty_cache()
    if args.grid in ("bmm", "both"):
        H = BMM_HIDDEN
        for seq in BMM_SEQS:
            for batch in BMM_BATCHES:
                a = torch.randint(-128, 127, (batch, seq, H), dtype=torch.int8, device=dev, generator=g)
                b = torch.randint(-128, 127, (batch, seq, H), dtype=torch.int8, device=dev, generator=g)
                C.bmm_s8t_s8n_s8t(a, b, 0.01)
                family = lib.ti_last_kernel().decode()
                ms = timed_ms([lambda: C.bmm_s8t_s8n_s8t(a, b, 0.01)], args.window_ms)
                row = {"grid": "bmm", "fn": "bmm_s8t_s8n_s8t", "batch": batch, "seq_len": seq, "hidden": H, "kernel": family}
                row.update(roofline(2.0 * batch * seq * seq * H, batch * (2 * seq * H + seq * seq), ms))
                print(json.dumps(row), flush=True)


if __name__ == "__main__":
    main()

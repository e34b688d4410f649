#!/usr/bin/env python3
"""Run one INT8 kernel repeatedly on synthetic data: the unit that profilers wrap.

Examples
  python torch-int_amd/benchmark/bench_kernel.py --op linear_b8_o8 --shape 8192 20480 5120
  python torch-int_amd/benchmark/bench_kernel.py --op bmm_f32t --shape 160 512 512 128
  python torch-int_amd/benchmark/bench_kernel.py --op ln_q --shape 2048 5120
  python torch-int_amd/benchmark/bench_kernel.py --op copy --shape 268435456      # bytes; counter calibration
  rocprofv3 --kernel-trace --stats --output-format csv -d out -- python3 .../bench_kernel.py --op ...

Prints one JSON line: mean microseconds per call (HIP events on the launch stream), algorithmic
TOPS and GB/s.  Mirrors upstream benchmark/bench_linear_kernels.py, bench_bmm.py and
bench_dq_add_ln_q.py (warm-up, then N timed calls between two events).
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

import torch  # noqa: E402
import torch_int._CUDA as C  # noqa: E402

LINEAR = {
    "linear_b32_o32": (torch.int32, 4, 4),
    "linear_b32_o32_scaled": (torch.int32, 4, 4),
    "linear_bfp32_ofp32": (torch.float32, 4, 4),
    "linear_b8_o8": (torch.int8, 1, 1),
    "linear_relu_b8_o8": (torch.int8, 1, 1),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--op", required=True, choices=list(LINEAR) + ["bmm_f32t", "bmm_s8t", "bmm_s32t", "ln_q", "copy"])
    ap.add_argument("--shape", type=int, nargs="+", required=True)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--alpha", type=float, default=0.001)
    ap.add_argument("--beta", type=float, default=0.01)
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(0)

    def s8(*shape, lo=-127):
        return torch.randint(lo, 128, shape, dtype=torch.int8, device=dev, generator=g)

    ops = nbytes = 0.0
    if args.op in LINEAR:
        M, N, K = args.shape
        bdt, bb, ob = LINEAR[args.op]
        x, w = s8(M, K), s8(N, K)
        bias = torch.randn(N, device=dev, generator=g) if bdt == torch.float32 else \
            torch.randint(-127, 128, (N,), device=dev, generator=g).to(bdt)
        fn = {"linear_b32_o32": lambda: C.linear_a8_w8_b32_o32(x, w, bias),
              "linear_b32_o32_scaled": lambda: C.linear_a8_w8_b32_o32_with_scaling(x, w, bias, args.alpha, args.beta),
              "linear_bfp32_ofp32": lambda: C.linear_a8_w8_bfp32_ofp32(x, w, bias, args.alpha, 1.0),
              "linear_b8_o8": lambda: C.linear_a8_w8_b8_o8(x, w, bias, args.alpha, args.beta),
              "linear_relu_b8_o8": lambda: C.linear_relu_a8_w8_b8_o8(x, w, bias, args.alpha, args.beta)}[args.op]
        ops, nbytes = 2.0 * M * N * K, M * K + N * K + N * bb + M * N * ob
    elif args.op.startswith("bmm"):
        B, M, N, K = args.shape
        a, b = s8(B, M, K, lo=0 if args.op == "bmm_s8t" else -127), s8(B, N, K)
        fn = {"bmm_f32t": lambda: C.bmm_s8t_s8n_f32t(a, b, args.alpha),
              "bmm_s8t": lambda: C.bmm_s8t_s8n_s8t(a, b, args.alpha),
              "bmm_s32t": lambda: C.bmm_s8t_s8n_s32t(a, b)}[args.op]
        ops, nbytes = 2.0 * B * M * N * K, B * (M * K + N * K + M * N * (1 if args.op == "bmm_s8t" else 4))
    elif args.op == "ln_q":
        rows, H = args.shape
        inp = torch.randint(-65536, 65536, (rows, H), dtype=torch.int32, device=dev, generator=g)
        res = torch.randn(rows, H, device=dev, generator=g)
        gamma, beta = torch.ones(H, device=dev), torch.zeros(H, device=dev)
        fn = lambda: C.dq_add_layernorm_q(inp, 0.01, res, gamma, beta, 1e-5)  # noqa: E731
        nbytes = 13.0 * rows * H + 8 * H
    else:  # plain device copy of a known size: reference reading for FETCH_SIZE / WRITE_SIZE
        n, = args.shape
        src = torch.empty(n, dtype=torch.uint8, device=dev).random_(generator=g)
        dst = torch.empty_like(src)
        fn = lambda: dst.copy_(src)  # noqa: E731
        nbytes = 2.0 * n

    for _ in range(args.warmup):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(args.iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    ms = start.elapsed_time(end) / args.iters
    print(json.dumps({"op": args.op, "shape": args.shape, "us": ms * 1e3, "TOPS": ops / ms / 1e9,
                      "GBps": nbytes / ms / 1e6, "iters": args.iters}), flush=True)


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Run one INT8 kernel repeatedly on synthetic data: the unit that profilers wrap.

Examples
  python torch-int_amd/benchmark/bench_kernel.py --op linear_b8_o8 --shape 8192 20480 5120
  python torch-int_amd/benchmark/bench_kernel.py --op bmm_f32t --shape 160 512 512 128
  python torch-int_amd/benchmark/bench_kernel.py --op ln_q --shape 2048 5120
  python torch-int_amd/benchmark/bench_kernel.py --op softmax_q --shape 4 40 512 512        # batch heads T S
  python torch-int_amd/benchmark/bench_kernel.py --op bmm_s8t_rowmajor --shape 288 1 128 544
  python torch-int_amd/benchmark/bench_kernel.py --op linear_b8_o8 --shape 1 20480 5120 --rotate 4   # cache-cold weights
  python torch-int_amd/benchmark/bench_kernel.py --op copy --shape 268435456      # bytes; counter calibration
  python torch-int_amd/benchmark/bench_kernel.py --op mfma_loop --shape 2 20000 --pattern random --iters 200
      # matrix-pipe ceiling: mode (0 MFMA only, 1 + LDS reads, 2 + LDS-DMA copies and barrier), steps per wave
  python torch-int_amd/benchmark/bench_kernel.py --op mfma_ceiling --shape 250    # all six figures, 250 ms windows
  python torch-int_amd/benchmark/bench_kernel.py --op copy_loop --shape 0 4000     # L2 -> CU copy rate: mode (0 into LDS, 1 into registers), steps
  python torch-int_amd/benchmark/bench_kernel.py --op mix_loop --shape 0 15 20000   # floor of a K step: tile (0 256x160, 1 128x80), parts
      # (bit set: 1 MFMAs, 2 fragment reads, 4 copies, 8 barrier), steps; us / steps = time per K step
  python torch-int_amd/benchmark/bench_kernel.py --op read_loop --shape 2 20480 5120 --rotate 13   # read rate of a weight matrix:
      # mode (0 flat, 1 flat non-temporal, 2 the streaming GEMM's copies alone, 3 those with the default cache policy), N, K
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
import torch_int._hip_ext as X  # noqa: E402

LINEAR = {
    "linear_b32_o32": (torch.int32, 4, 4),
    "linear_b32_o32_scaled": (torch.int32, 4, 4),
    "linear_bfp32_ofp32": (torch.float32, 4, 4),
    "linear_b8_o8": (torch.int8, 1, 1),
    "linear_relu_b8_o8": (torch.int8, 1, 1),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--op", required=True, choices=list(LINEAR) + ["bmm_f32t", "bmm_s8t", "bmm_s32t", "bmm_s8t_rowmajor", "ln_q", "ln_q_f16", "add_ln_q",
                                               "softmax_q", "qk_softmax_q", "attn_prefill", "decode_attn", "transpose_last2", "copy",
                                               "mfma_loop", "mfma_ceiling", "store_loop", "copy_loop", "mix_loop", "read_loop"])
    ap.add_argument("--shape", type=int, nargs="+", required=True)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--alpha", type=float, default=0.001)
    ap.add_argument("--beta", type=float, default=0.01)
    ap.add_argument("--rotate", type=int, default=1,
                    help="copies of the large read-only operand used round-robin (defeats the 256 MB last-level cache)")
    ap.add_argument("--pattern", choices=["constant", "random"], default="random",
                    help="operand bytes of --op mfma_loop")
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    if args.op == "mfma_ceiling":
        print(json.dumps({"op": args.op, "window_ms": args.shape[0], "TOPS": X.measure_mfma_ceiling(float(args.shape[0]))}),
              flush=True)
        return
    g = torch.Generator(device=dev).manual_seed(0)

    def s8(*shape, lo=-127):
        return torch.randint(lo, 128, shape, dtype=torch.int8, device=dev, generator=g)

    ops = nbytes = 0.0
    if args.op in LINEAR:
        M, N, K = args.shape
        bdt, bb, ob = LINEAR[args.op]
        x, ws = s8(M, K), [s8(N, K) for _ in range(args.rotate)]
        w = ws[0]
        bias = torch.randn(N, device=dev, generator=g) if bdt == torch.float32 else \
            torch.randint(-127, 128, (N,), device=dev, generator=g).to(bdt)
        fn = {"linear_b32_o32": lambda: C.linear_a8_w8_b32_o32(x, w, bias),
              "linear_b32_o32_scaled": lambda: C.linear_a8_w8_b32_o32_with_scaling(x, w, bias, args.alpha, args.beta),
              "linear_bfp32_ofp32": lambda: C.linear_a8_w8_bfp32_ofp32(x, w, bias, args.alpha, 1.0),
              "linear_b8_o8": lambda: C.linear_a8_w8_b8_o8(x, w, bias, args.alpha, args.beta),
              "linear_relu_b8_o8": lambda: C.linear_relu_a8_w8_b8_o8(x, w, bias, args.alpha, args.beta)}[args.op]
        ops, nbytes = 2.0 * M * N * K, M * K + N * K + N * bb + M * N * ob
        if args.rotate > 1:
            variants, kind = [], args.op
            for w in ws:
                variants.append({"linear_b32_o32": lambda w=w: C.linear_a8_w8_b32_o32(x, w, bias),
                                 "linear_b32_o32_scaled": lambda w=w: C.linear_a8_w8_b32_o32_with_scaling(x, w, bias, args.alpha, args.beta),
                                 "linear_bfp32_ofp32": lambda w=w: C.linear_a8_w8_bfp32_ofp32(x, w, bias, args.alpha, 1.0),
                                 "linear_b8_o8": lambda w=w: C.linear_a8_w8_b8_o8(x, w, bias, args.alpha, args.beta),
                                 "linear_relu_b8_o8": lambda w=w: C.linear_relu_a8_w8_b8_o8(x, w, bias, args.alpha, args.beta)}[kind])
            state = {"i": 0}

            def fn():
                state["i"] = (state["i"] + 1) % len(variants)
                return variants[state["i"]]()
    elif args.op.startswith("bmm"):
        B, M, N, K = args.shape
        a, b = s8(B, M, K, lo=0 if args.op == "bmm_s8t" else -127), s8(B, N, K)
        fn = {"bmm_f32t": lambda: C.bmm_s8t_s8n_f32t(a, b, args.alpha),
              "bmm_s8t": lambda: C.bmm_s8t_s8n_s8t(a, b, args.alpha),
              "bmm_s32t": lambda: C.bmm_s8t_s8n_s32t(a, b)}[args.op]
        ops, nbytes = 2.0 * B * M * N * K, B * (M * K + N * K + M * N * (1 if args.op == "bmm_s8t" else 4))
    elif args.op == "bmm_s8t_rowmajor":
        B, M, N, K = args.shape
        a, b = s8(B, M, K, lo=0), s8(B, K, N)
        fn = lambda: X.bmm_s8t_s8t_s8t(a, b, args.alpha)  # noqa: E731
        ops, nbytes = 2.0 * B * M * N * K, B * (M * K + N * K + M * N)
    elif args.op == "softmax_q":
        batch, heads, T, S = args.shape
        scores = torch.randn(batch * heads, T, S, device=dev, generator=g) * 4
        mask = torch.zeros(T, S, device=dev).masked_fill(
            torch.triu(torch.ones(T, S, dtype=torch.bool, device=dev), 1 + S - T), torch.finfo(torch.float32).min)
        mask = mask[None, None].expand(batch, 1, T, S).contiguous()
        fn = lambda: X.attn_softmax_q(scores, mask, heads)  # noqa: E731
        nbytes = 5.0 * batch * heads * T * S + 4.0 * batch * T * S
    elif args.op == "qk_softmax_q":
        # fused Q.K^T + mask + softmax + quantise: batch, heads, query rows, key rows (head size 128, causal mask)
        batch, heads, T, S = args.shape
        q, k = s8(batch * heads, T, 128), s8(batch * heads, S, 128)
        mask = torch.zeros(T, S, device=dev).masked_fill(
            torch.triu(torch.ones(T, S, dtype=torch.bool, device=dev), 1 + S - T), torch.finfo(torch.float32).min)
        mask = mask[None, None].expand(batch, 1, T, S).contiguous()
        fn = lambda: X.attn_qk_softmax_q(q, k, mask, args.alpha, heads)  # noqa: E731
        ops = 2.0 * batch * heads * T * S * 128
        nbytes = batch * heads * (T * 128 + S * 128 + T * S) + 4.0 * batch * T * S
    elif args.op == "attn_prefill":
        # Q.K^T + softmax-quant + P.V + head merge in one launch: batch, heads, query rows, key rows (head size 128)
        batch, heads, T, S = args.shape
        q, k, vt = s8(batch * heads, T, 128), s8(batch * heads, S, 128), s8(batch * heads, 128, S)
        mask = torch.zeros(T, S, device=dev).masked_fill(
            torch.triu(torch.ones(T, S, dtype=torch.bool, device=dev), 1 + S - T), torch.finfo(torch.float32).min)
        mask = mask[None, None].expand(batch, 1, T, S).contiguous()
        fn = lambda: X.attn_prefill(q, k, vt, mask, args.alpha, 0.004, heads)  # noqa: E731
        ops = 4.0 * batch * heads * T * S * 128
        nbytes = batch * heads * (2 * T * 128 + 2 * S * 128) + 4.0 * batch * T * S
    elif args.op == "decode_attn":
        # one decode step's attention: batch, heads, cached positions, head size, new tokens; --rotate cache copies
        batch, heads, filled, d, T = args.shape
        cap = -(-(filled + T + 64) // 16) * 16
        caches = [(s8(batch, heads, cap, d), s8(batch, heads, cap, d)) for _ in range(args.rotate)]
        q, kn, vn = s8(batch, heads, T, d), s8(batch, heads, T, d), s8(batch, heads, T, d)
        mask = torch.zeros(batch, 1, T, filled + T, device=dev)
        state = {"i": 0}

        def fn():
            state["i"] = (state["i"] + 1) % len(caches)
            kb, vb = caches[state["i"]]
            return X.decode_attention(q, kn, vn, kb, vb, filled, mask, 0.001, 0.004)
        nbytes = 2.0 * batch * heads * (filled + T) * d
    elif args.op == "add_ln_q":
        rows, H = args.shape
        x = torch.randn(rows, H, device=dev, generator=g)
        res = torch.randn(rows, H, device=dev, generator=g)
        gamma, beta = torch.ones(H, device=dev), torch.zeros(H, device=dev)
        fn = lambda: X.add_layernorm_q(x, res, gamma, beta, 1e-5)  # noqa: E731
        nbytes = 13.0 * rows * H + 8 * H
    elif args.op == "ln_q":
        rows, H = args.shape
        inp = torch.randint(-65536, 65536, (rows, H), dtype=torch.int32, device=dev, generator=g)
        res = torch.randn(rows, H, device=dev, generator=g)
        gamma, beta = torch.ones(H, device=dev), torch.zeros(H, device=dev)
        fn = lambda: C.dq_add_layernorm_q(inp, 0.01, res, gamma, beta, 1e-5)  # noqa: E731
        nbytes = 13.0 * rows * H + 8 * H
    elif args.op == "ln_q_f16":
        rows, H = args.shape
        inp = torch.randint(-4096, 4096, (rows, H), dtype=torch.int32, device=dev, generator=g)
        res = torch.randn(rows, H, device=dev, generator=g).half()
        gamma, beta = torch.ones(H, device=dev).half(), torch.zeros(H, device=dev).half()
        fn = lambda: C.dq_add_layernorm_q(inp, 0.01, res, gamma, beta, 1e-5)  # noqa: E731
        nbytes = 9.0 * rows * H + 4 * H
    elif args.op == "transpose_last2":
        # int8 [B, R, C] -> [B, C, R]: V -> V^T in front of P.V; --rotate sources so that none stays cached
        B, R, C_ = args.shape
        srcs = [s8(B, R, C_) for _ in range(max(1, args.rotate))]
        turn = [0]

        def fn():
            turn[0] = (turn[0] + 1) % len(srcs)
            return X.transpose_last2(srcs[turn[0]])
        nbytes = 2.0 * B * R * C_
    elif args.op == "mfma_loop":
        mode, steps = args.shape
        data = (torch.full((1 << 20,), 1, dtype=torch.int8, device=dev) if args.pattern == "constant"
                else s8(1 << 20))
        sink = torch.zeros(1, dtype=torch.int32, device=dev)
        ops = float(X.diag_mfma_loop(mode, data, steps, sink))
        fn = lambda: X.diag_mfma_loop(mode, data, steps, sink)  # noqa: E731
    elif args.op == "store_loop":
        # fp32 [M, N] written with the 256x160 kernel's epilogue stores by `workgroups` workgroups, `reps` times
        M, N, workgroups, reps = args.shape
        out = torch.empty(M, N, device=dev)
        nbytes = float(X.diag_store_loop(out, workgroups, reps))
        fn = lambda: X.diag_store_loop(out, workgroups, reps)  # noqa: E731
    elif args.op == "mix_loop":
        # the instruction mix of one K step of the 256x160 (shape 0) or 128x80 (shape 1) tile, parts as a bit set
        shape, parts, steps = args.shape
        data = (torch.full((3 << 20,), 1, dtype=torch.int8, device=dev) if args.pattern == "constant" else s8(3 << 20))
        sink = torch.zeros(1, dtype=torch.int32, device=dev)
        ops = float(X.diag_mix_loop(shape, parts, data, steps, sink)) if parts & 1 else 0.0
        fn = lambda: X.diag_mix_loop(shape, parts, data, steps, sink)  # noqa: E731
    elif args.op == "copy_loop":
        # every CU fetches 48 KiB per step from an L2-resident 2 MiB with the mainloop's access pattern, nothing else
        mode, steps = args.shape
        data, sink = s8(2 << 20), torch.zeros(1, dtype=torch.int32, device=dev)
        nbytes = float(X.diag_copy_loop(mode, data, steps, sink))
        fn = lambda: X.diag_copy_loop(mode, data, steps, sink)  # noqa: E731
    elif args.op == "read_loop":
        # one read-only pass over an int8 [N, K] matrix; --rotate copies so that none stays in the last-level cache
        mode, N, K = args.shape
        mats, sink = [s8(N, K) for _ in range(max(1, args.rotate))], torch.zeros(1, dtype=torch.int32, device=dev)
        nbytes = float(N) * K
        state = {"i": 0}

        def fn():
            state["i"] += 1
            X.diag_read_loop(mode, mats[state["i"] % len(mats)], sink)
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

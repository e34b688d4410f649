#!/usr/bin/env python3
"""Headline benchmark: the W8A8 linear-kernel sweep at OPT-13B shapes on one MI355X.

One "step" is one pass over the linear-kernel sweep: (N,K) in {(5120,5120), (20480,5120),
(5120,20480)} x M in {1,16,128,512,2048,8192} x the four variants (s32 bias/out, fp32
bias/out, s8 bias/out, fused-ReLU s8 out) = 72 GEMM launches on synthetic int8 data that
is resident in HBM before the clock starts.  `value` = 2*M*N*K summed over the sweep,
divided by the wall time of a step, in TOPS.

Also reported on the same JSON line:
  roofline      the dominant kernel of the sweep (the kernel family with the largest share of
                the launch time): ops per launch / mean launch duration over the launches the
                library routes to it, against 5.0 POP/s, with the other MFMA kernel family and
                all MFMA-bound launches beside it.  The top-level figures come from HIP events
                recorded around the launches inside the timed steps; `sustained` repeats
                the measurement with the reference's own protocol (benchmark/utils.py:81-96:
                100 warm-up launches, then a window of at least 200 ms of back-to-back
                launches of one case), where the clock has settled under the power limit;
  cpu_baseline  the reference's CPU integer emulation (torch int32 matmul + the fp32
                epilogue) timed on this box's host cores on a bounded sample;
  cases         per-case microseconds (sustained protocol; the HBM-bound cases rotate
                through enough weight copies to defeat the 256 MB last-level cache), TOPS,
                GB/s and the binding roofline;
  hbm_kernels   attention BMMs and dq_add_layernorm_q against the 8 TB/s HBM roofline;
  decoder_layer_ms   Int8OPTDecoderLayer at OPT-13B shape (batch 4, seq 512).
"""
import argparse
import contextlib
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "torch-int_amd"), ROOT):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_INT8_TOPS = 5000.0   # MI355X dense INT8 MFMA, TOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s
# Kernel families the large (M >= 2048) sweep cases are routed to, by the label ti_last_kernel() reports: the
# kernel template behind the label at these shapes (K is a multiple of 128 everywhere in the sweep) and the HBM-side
# bytes per launch, averaged over the sweep launches that reach it.  The byte counts cannot be taken from inside
# the process: they come from rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of this script's own sweep; commands,
# raw counter values and the calibration against a plain copy kernel are in profiles/.
FAMILIES = {
    # 233 272 KiB x 2.000 fetched + 77 050 KiB written per launch, mean over its 24 launches per step (measured with
    # the 4 x 8 band of 256x160 tiles per XCD and 3 LDS stages: profiles/bench_py_kernel_trace.md, section 3)
    "pipe16_256x160": {"kernel": "gemm_pipe16q_kernel<Pipe16QCfg<256,160,4,2,KIND,false,3,false>>", "traffic": 0.557e9},
    # 614 663 KiB x 2.000 fetched + 424 056 KiB written per launch, mean over its 4 launches per step
    "pipe_256x256": {"kernel": "gemm_pipe2_kernel<Pipe2Cfg<256,256,2,4,KIND,SWAP>>", "traffic": 1.694e9},
}
# The counter runs behind FAMILIES[*]["traffic"] were made on the kernels as this hash of their source file describes
# them (first 16 hex digits of the SHA-256 of torch-int_amd/csrc/gemm_s8_impl.h).  When the file has changed since,
# the bench line says so next to the figure instead of passing an old measurement off as current.
TRAFFIC_SOURCE_SHA16 = "7d067f298d6aa2ea"


def traffic_is_current():
    import hashlib
    try:
        with open(os.path.join(ROOT, "torch-int_amd", "csrc", "gemm_s8_impl.h"), "rb") as f:
            return hashlib.sha256(f.read()).hexdigest()[:16] == TRAFFIC_SOURCE_SHA16
    except OSError:
        return None


SHAPES = [(5120, 5120), (20480, 5120), (5120, 20480)]   # (N, K): qkv/out_proj, fc1, fc2
MS = [1, 16, 128, 512, 2048, 8192]
VARIANTS = ["b32_o32", "bfp32_ofp32", "b8_o8", "relu_b8_o8"]
BIAS_BYTES = {"b32_o32": 4, "bfp32_ofp32": 4, "b8_o8": 1, "relu_b8_o8": 1}
OUT_BYTES = {"b32_o32": 4, "bfp32_ofp32": 4, "b8_o8": 1, "relu_b8_o8": 1}


class Telemetry:
    """Shader clock and board power of the GPU while a measurement runs, read by a host thread from the amdgpu
    driver's text files: `pp_dpm_sclk` (the line marked * is the current clock, MHz) and hwmon `power1_input`
    (or `power1_average`; microwatts, with `power1_cap` = the board's power limit).  `with tele.window(label):`
    samples every `period_s` for as long as the block runs and keeps mean / min / max under `label`.  Where the
    files do not exist the record says so and nothing else changes."""

    def __init__(self, period_s=0.01):
        import glob
        self.period_s = period_s
        self.windows = {}
        self.sclk_path = self.power_path = None
        self.cap_w = None
        for card in sorted(glob.glob("/sys/class/drm/card[0-9]*")):
            try:
                if open(card + "/device/vendor").read().strip() != "0x1002":
                    continue
            except OSError:
                continue
            if os.path.exists(card + "/device/pp_dpm_sclk"):
                self.sclk_path = card + "/device/pp_dpm_sclk"
            for hw in sorted(glob.glob(card + "/device/hwmon/hwmon*")):
                for name in ("power1_input", "power1_average"):
                    if self.power_path is None and os.path.exists(hw + "/" + name):
                        self.power_path = hw + "/" + name
                try:
                    self.cap_w = int(open(hw + "/power1_cap").read()) / 1e6
                except (OSError, ValueError):
                    pass
            break   # the first AMD card: this build runs on one GPU

    def available(self):
        return self.sclk_path is not None or self.power_path is not None

    def _read(self):
        mhz = watts = None
        try:
            if self.sclk_path:
                for line in open(self.sclk_path):
                    if "*" in line:
                        mhz = float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
            if self.power_path:
                watts = int(open(self.power_path).read()) / 1e6
        except (OSError, ValueError, IndexError):
            pass
        return mhz, watts

    def window(self, label):
        import contextlib
        import threading

        @contextlib.contextmanager
        def cm():
            if not self.available():
                yield
                return
            stop, samples = threading.Event(), []

            def run():
                while not stop.is_set():
                    samples.append(self._read())
                    stop.wait(self.period_s)
            th = threading.Thread(target=run, daemon=True)
            th.start()
            try:
                yield
            finally:
                stop.set()
                th.join()
                clk = [m for m, _ in samples if m is not None]
                pw = [w for _, w in samples if w is not None]
                rec = {"samples": len(samples)}
                if clk:
                    rec.update(sclk_mhz_mean=round(sum(clk) / len(clk), 1), sclk_mhz_min=min(clk), sclk_mhz_max=max(clk))
                if pw:
                    rec.update(power_w_mean=round(sum(pw) / len(pw), 1), power_w_min=round(min(pw), 1), power_w_max=round(max(pw), 1))
                self.windows[label] = rec
        return cm()

    def report(self):
        if not self.available():
            return {"available": False, "note": "no amdgpu pp_dpm_sclk / hwmon power file under /sys/class/drm on this box"}
        return {"available": True, "sclk_file": self.sclk_path, "power_file": self.power_path, "power_cap_w": self.cap_w,
                "period_ms": self.period_s * 1e3, "windows": self.windows,
                "note": "host-thread samples of the driver's text files during each measurement window; sclk is the "
                        "driver's current shader clock (one figure for the whole device), power the board's input power"}


def gemm_bytes(M, N, K, variant):
    return M * K + N * K + N * BIAS_BYTES[variant] + M * N * OUT_BYTES[variant]


def build_sweep(torch, C, dev):
    g = torch.Generator().manual_seed(0)

    def s8(*shape):
        return torch.randint(-127, 128, shape, dtype=torch.int8, generator=g).to(dev)

    cases = []
    for (N, K) in SHAPES:
        w = s8(N, K)
        bias = {
            "b32_o32": torch.randint(-65535, 65535, (N,), dtype=torch.int32, generator=g).to(dev),
            "bfp32_ofp32": torch.randn(N, generator=g).to(dev),
            "b8_o8": s8(N),
        }
        bias["relu_b8_o8"] = bias["b8_o8"]
        for M in MS:
            x = s8(M, K)
            for v in VARIANTS:
                alpha = float(torch.empty(1).uniform_(1e-4, 1e-2, generator=g))
                beta = float(torch.empty(1).uniform_(1e-4, 1e-2, generator=g))
                def make(w, v=v, x=x, b=bias[v], a=alpha, be=beta):
                    if v == "b32_o32":
                        return lambda: C.linear_a8_w8_b32_o32(x, w, b)
                    if v == "bfp32_ofp32":
                        return lambda: C.linear_a8_w8_bfp32_ofp32(x, w, b, a, be)
                    if v == "b8_o8":
                        return lambda: C.linear_a8_w8_b8_o8(x, w, b, a, be)
                    return lambda: C.linear_relu_a8_w8_b8_o8(x, w, b, a, be)
                cases.append({"variant": v, "M": M, "N": N, "K": K, "fn": make(w), "make": make, "w": w, "x": x, "b": bias[v],
                              "ops": 2.0 * M * N * K, "bytes": float(gemm_bytes(M, N, K, v))})
    return cases


def sustained_ms(torch, fns, window_ms=200.0, warm_launches=100):
    """Mean launch duration in ms under upstream's protocol (benchmark/utils.py:81-96): 100 warm-up
    launches, then back-to-back launches between two HIP events on the launch stream, enough of them
    to fill `window_ms`.  `fns` is a list of equivalent closures (e.g. one per weight copy) used round-robin."""
    n = len(fns)
    for i in range(warm_launches):
        fns[i % n]()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for i in range(10):
        fns[i % n]()
    end.record()
    torch.cuda.synchronize()
    est = max(start.elapsed_time(end) / 10, 1e-3)
    iters = max(20, int(window_ms / est) + 1)
    start.record()
    for i in range(iters):
        fns[i % n]()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def cpu_baseline(torch, C=None, dev=None):
    """torch CPU int32 matmul + the oracle's fp32 epilogue (the reference's integer emulation), on an M=256
    slice of each of the sweep's three (N, K) shapes, all four variants: 10-20 s of CPU work.  The same twelve
    problems then run through the HIP path and every output element is compared with the CPU result (the oracle
    as the checker): `gpu_outputs_checked` / `gpu_mismatches`."""
    from oracle import oracle as orc
    g = torch.Generator().manual_seed(0)
    M = 256
    ops = dt = 0.0
    checked = bad = 0
    for N, K in SHAPES:
        x = torch.randint(-127, 128, (M, K), dtype=torch.int8, generator=g)
        w = torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g)
        b8 = torch.randint(-127, 128, (N,), dtype=torch.int8, generator=g)
        b32 = torch.randint(-65535, 65535, (N,), dtype=torch.int32, generator=g)
        bf = torch.randn(N, generator=g)
        t0 = time.perf_counter()
        refs = [orc.linear_a8_w8_b32_o32(x, w, b32, acc_fn=orc.gemm_acc_torch),
                orc.linear_a8_w8_bfp32_ofp32(x, w, bf, 0.001, 1.0, acc_fn=orc.gemm_acc_torch),
                orc.linear_a8_w8_b8_o8(x, w, b8, 0.001, 0.01, acc_fn=orc.gemm_acc_torch),
                orc.linear_relu_a8_w8_b8_o8(x, w, b8, 0.001, 0.01, acc_fn=orc.gemm_acc_torch)]
        dt += time.perf_counter() - t0
        ops += 4 * 2.0 * M * N * K
        if C is not None:
            xd, wd = x.to(dev), w.to(dev)
            outs = [C.linear_a8_w8_b32_o32(xd, wd, b32.to(dev)), C.linear_a8_w8_bfp32_ofp32(xd, wd, bf.to(dev), 0.001, 1.0),
                    C.linear_a8_w8_b8_o8(xd, wd, b8.to(dev), 0.001, 0.01),
                    C.linear_relu_a8_w8_b8_o8(xd, wd, b8.to(dev), 0.001, 0.01)]
            for out, ref in zip(outs, refs):
                checked += ref.numel()
                bad += int((out.cpu() != ref).sum())
    shapes = ", ".join(f"{N}x{K}" for N, K in SHAPES)
    res = {"value": ops / dt / 1e12, "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"4 variants x M={M} rows of each (N,K) in {{{shapes}}}: torch int32 matmul + fp32 epilogue, "
                     f"{dt:.1f} s, host cpu_count={os.cpu_count()}"}
    if C is not None:
        res["gpu_outputs_checked"] = checked
        res["gpu_mismatches"] = bad
    return res


def check_timed_outputs(torch, cases):
    """Every timed b32_o32 case (integer result: acc + bias) against an fp64 product computed by torch on the device,
    on the first and last eight rows of the output, all columns: ties the launches that are timed to correct
    accumulators at the timed shapes without leaving the GPU.  Returns (elements checked, mismatches)."""
    checked = bad = 0
    for c in cases:
        if c["variant"] != "b32_o32":
            continue
        out = c["fn"]()
        M = c["M"]
        rows = sorted(set(range(min(M, 8))) | set(range(max(M - 8, 0), M)))
        x, w, b = c["x"], c["w"], c["b"]
        ref = torch.zeros((len(rows), c["N"]), dtype=torch.float64, device=out.device)
        xs = x[rows].double()
        for k0 in range(0, c["K"], 2560):   # fp64 is exact here; slices keep the converted weights small
            ref += xs[:, k0:k0 + 2560] @ w[:, k0:k0 + 2560].double().t()
        ref = (ref.round().long() + b.long()[None]).to(torch.int32)
        checked += ref.numel()
        bad += int((out[rows] != ref).sum())
    return checked, bad


def hbm_kernels(torch, C, dev):
    """Attention products and LayerNorm-quant against the HBM roofline (algorithmic bytes / duration).
    Inputs rotate through enough copies (> 256 MB) that reads cannot be served from the last-level cache."""
    out = []
    g = torch.Generator().manual_seed(1)

    def rot(t, total_bytes):
        n = min(8, max(2, -(-320 * 2 ** 20 // total_bytes)))
        return [t] + [t.clone() for _ in range(n - 1)]

    for S in (128, 512, 2048):
        q = torch.randint(-127, 128, (160, S, 128), dtype=torch.int8, generator=g).to(dev)
        k = torch.randint(-127, 128, (160, S, 128), dtype=torch.int8, generator=g).to(dev)
        p = torch.randint(0, 128, (160, S, S), dtype=torch.int8, generator=g).to(dev)
        vt = torch.randint(-127, 128, (160, 128, S), dtype=torch.int8, generator=g).to(dev)
        ks = rot(k, 2 * k.numel())
        ms = sustained_ms(torch, [lambda k=k: C.bmm_s8t_s8n_f32t(q, k, 0.002) for k in ks], window_ms=60.0)
        by = 160.0 * (2 * S * 128 + 4 * S * S)
        out.append({"kernel": "bmm_s8t_s8n_f32t", "shape": [160, S, S, 128], "us": ms * 1e3,
                    "GBps": by / ms / 1e6, "frac": by / ms / 1e6 / PEAK_HBM_GBS})
        ps = rot(p, p.numel())
        ms = sustained_ms(torch, [lambda p=p: C.bmm_s8t_s8n_s8t(p, vt, 0.002) for p in ps], window_ms=60.0)
        by = 160.0 * (S * S + 128 * S + S * 128)
        out.append({"kernel": "bmm_s8t_s8n_s8t", "shape": [160, S, 128, S], "us": ms * 1e3,
                    "GBps": by / ms / 1e6, "frac": by / ms / 1e6 / PEAK_HBM_GBS})
        # the whole attention of a prefill in one launch (no counterpart upstream; replaces the two products above, the
        # softmax chain and the head merge): bytes = q, k, v^T, context and one pass over the causal mask
        if S >= 128:   # at S = 128 it replaces two launch-bound products of 7 us each
            import torch_int._hip_ext as X
            neg = torch.finfo(torch.float32).min
            mask = torch.zeros(S, S, device=dev).masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool, device=dev), 1), neg)
            mask = mask[None, None].expand(4, 1, S, S).contiguous()
            # checked once, then called as Int8OPTAttention calls it (the argument checks cost more host time than the
            # 128-key kernel takes on the device)
            assert X.can_attn_prefill(q, k, vt, mask, 4, 40)
            ms = sustained_ms(torch, [lambda: X.attn_prefill(q, k, vt, mask, 0.002, 0.004, 40, checked=True)],
                              window_ms=60.0, warm_launches=10)
            by = 160.0 * 4 * S * 128 + 4.0 * 4 * S * S
            out.append({"kernel": "attn_prefill (fused, causal mask)", "shape": [160, S, S, 128], "us": ms * 1e3,
                        "GBps": by / ms / 1e6, "frac": by / ms / 1e6 / PEAK_HBM_GBS, "bound": "valu"})
        del p, ps, ks
    rows, H = 2048, 5120
    inp = torch.randint(-65536, 65536, (rows, H), dtype=torch.int32, generator=g).to(dev)
    res = torch.randn(rows, H, generator=g).to(dev)
    gamma, beta = torch.ones(H, device=dev), torch.zeros(H, device=dev)
    pairs = list(zip(rot(inp, 8 * inp.numel()), rot(res, 8 * res.numel())))
    ms = sustained_ms(torch, [lambda i=i, r=r: C.dq_add_layernorm_q(i, 0.01, r, gamma, beta, 1e-5) for i, r in pairs],
                      window_ms=60.0)
    by = 13.0 * rows * H + 8 * H
    out.append({"kernel": "dq_add_layernorm_q", "shape": [rows, H], "us": ms * 1e3,
                "GBps": by / ms / 1e6, "frac": by / ms / 1e6 / PEAK_HBM_GBS})
    pairs16 = [(i, r.half()) for i, r in pairs]
    g16, b16 = gamma.half(), beta.half()
    ms = sustained_ms(torch, [lambda i=i, r=r: C.dq_add_layernorm_q(i, 0.01, r, g16, b16, 1e-5) for i, r in pairs16],
                      window_ms=60.0)
    by = 9.0 * rows * H + 4 * H
    out.append({"kernel": "dq_add_layernorm_q (fp16 residual)", "shape": [rows, H], "us": ms * 1e3,
                "GBps": by / ms / 1e6, "frac": by / ms / 1e6 / PEAK_HBM_GBS})
    return out


def decoder_layer_ms(torch, dev):
    from torch_int.models.opt import Int8OPTDecoderLayer
    torch.manual_seed(0)
    D, H, F, B, T = 5120, 40, 20480, 4, 512
    layer = Int8OPTDecoderLayer(D, H, F)
    for lin in (layer.self_attn.q_proj, layer.self_attn.k_proj, layer.self_attn.v_proj, layer.fc1):
        lin.bias = torch.randint(-127, 128, (1, lin.out_features), dtype=torch.int8)
        lin.a.fill_(float(torch.empty(1).uniform_(1e-4, 1e-2)))
        lin.b.fill_(float(torch.empty(1).uniform_(1e-4, 1e-2)))
    for lin in (layer.self_attn.out_proj, layer.fc2):
        lin.bias = torch.randn(1, lin.out_features)
        lin.a.fill_(float(torch.empty(1).uniform_(1e-4, 1e-2)))
    layer.self_attn.qk_bmm.a.fill_(0.003)
    layer.self_attn.pv_bmm.a.fill_(0.004)
    layer = layer.to(dev)
    hidden = torch.randn(B, T, D, device=dev)
    mask = torch.zeros(T, T, device=dev).masked_fill(
        torch.triu(torch.ones(T, T, dtype=torch.bool, device=dev), 1), torch.finfo(torch.float32).min)
    mask = mask[None, None].expand(B, 1, T, T).contiguous()
    # the layer updates its input in place (as upstream does); timing it on the same tensor again and again keeps
    # a 42 MB copy out of the measurement, and LayerNorm keeps the growing residual in range
    return sustained_ms(torch, [lambda: layer(hidden, attention_mask=mask)], window_ms=300.0, warm_launches=20)


def opt66b_model(torch, dev):
    """The OPT-66B-shaped Int8OPTForCausalLM at full depth (64 layers, 65 GB of random int8 weights generated on the
    device): decoder stack of a 512-token prefill and the per-token time of 32 decode steps, batch 1 and 4.  The
    protocol of torch-int_amd/benchmark/bench_opt.py (upstream benchmark/bench_opt.py times the same stack)."""
    import importlib.util
    spec = importlib.util.spec_from_file_location(
        "ti_bench_opt", os.path.join(ROOT, "torch-int_amd", "benchmark", "bench_opt.py"))
    bo = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bo)
    model, cfg = bo.build("opt-66b", 0, dev)
    int8_bytes = sum(b.numel() for _, b in model.named_buffers() if b.dtype == torch.int8)
    D, H, F, L = bo.MODELS["opt-66b"]
    out = {"model": "opt-66b", "layers": L, "int8_weight_GB": int8_bytes / 1e9, "seq": 512, "decode_steps": 32}
    g = torch.Generator(device=dev).manual_seed(1)
    with torch.no_grad():
        for bsz in (4, 1):
            ids = torch.randint(2, cfg.vocab_size, (bsz, 512), device=dev, generator=g)
            model.model(ids, use_cache=True)   # warm-up
            torch.cuda.synchronize()
            t = time.perf_counter()
            for _ in range(3):
                model.model(ids, use_cache=True)
            torch.cuda.synchronize()
            stack_ms = (time.perf_counter() - t) * 1e3 / 3
            o = model(ids, use_cache=True)
            past, tok = o.past_key_values, o.logits[:, -1].argmax(-1, keepdim=True)
            steps = []
            for _ in range(32):
                torch.cuda.synchronize()
                t = time.perf_counter()
                o = model(tok, past_key_values=past, use_cache=True)
                torch.cuda.synchronize()
                steps.append((time.perf_counter() - t) * 1e3)
                past, tok = o.past_key_values, o.logits[:, -1].argmax(-1, keepdim=True)
            med = sorted(steps)[len(steps) // 2]
            ops = 2.0 * bsz * 512 * L * (4 * D * D + 2 * D * F)
            out[f"batch{bsz}"] = {"decoder_stack_ms": stack_ms, "decoder_stack_linear_TOPS": ops / stack_ms / 1e9,
                                  "decode_ms_per_token": med, "decode_weight_GBps": int8_bytes / 1e9 / (med / 1e3),
                                  "logits_finite": bool(torch.isfinite(o.logits).all())}
            del o, past
    del model
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the matrix-pipe ceiling loops")
    ap.add_argument("--sweep-only", action="store_true", help="skip the per-case, HBM-kernel, layer and model sections")
    ap.add_argument("--no-model", action="store_true", help="skip the 64-layer OPT-66B model section")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (the path has no collectives); use --gpus 1")

    import torch
    import torch_int._CUDA as C
    if not torch.cuda.is_available():
        sys.exit("bench.py: no HIP device; the INT8 kernels have no CPU fallback")
    dev = torch.device("cuda:0")
    assert C._lib.ti_init() == 0, C._lib.ti_last_error().decode()

    cases = build_sweep(torch, C, dev)
    sweep_ops = sum(c["ops"] for c in cases)
    C._lib.ti_last_kernel.restype = ctypes.c_char_p
    for c in cases:   # one untimed call each: which kernel family does the library pick for this case?
        c["fn"]()
        c["kernel"] = C._lib.ti_last_kernel().decode()
    torch.cuda.synchronize()

    # launches bracketed by HIP events: everything from M = 512 up (all the cases the tiled MFMA kernels take)
    heavy = [i for i, c in enumerate(cases) if c["M"] >= 512]
    ridge = PEAK_INT8_TOPS * 1e3 / PEAK_HBM_GBS   # ops per byte above which the MFMA roofline binds
    marks = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in heavy]
             for _ in range(args.steps)]

    # A pair of event records costs the stream about 10 us (the command processor serialises on each), which is
    # 4 % of a step if every heavy launch of every step carries one.  Each timed step therefore brackets a
    # rotating quarter of them: launch k in the steps i with (k + i) % stride == 0, so every launch is sampled in
    # steps / stride of the timed steps and every step carries the same share of the overhead.
    stride = max(1, min(4, args.steps))

    def step(ev=None, i=0):
        k = 0
        for c in cases:
            if c["M"] >= 512:
                if ev is not None and (k + i) % stride == 0:
                    ev[k][0].record()
                    c["fn"]()
                    ev[k][1].record()
                else:
                    c["fn"]()
                k += 1
            else:
                c["fn"]()

    tele = Telemetry()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    with tele.window("timed_sweep_steps"):
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(marks[i], i)
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    def launch_ms(k):   # mean duration of heavy launch k over the steps that bracketed it
        took = [marks[i][k][0].elapsed_time(marks[i][k][1]) for i in range(args.steps) if (k + i) % stride == 0]
        return sum(took) / len(took)

    per_launch = [launch_ms(k) for k in range(len(heavy))]
    bound_k = [k for k, i in enumerate(heavy) if cases[i]["ops"] / cases[i]["bytes"] >= ridge]
    heavy_ms = sum(per_launch[k] for k in bound_k)   # per step
    heavy_ops = sum(cases[heavy[k]]["ops"] for k in bound_k)
    # the dominant kernel: the family that takes the largest share of the timed launches
    fam = {}
    for k, i in enumerate(heavy):
        t = per_launch[k]
        f = fam.setdefault(cases[i]["kernel"], {"ms": 0.0, "ops": 0.0, "idx": []})
        f["ms"] += t
        f["ops"] += cases[i]["ops"]
        f["idx"].append(k)
    DOMINANT = max(fam, key=lambda name: fam[name]["ms"])
    dom = fam[DOMINANT]["idx"]
    dom_ms = fam[DOMINANT]["ms"]
    dom_ops = fam[DOMINANT]["ops"]
    value = sweep_ops / (ms_per_step * 1e-3) / 1e12

    result = {
        "metric": "INT8 GEMM TOPS at OPT-13B shapes (W8A8 linear sweep)", "value": value, "unit": "TOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "OPT-13B W8A8 linear sweep: (N,K) in {5120x5120, 20480x5120, 5120x20480} x "
                               "M in {1,16,128,512,2048,8192} x {b32_o32, bfp32_ofp32, b8_o8, relu_b8_o8}",
                   "launches_per_step": len(cases), "ops_per_step": sweep_ops},
    }

    achieved = dom_ops / dom_ms / 1e9
    n_checked, n_bad = check_timed_outputs(torch, cases)
    result["outputs_checked"] = {"elements": n_checked, "mismatches": n_bad,
                                 "what": "the 18 timed b32_o32 cases, first and last 8 rows, against an fp64 product on the "
                                         "device; cpu_baseline.gpu_mismatches covers the other epilogues at M = 256"}
    result["roofline"] = {
        "bound": "mfma", "achieved": achieved, "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
        "frac": achieved / PEAK_INT8_TOPS, "traffic": FAMILIES.get(DOMINANT, {}).get("traffic"),
        "traffic_source": {"counter_run_on_kernel_source_sha16": TRAFFIC_SOURCE_SHA16,
                           "kernel_source_unchanged_since": traffic_is_current()},
        "kernel": FAMILIES.get(DOMINANT, {}).get("kernel", DOMINANT) + " (the sweep cases the library routes to it: "
                  + ", ".join(sorted({f"{cases[heavy[k]]['M']}x{cases[heavy[k]]['N']}x{cases[heavy[k]]['K']}" for k in dom})) + ")",
        "family": DOMINANT,
        "ops_per_launch": dom_ops / len(dom), "avg_launch_ms": dom_ms / len(dom), "launches_per_step": len(dom),
        "protocol": "HIP events around these launches inside the timed steps; each step brackets a rotating quarter of them "
                    "(every launch is sampled in steps / 4 of the timed steps)",
        "all_mfma_bound_cases": {"achieved": heavy_ops / heavy_ms / 1e9, "frac": heavy_ops / heavy_ms / 1e9 / PEAK_INT8_TOPS,
                                 "launches_per_step": len(bound_k), "avg_launch_ms": heavy_ms / len(bound_k)},
        "families": {name: {"kernel": FAMILIES.get(name, {}).get("kernel", name), "launches_per_step": len(f["idx"]),
                            "avg_launch_ms": f["ms"] / len(f["idx"]), "achieved": f["ops"] / f["ms"] / 1e9,
                            "frac": f["ops"] / f["ms"] / 1e9 / PEAK_INT8_TOPS,
                            "traffic": FAMILIES.get(name, {}).get("traffic")} for name, f in fam.items()}}

    if not args.no_ceiling:
        # what the matrix pipe of this board sustains on constant / random operand bytes (diagnostic loops, no GEMM)
        import torch_int._hip_ext as X
        m = X.measure_mfma_ceiling(window_ms=250.0, window=lambda label: tele.window("ceiling_" + label))
        result["roofline"]["measured_ceiling"] = {
            "unit": "TOP/s", "constant": m["mfma_only_constant"], "random": m["mfma_only_random"],
            "lds_fed": m["lds_fed_random"], "all": m,
            "frac_of_lds_fed": achieved / m["lds_fed_random"],
            "step_mix": m["step_mix_256x160_random"], "frac_of_step_mix": achieved / m["step_mix_256x160_random"],
            "note": "back-to-back launches of ti_diag_mfma_loop over 250 ms windows: v_mfma_i32_32x32x32_i8 only "
                    "(constant / random operand bytes), and with LDS fragment reads, global->LDS copies and a barrier "
                    "per step on random bytes (lds_fed); step_mix = ti_diag_mix_loop, the instructions of one K step of "
                    "the 256x160 tile and nothing else (40 v_mfma_i32_16x16x64_i8, 18 fragment reads, 7 copies and a "
                    "barrier per wave) on random bytes: the rate no kernel with this mainloop can exceed on this board; "
                    "the published peak stays the denominator of frac"}
    if not args.sweep_only:
        # per-case launch durations, upstream's protocol; HBM-bound cases rotate weight copies (> 256 MB in total)
        table = []
        mfma_ops = mfma_ms = 0.0
        copies = {}
        for c in cases:
            # the binding roofline by arithmetic intensity (ridge = 5000 TOP/s / 8000 GB/s = 625 ops per byte)
            bound = "mfma" if c["ops"] / c["bytes"] >= PEAK_INT8_TOPS * 1e3 / PEAK_HBM_GBS else "hbm"
            fns = [c["fn"]]
            if c["M"] < 2048:   # weights dominate the traffic: keep them out of the last-level cache
                key = (c["N"], c["K"])
                if key not in copies:
                    # one (N, K) at a time: the copies of the previous shape go back to the device first, so that
                    # torch's caching allocator is not left with gigabytes of split blocks (every output
                    # allocation then costs the host about 10 us, which a 7 us launch cannot hide)
                    copies.clear()
                    torch.cuda.empty_cache()
                    n_copies = -(-320 * 2 ** 20 // (c["N"] * c["K"]))
                    copies[key] = [c["w"]] + [c["w"].clone() for _ in range(n_copies - 1)]
                fns = [c["make"](w) for w in copies[key]]
            label = f"sustained_{c['variant']}_{c['M']}x{c['N']}x{c['K']}"
            with (tele.window(label) if c["kernel"] == DOMINANT and c["M"] >= 2048 and c["variant"] in ("b8_o8", "bfp32_ofp32")
                  else contextlib.nullcontext()):
                ms = sustained_ms(torch, fns, window_ms=200.0 if c["M"] >= 512 and c["kernel"] == DOMINANT or c["M"] >= 2048 else 60.0)
            tops = c["ops"] / ms / 1e9
            gbs = c["bytes"] / ms / 1e6
            frac = tops / PEAK_INT8_TOPS if bound == "mfma" else gbs / PEAK_HBM_GBS
            table.append({"variant": c["variant"], "M": c["M"], "N": c["N"], "K": c["K"], "kernel": c["kernel"],
                          "us": round(ms * 1e3, 2),
                          "TOPS": round(tops, 1), "GBps": round(gbs, 1), "bound": bound, "frac": round(frac, 4)})
            if c["kernel"] == DOMINANT and c["M"] >= 512:
                mfma_ops += c["ops"]
                mfma_ms += ms
        del copies
        sustained = mfma_ops / mfma_ms / 1e9
        result["roofline"]["sustained"] = {
            "achieved": sustained, "frac": sustained / PEAK_INT8_TOPS, "avg_launch_ms": mfma_ms / len(dom),
            "protocol": "same cases, each alone: 100 warm-up launches, then >= 200 ms of back-to-back launches "
                        "between two HIP events (upstream benchmark/utils.py:81-96)"}
        result["cases"] = table
        torch.cuda.empty_cache()   # the per-case section leaves gigabytes of split blocks in the caching allocator
        result["hbm_kernels"] = hbm_kernels(torch, C, dev)
        with tele.window("decoder_layer"):
            result["decoder_layer_ms"] = decoder_layer_ms(torch, dev)
        if not args.no_model:
            result["opt66b"] = opt66b_model(torch, dev)
    # clocks and board power during the windows above: what the power-limit account of the MFMA figures rests on
    result["roofline"]["telemetry"] = tele.report()
    # The published 5.0 POP/s is the matrix pipe at the maximum shader clock.  With the clock the driver reported
    # during the sustained windows of the dominant family (the board holds its power cap there and lowers the clock
    # to do so), the same pipe peaks at 5.0 POP/s x sclk / sclk_max: `frac_at_measured_clock` is the achieved rate
    # against that, i.e. how busy the kernel keeps the pipe at the clock the power limit leaves it.  `frac` above
    # stays priced against the published figure.
    wins = [w for name, w in tele.windows.items() if name.startswith("sustained_") and "sclk_mhz_mean" in w]
    sclk_max = None
    try:
        if tele.sclk_path:
            sclk_max = max(float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
                           for line in open(tele.sclk_path) if ":" in line)
    except (OSError, ValueError):
        sclk_max = None
    if wins and sclk_max and "sustained" in result["roofline"]:
        sclk = sum(w["sclk_mhz_mean"] for w in wins) / len(wins)
        power = [w["power_w_mean"] for w in wins if "power_w_mean" in w]
        result["roofline"]["at_measured_clock"] = {
            "sclk_mhz_mean": round(sclk, 1), "sclk_mhz_max": sclk_max,
            "power_w_mean": round(sum(power) / len(power), 1) if power else None, "power_cap_w": tele.cap_w,
            "peak_at_that_clock": round(PEAK_INT8_TOPS * sclk / sclk_max, 1),
            "frac_at_measured_clock": round(result["roofline"]["sustained"]["achieved"] / (PEAK_INT8_TOPS * sclk / sclk_max), 4),
            "windows": len(wins)}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, C, dev)
    print(json.dumps(result), flush=True)
    mismatches = n_bad + result.get("cpu_baseline", {}).get("gpu_mismatches", 0)
    if mismatches:
        sys.exit(f"bench.py: {mismatches} output elements differ from their references; the figures above are void")


if __name__ == "__main__":
    main()

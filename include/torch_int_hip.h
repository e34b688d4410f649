/*
 * C ABI of libtorch_int_hip.so: hand-written gfx950 (MI355X) kernels for the
 * INT8 W8A8 operator set of torch-int.  Each entry point replaces one function
 * bound by the upstream pybind11 module `torch_int._CUDA`
 * (torch_int/kernels/bindings.cpp:5-20) and is what a binding for that module
 * calls after it has validated and allocated tensors.
 *
 * Conventions shared by every entry point
 *   - all pointers are DEVICE pointers on the current HIP device; operands are
 *     packed row-major with the innermost dimension contiguous;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); the
 *     call only enqueues work, it never synchronises, allocates or frees;
 *   - the return value is 0 on success, otherwise a TI_ERR_* code, and
 *     ti_last_error() gives a human-readable reason for the calling thread;
 *     on error nothing has been launched;
 *   - zero-sized problems (M, N or batch == 0) succeed without a launch;
 *     K == 0 yields the epilogue of an all-zero accumulator.
 *
 * Arithmetic (identical in all kernels)
 *   acc = sum_k int32(x[m,k]) * int32(w[n,k])      exact int32
 *   t   = fmaf(alpha, float(acc), beta * float(bias[n]))
 *   s8 outputs  = (int8) rint(clamp(t, -128, 127))      round-half-to-even
 *   s32 scaled  = saturating (int32) rint(t)
 */
#ifndef TORCH_INT_HIP_H
#define TORCH_INT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TI_OK 0
#define TI_ERR_INVALID_ARG 1   /* null pointer, negative size, size beyond int32 tiling limits */
#define TI_ERR_ALIGNMENT 2     /* pointer not aligned to its element size */
#define TI_ERR_LAUNCH 3        /* hipLaunchKernel reported an error */
#define TI_ERR_NO_DEVICE 4     /* no usable gfx950 device */

/* Library version (major*10000 + minor*100 + patch). */
int ti_version(void);

/* Reason for the last non-zero return on this thread ("" if none). */
const char* ti_last_error(void);

/* Verifies that a HIP device is present and is gfx950; returns TI_OK or
 * TI_ERR_NO_DEVICE.  Optional: every entry point works without it.  It also does, for the current device, the two
 * one-time steps that the first calls would otherwise do: it resolves the address of the built-in scratch buffer
 * of ti_linear_a8_w8_b8_o8_noalloc, and it runs the placement probe of the one-launch split-K (ti_fused_splitk;
 * one small kernel on the null stream, 1 KB of mapped host memory, one synchronisation). */
int ti_init(void);

/* Bytes of scratch the linear entry points can use for (M,N,K) to split the K
 * loop over workgroups when the output has too few tiles to fill the chip
 * (16 < M <= 1024 with a long K, or the last rows of a larger M: see ti_linear_row_split);
 * 0 when no split is worthwhile.  Passing a smaller or NULL workspace is always legal and
 * only selects a non-split kernel. */
int64_t ti_linear_workspace_bytes(int64_t M, int64_t N, int64_t K);

/* Diagnostic: the number r of rows that a linear of this shape cuts off its end and runs as a second, small
 * problem (0 = none).  Tiled kernels pay for whole tiles of 256 rows and whole rounds of 256 CUs; when M > 1024 has
 * a few rows (<= 128) beyond a multiple of 256 and the cost model prices "M - r rows on tiles + r rows through the
 * split-K / streaming kernels" clearly below the whole, the library launches the two (ti_last_kernel then reads
 * "<family>+<family>").  Same bytes out either way.  The reference's CUTLASS kernels predicate partial tiles instead
 * (torch_int/kernels/linear.cu:35-45); prefill lengths are only padded to 16 (torch_int/models/opt.py:375-383). */
int ti_linear_row_split(int64_t M, int64_t N, int64_t K);

/* Diagnostics: the kernel family the calling thread's last linear / bmm_s8t_s8n_* call launched
 * ("pipe_256x256", "pipe16_256x160", "pipe16_256x288", "pipe16_256x128", "pipe16_128x80", "pipe16_128x192", "pipe16_256x192", "pipe_128x128",
 * "splitk_<tile>" and "fusedk_<tile>" for the two- and one-launch split-K forms, "stream", "stream_parts" (the streaming
 * kernel on the view with rows cut into parts), "gemv" (one row of activations), "skinny", "tile_*",
 * "scalar"; grouped launches add "_group": "stream_group", "gemv_group", "pipe16_256x160_group", "pipe16_256x288_group",
 * "pipe16_256x128_group"; "<family>+<family>" when the last rows ran as a second problem, see ti_linear_row_split;
 * "" before the first call).  Benchmarks use it to label their rows. */
const char* ti_last_kernel(void);

/* Switch (no counterpart in the reference): split-K linears whose tile is one of the 16x16-block kernel's and
 * divides M run as ONE launch ("fusedk_*" in ti_last_kernel): the K slices of an output tile run on workgroups
 * of one XCD and meet in its L2, the last wave to arrive adds them up and applies the epilogue; same bits as the
 * two-launch form ("splitk_*": raw int32 slices + a reduction kernel), which everything else takes.
 * enable = 1 / 0 turns the one-launch form on / off for the process, -1 leaves it; returns the setting before
 * the call.  Default on, or off with the environment variable TORCH_INT_FUSED_SPLITK=0.  The form also stays off
 * on a device whose workgroup placement is not "ids congruent mod 8 share an XCD" (probed at the first use),
 * for more than 8 streams per device, and while a stream is being captured before the first use on its device.
 * Each stream has arrival counters of its own (8 sets per device; a stream that has gone idle hands its set on when
 * a ninth stream needs one).  The first split-K call on a stream runs a placement probe on it: one small kernel and
 * ONE SYNCHRONISATION of that stream (not during a capture, where the call takes the two-launch form instead, and
 * not from ti_linear_a8_w8_b8_o8_noalloc); ti_init() does it for the null stream.
 * Workspace: the one-launch form needs `workspace` on a 256-byte boundary (a 16-byte aligned one takes the
 * two-launch form).
 * HIP graphs: a launch recorded into a graph keeps the arrival counters (and the caller's workspace) of the stream
 * it was recorded on.  Replays of such a graph must therefore not overlap in time with other split-K linears
 * issued on the recording stream, nor with replays of another graph recorded on that same stream.
 * Misplacement: every one-launch GEMM checks that the workgroups of a tile ran on one XCD.  If one did not, the
 * output of THAT call cannot be trusted although it returned TI_OK (the check runs on the device, after the call
 * has returned): the next linear / bmm call on the device, whatever its shape, returns TI_ERR_LAUNCH once, naming
 * the earlier call as the one to re-run, and the form switches itself off; a caller that makes no further call
 * asks ti_fused_splitk_faulted() after it has synchronised.  No box of this pool has ever raised it. */
int ti_fused_splitk(int enable);

/* 1 when a one-launch split-K GEMM that has finished on the current device found a workgroup on an unexpected XCD
 * (see ti_fused_splitk), else 0.  Reads one word of host memory; call it after synchronising with the launches in
 * question.  No counterpart in the reference. */
int ti_fused_splitk_faulted(void);

/* Self-tests of the one-launch split-K's host-side bookkeeping (no GPU call, no counterpart in the reference):
 * ti_selftest_fused_flag_action = what a GEMM call does for a device state (0 not probed, 1 usable, -1 off) and a
 * misplacement flag: 1 go on, 0 take the two-launch form, -1 report the misplacement;
 * ti_selftest_fused_slot = the slot of `stream` in a table of `cap` (<= 32) streams, bit i of live_mask / busy_mask
 * saying whether slot i is registered / still has work queued; *fresh = 1 when the stream was not registered. */
int ti_selftest_fused_flag_action(int state, int flag, int enabled, int64_t counters, int64_t max_counters);
int ti_selftest_fused_slot(int64_t* table, uint32_t* live_mask, int cap, int64_t stream, uint32_t busy_mask,
                           int* fresh);

/* Diagnostic (no counterpart in the reference; computes nothing): one launch that issues the instruction mix of
 * the tiled GEMM mainloop `iters` times per wave on the first MiB of `data` (device memory, at least 1 MiB, 16-byte
 * aligned), so that a benchmark can measure what the matrix pipe of this board sustains for a given operand
 * pattern (fill `data` with a constant or with random bytes).  mode 0: v_mfma_i32_32x32x32_i8 only; 1: plus the
 * LDS fragment reads; 2: plus global->LDS copies from an L2-resident source and a workgroup barrier per step.
 * `sink` is one int32 of device memory (written only if the accumulators hit a magic value).
 * ti_diag_mfma_loop_ops(iters) = integer operations one such launch performs on the current device. */
int ti_diag_mfma_loop(int mode, const int8_t* data, int64_t data_bytes, int64_t iters, int32_t* sink, void* stream);
int64_t ti_diag_mfma_loop_ops(int64_t iters);

/* Diagnostic (no counterpart in the reference): `workgroups` workgroups write 1.0f to every element of the fp32
 * matrix out[M, N] (row-major; M a multiple of 256, N of 160), `reps` times, tile by tile with the store instructions
 * and addresses of the 256x160 GEMM kernel's 32-bit epilogue and nothing else: a benchmark times it to learn what
 * one CU (few workgroups) or the whole chip (one workgroup per CU) can store. */
int ti_diag_store_loop(float* out, int64_t M, int64_t N, int workgroups, int reps, void* stream);

/* Diagnostic (no counterpart in the reference; computes nothing): one workgroup of eight waves per CU fetches, `iters`
 * times, 48 KiB (a 256x160 tile's share of one 128-byte K step) as row pieces of 128 contiguous bytes from rows 5120
 * bytes apart in the first 2 MiB of `data` (device memory, at least 2 MiB, 16-byte aligned; shared by all workgroups,
 * so it is served by the L2), two steps in flight.  mode 0: global->LDS copies; 1: 16-byte loads into registers.  A
 * benchmark times it to learn what the copy path alone delivers per CU.  `sink` as for ti_diag_mfma_loop.
 * ti_diag_copy_loop_bytes(iters) = bytes one such launch fetches on the current device. */
int ti_diag_copy_loop(int mode, const int8_t* data, int64_t data_bytes, int64_t iters, int32_t* sink, void* stream);
int64_t ti_diag_copy_loop_bytes(int64_t iters);

/* Diagnostic (no counterpart in the reference; computes nothing): one pass over an int8 matrix data[N][K] (N a multiple
 * of 16, K of 1024, 16-byte aligned device memory of N*K bytes) with the loads alone, to learn what a kernel that reads
 * its weights once can reach.  mode 0: flat 4 KiB pieces per workgroup, four loads in flight per lane; 1: the same,
 * non-temporal; 2: the copy pipeline of the M <= 16 streaming GEMM without its arithmetic (strips of 16 rows, 1 KiB per
 * row and global->LDS copy, three stages, one wait and barrier per block, two workgroups per CU, non-temporal copies);
 * 3: mode 2 with the default cache policy.  `sink` as for ti_diag_mfma_loop. */
int ti_diag_read_loop(int mode, const int8_t* data, int64_t N, int64_t K, int32_t* sink, void* stream);

/* Diagnostic (no counterpart in the reference; computes nothing): one workgroup per CU issues, `iters` times, the
 * instructions a wave of the 16x16-block GEMM kernels issues per 128-byte K step and nothing else, on operands that
 * change every step.  shape 0 = the 256x160 tile (8 waves, each 40 v_mfma_i32_16x16x64_i8, 18 ds_read_b128, 7 1-KiB
 * global->LDS copies), shape 1 = the 128x80 tile (4 waves, each 20 / 14 / 7).  parts is a bit set: 1 MFMAs, 2 fragment
 * reads, 4 copies and their wait, 8 workgroup barrier.  `data`: at least 3 MiB of device memory, 16-byte aligned (fill
 * it with random bytes); `sink` as for ti_diag_mfma_loop.  The time per step of parts = 15 is the floor of that
 * kernel's K step on the board; ti_diag_mix_loop_ops(shape, iters) = integer operations of a launch with bit 1 set. */
int ti_diag_mix_loop(int shape, int parts, const int8_t* data, int64_t data_bytes, int64_t iters, int32_t* sink,
                     void* stream);
int64_t ti_diag_mix_loop_ops(int shape, int64_t iters);

/* ---- W8A8 linear: out[M,N] = epilogue(x[M,K] . w[N,K]^T, bias[N]) ---- */

/* replaces linear_a8_w8_b32_o32 (torch_int/kernels/linear.cu:13-136;
 * declared torch_int/kernels/include/linear.h:6-9): out = acc + bias, int32. */
int ti_linear_a8_w8_b32_o32(const int8_t* x, const int8_t* w, const int32_t* bias, int32_t* out,
                            int64_t M, int64_t N, int64_t K,
                            void* workspace, int64_t workspace_bytes, void* stream);

/* replaces linear_a8_w8_b32_o32_with_scaling (linear.cu:139-243; linear.h:12-17):
 * out = sat_s32(rint(alpha*acc + beta*bias)). */
int ti_linear_a8_w8_b32_o32_with_scaling(const int8_t* x, const int8_t* w, const int32_t* bias,
                                         int32_t* out, int64_t M, int64_t N, int64_t K,
                                         float alpha, float beta,
                                         void* workspace, int64_t workspace_bytes, void* stream);

/* replaces linear_a8_w8_bfp32_ofp32 (linear.cu:246-365; linear.h:20-25):
 * out = alpha*acc + beta*bias, fp32 bias and output. */
int ti_linear_a8_w8_bfp32_ofp32(const int8_t* x, const int8_t* w, const float* bias, float* out,
                                int64_t M, int64_t N, int64_t K, float alpha, float beta,
                                void* workspace, int64_t workspace_bytes, void* stream);

/* replaces linear_a8_w8_b8_o8 (linear.cu:369-473; linear.h:36-41):
 * out = s8(rint(clamp(alpha*acc + beta*bias, -128, 127))). */
int ti_linear_a8_w8_b8_o8(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out,
                          int64_t M, int64_t N, int64_t K, float alpha, float beta,
                          void* workspace, int64_t workspace_bytes, void* stream);

/* ti_linear_a8_w8_b8_o8 for callers that cannot allocate device memory or pass a workspace (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.
 * Same arguments minus the workspace, same bytes out.  The split-K partial products go to a buffer of
 * TI_NOALLOC_SCRATCH_BYTES that is part of the library's device image (one copy per GPU, held until the
 * process ends); the call allocates and frees nothing.  Shapes whose split needs more
 * (ti_linear_workspace_bytes(M, N, K) > TI_NOALLOC_SCRATCH_BYTES) are refused with TI_ERR_INVALID_ARG.
 * Every call on a GPU shares that GPU's buffer: calls that may overlap in time on one GPU (different
 * streams, different threads) race and must be serialised by the caller.  The buffer needs no clearing
 * between calls (every partial product is written before it is read).  ti_init() resolves the buffer's address
 * for the current device; without it the first call on a device does.  The one-launch split-K is used only on a
 * device where its probe has already run (ti_init() or an earlier workspace call), since the probe allocates. */
#define TI_NOALLOC_SCRATCH_BYTES (40 * 1024 * 1024)
int ti_linear_a8_w8_b8_o8_noalloc(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out,
                                  int64_t M, int64_t N, int64_t K, float alpha, float beta, void* stream);

/* linear_a8_w8_b8_o8 whose [M, N] result is stored head-major: with M = B*T rows and N = H*head_dim columns,
 * element (b*T + t, h*head_dim + dd) goes to out[b][h][t][dd] of a packed [B, H, T, head_dim] tensor.  The
 * values are those of ti_linear_a8_w8_b8_o8; this replaces the `view(B,T,H,d).transpose(1,2).contiguous()`
 * that follows the q/k/v projections (torch_int/models/opt.py:80-81).  T divides M, head_dim divides N and is
 * a multiple of 16. */
int ti_linear_a8_w8_b8_o8_heads(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out, int64_t M,
                                int64_t N, int64_t K, float alpha, float beta, int64_t T, int64_t head_dim,
                                void* workspace, int64_t workspace_bytes, void* stream);

/* `count` (<= 4) linear_a8_w8_b8_o8 problems that share the input x[M,K] and the shape: out[i] =
 * s8(rint(clamp(alpha[i]*(x . w[i]^T) + beta[i]*bias[i]))).  w, bias, out, alpha, beta are HOST arrays of
 * `count` device pointers / scalars.  The q, k and v projections of one attention block
 * (torch_int/models/opt.py:108-126 calls them one after the other); for M <= 16 with K % 1024 == 0 all
 * weights are streamed by a single launch, for M > 128 with N % 160 == 0 or N % 288 == 0 and K % 128 == 0 the
 * problems are the batches of one persistent tiled launch, other shapes run problem by problem.  Results are those of
 * `count` separate calls. */
int ti_linear_a8_w8_b8_o8_group(const int8_t* x, const int8_t* const* w, const int8_t* const* bias,
                                int8_t* const* out, const float* alpha, const float* beta, int64_t count,
                                int64_t M, int64_t N, int64_t K, void* stream);

/* ti_linear_a8_w8_b8_o8_group with every output stored head-major as by ti_linear_a8_w8_b8_o8_heads: the
 * q, k and v projections of a prefill (torch_int/models/opt.py:108-126 followed by the `_shape` permutations,
 * :80-81) as one call.  When N is a multiple of 160 or 288, K of 128 and M > 128, the problems run as the
 * batches of one persistent launch; other shapes run problem by problem.  Results are those of `count`
 * separate calls. */
int ti_linear_a8_w8_b8_o8_group_heads(const int8_t* x, const int8_t* const* w, const int8_t* const* bias,
                                      int8_t* const* out, const float* alpha, const float* beta, int64_t count,
                                      int64_t M, int64_t N, int64_t K, int64_t T, int64_t head_dim, void* stream);

/* Diagnostic (no counterpart in the reference): 1 when a group call of `count` problems of that shape runs as ONE
 * launch on the current device (the streaming kernel for M <= 16 with K % 1024 == 0; a persistent tiled launch when
 * the 256x160, 256x288 or 256x128 tiles divide N, K % 128 == 0, M > 128, and the cost model does not price the
 * problems' own one-round tilings below it), 0 when it loops over the problems - without the split-K workspace that
 * separate ti_linear_a8_w8_b8_o8 calls could be given, so a caller that holds one does better with those. */
int ti_linear_group_is_one_launch(int64_t M, int64_t N, int64_t K, int count);

/* replaces linear_relu_a8_w8_b8_o8 (linear.cu:476-625; linear.h:28-33):
 * out = s8(rint(min(max(alpha*acc + beta*bias, 0), 127))). */
int ti_linear_relu_a8_w8_b8_o8(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out,
                               int64_t M, int64_t N, int64_t K, float alpha, float beta,
                               void* workspace, int64_t workspace_bytes, void* stream);

/* ---- batched A . B^T: c[b,M,N] = epilogue(a[b,M,K] . b[b,N,K]^T) ---- */

/* replaces bmm_s8t_s8n_f32t (torch_int/kernels/bmm.cu:10-108; include/bmm.h:4):
 * c = alpha * float(acc). */
int ti_bmm_s8t_s8n_f32t(const int8_t* a, const int8_t* b, float* c,
                        int64_t batch, int64_t M, int64_t N, int64_t K, float alpha, void* stream);

/* replaces bmm_s8t_s8n_s8t (bmm.cu:110-208; bmm.h:6):
 * c = s8(rint(clamp(alpha * float(acc), -128, 127))). */
int ti_bmm_s8t_s8n_s8t(const int8_t* a, const int8_t* b, int8_t* c,
                       int64_t batch, int64_t M, int64_t N, int64_t K, float alpha, void* stream);

/* replaces bmm_s8t_s8n_s32t (bmm.cu:210-295; bmm.h:8): c = acc. */
int ti_bmm_s8t_s8n_s32t(const int8_t* a, const int8_t* b, int32_t* c,
                        int64_t batch, int64_t M, int64_t N, int64_t K, void* stream);

/* The three batched products with a split-K workspace (no counterpart in the reference, whose GemmBatched takes
 * none): same arguments, same bytes out as ti_bmm_s8t_s8n_*.  When the problems together have too few output tiles
 * to fill the chip and the inner dimension is long - upstream's own benchmark/bench_bmm.py:9-15 multiplies
 * [batch, seq, 12288] operands, batch 1..16 - K is cut into slices that run side by side (raw int32 partial
 * products in `workspace`, then one reduction launch; a single problem takes the linears' forms, the one-launch one
 * included).  ti_bmm_workspace_bytes = bytes that lets the library do so for a shape (0 = it would not split;
 * attention-shaped products, K = head size, never do); a smaller or NULL workspace only selects the unsplit kernels. */
int64_t ti_bmm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K);
int ti_bmm_s8t_s8n_f32t_ws(const int8_t* a, const int8_t* b, float* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                           float alpha, void* workspace, int64_t workspace_bytes, void* stream);
int ti_bmm_s8t_s8n_s8t_ws(const int8_t* a, const int8_t* b, int8_t* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                          float alpha, void* workspace, int64_t workspace_bytes, void* stream);
int ti_bmm_s8t_s8n_s32t_ws(const int8_t* a, const int8_t* b, int32_t* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                           void* workspace, int64_t workspace_bytes, void* stream);

/* ---- fused dequantise + residual add + LayerNorm + quantise ---- */

/* replaces dq_add_layernorm_q (torch_int/kernels/fused.cu:5-25; include/fused.h:6-14):
 *   r_out[row,i] = fmaf(input_scale, float(input[row,i]), residual[row,i])
 *   q_out[row,i] = s8(rint(clamp(LN(r_out[row,:])[i] * gamma[i] + beta[i], -128, 127)))
 * over `rows` rows of H elements; biased variance, eps added before the sqrt.
 * r_out may alias residual (in-place residual stream). */
int ti_dq_add_layernorm_q(const int32_t* input, float input_scale, const float* residual,
                          const float* gamma, const float* beta, float eps,
                          float* r_out, int8_t* q_out, int64_t rows, int64_t H, void* stream);

/* dq_add_layernorm_q on an fp16 residual stream with fp16 gamma and beta (the reference's op is ATen and takes
 * them: torch_int/kernels/fused.cu:17-24, called that way by benchmark/bench_dq_add_ln_q.py:37-45).  residual,
 * gamma, beta and r_out point to IEEE binary16 values.  The arithmetic is fp32 and rounds where the reference's
 * chain of torch ops on fp16 tensors rounds:
 *   r_out = f16(fmaf(input_scale, float(f16(input)), float(residual)))     (|input| >= 65520 -> infinity)
 *   y     = f16(LN(float(r_out))[i] * float(gamma[i]) + float(beta[i]))
 *   q_out = s8(rint(clamp(float(y), -128, 127)))
 * r_out may alias residual. */
int ti_dq_add_layernorm_q_f16(const int32_t* input, float input_scale, const void* residual, const void* gamma,
                              const void* beta, float eps, void* r_out, int8_t* q_out, int64_t rows, int64_t H,
                              void* stream);

/* ---- fused element-wise chains of the OPT blocks (no counterpart in the reference's native
 * module: upstream runs these as sequences of torch ops) ---- */

/* inout[m,n] = inout[m,n] + fmaf(alpha, acc, beta*bias[n]): linear_a8_w8_bfp32_ofp32 whose result is added
 * (one fp32 add, after the linear's own rounding) into a tensor that is already there.  Replaces
 * `residual.add_(fc2(x))` (torch_int/models/opt.py:287-289) without the intermediate [M,N] tensor. */
int ti_linear_a8_w8_bfp32_ofp32_acc(const int8_t* x, const int8_t* w, const float* bias, float* inout,
                                    int64_t M, int64_t N, int64_t K, float alpha, float beta,
                                    void* workspace, int64_t workspace_bytes, void* stream);

/* x != NULL: residual[row,i] += x[row,i] (in place), then
 *            q_out = s8(clamp(rint(LN(residual[row,:])[i] * gamma[i] + beta[i]), -128, 127));
 * x == NULL: the same without the add (residual is only read).
 * Replaces `residual.add_(h); LayerNormQ(residual)` (torch_int/models/opt.py:281-283) and
 * LayerNormQ.forward on fp32 input (torch_int/nn/fused.py:13-18). */
int ti_add_layernorm_q(const float* x, float* residual, const float* gamma, const float* beta, float eps,
                       int8_t* q_out, int64_t rows, int64_t H, void* stream);

/* ti_add_layernorm_q on an fp16 residual stream with fp16 x, gamma and beta (LayerNormQ of a model converted
 * with .half(), torch_int/nn/fused.py:13-18): residual = f16(float(residual) + float(x)) in place when x != NULL,
 * then y = f16(LN(float(residual)) * gamma + beta), q_out = s8(rint(clamp(float(y), -128, 127))). */
int ti_add_layernorm_q_f16(const void* x, void* residual, const void* gamma, const void* beta, float eps,
                           int8_t* q_out, int64_t rows, int64_t H, void* stream);

/* The same with an fp32 x on the fp16 stream: residual = f16(float(residual) + float(f16(x))) in place, i.e.
 * `residual.add_(x.to(residual.dtype))` as the decoder layer adds the fp32 output of out_proj to an fp16 residual
 * (torch_int/models/opt.py:281), then the LayerNorm-quantiser as above.  x must not be NULL. */
int ti_add_layernorm_q_f16_xf32(const float* x, void* residual, const void* gamma, const void* beta, float eps,
                                int8_t* q_out, int64_t rows, int64_t H, void* stream);

/* residual[i] = f16(float(residual[i]) + float(f16(x[i]))) for n elements, in place: `residual.add_(x.to(residual.dtype))`
 * of an fp32 x on an fp16 residual stream in one pass (torch_int/models/opt.py:289, the fp32 output of fc2). */
int ti_add_f16_xf32(const float* x, void* residual, int64_t n, void* stream);

/* probs[b*heads+h, t, s] = s8(rint(127 * softmax_s(max(scores[b*heads+h,t,s] + mask[b,0,t,s], -FLT_MAX))));
 * scores [batch*heads, T, S] fp32, mask [batch, 1, T, S] fp32 or NULL.
 * Replaces the mask add, clamp, softmax, *127, round and int8 cast between the two
 * attention products (torch_int/models/opt.py:144-178). */
int ti_attn_softmax_q(const float* scores, const float* mask, int8_t* probs, int64_t batch, int64_t heads,
                      int64_t T, int64_t S, void* stream);

/* bmm_s8t_s8n_f32t whose operands need not be packed along the batch dimension: stride_a / stride_b are the
 * elements between consecutive batches of a / b (0 = packed; each [M,K] / [N,K] matrix itself stays packed).
 * Lets Q.K^T read K from a KV-cache buffer that has spare room after every head
 * (torch_int/models/opt.py:128-133 concatenates the cache instead). */
int ti_bmm_s8t_s8n_f32t_strided(const int8_t* a, const int8_t* b, float* c, int64_t batch, int64_t M, int64_t N,
                                int64_t K, int64_t stride_a, int64_t stride_b, float alpha, void* stream);

/* c[b,M,N] = s8(rint(clamp(alpha * a[b,M,K] . bm[b,K,N], -128, 127))) with bm ROW-major (not transposed):
 * the P.V product on V as the KV cache stores it, replacing `value_states.transpose(1, 2).contiguous()`
 * followed by bmm_s8t_s8n_s8t (torch_int/models/opt.py:180-182) when few query rows are live
 * (incremental decoding).  Any M works, 16 rows per pass over bm; any K and N (no multiple-of-16 rule).
 * stride_b = elements between consecutive batches of bm (0 = packed K*N). */
int ti_bmm_s8t_s8t_s8t(const int8_t* a, const int8_t* bm, int8_t* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                       int64_t stride_b, float alpha, void* stream);

/* dst[b, y, x, :] = src[b, x, y, :] for int8 [B, X, Y, D]: the head split / merge
 * `view(B,T,H,d).transpose(1,2).contiguous()` (torch_int/models/opt.py:80-81,189-196). */
int ti_permute_0213_s8(const int8_t* src, int8_t* dst, int64_t B, int64_t X, int64_t Y, int64_t D, void* stream);

/* dst[b, c, r] = src[b, r, c] for int8 [B, R, C]: `value_states.transpose(1, 2).contiguous()`
 * (torch_int/models/opt.py:180). */
int ti_transpose_last2_s8(const int8_t* src, int8_t* dst, int64_t B, int64_t R, int64_t C, void* stream);

/* k_buf[bh, S + t, :] = k_new[bh, t, :] and v_buf[bh, S + t, :] = v_new[bh, t, :] for t < T: appends the new
 * tokens' keys and values ([BH, T, D] packed) to cache buffers [BH, cap, D] that hold S positions, in one launch.
 * Replaces the two `torch.cat([past, new], dim=2)` of torch_int/models/opt.py:128-133, which copy the whole
 * cache at every decode step. */
int ti_kv_append_s8(const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf, int64_t BH, int64_t T,
                    int64_t D, int64_t cap, int64_t S, void* stream);

/* The attention of a prefill step in one launch (torch_int/models/opt.py:137-196): ctx[b, t, h*D:(h+1)*D] =
 * s8(alpha_pv * sum_s p[t, s] * v[s, :]) with p the int8 probabilities of ti_attn_qk_softmax_q, i.e. the chain
 * ti_bmm_s8t_s8n_f32t, ti_attn_softmax_q, ti_bmm_s8t_s8n_s8t and the head merge `transpose(1,2).reshape(...)`,
 * same bits, without the score and probability tensors.  vt is V transposed, [BH, D, S] packed (what
 * ti_transpose_last2_s8 makes, as upstream's `value_states.transpose(1,2).contiguous()`); ctx is [BH/heads, T,
 * heads*D] packed.  Limits (ti_attn_prefill_supported): S a multiple of 16 in [16, 4096] and D a multiple of 16 up to
 * 128 (OPT-2.7B: 80; rows keep their own length in memory).  Up to 576 keys all keys
 * of a head sit in the LDS and are swept once; other shapes sweep the keys three times in tiles of 256 (row maximum, row
 * sum, probabilities): the same bits either way. */
int ti_attn_prefill_supported(int64_t T, int64_t S, int64_t D);
int ti_attn_prefill_s8(const int8_t* q, const int8_t* k, const int8_t* vt, const float* mask, int8_t* ctx, int64_t BH,
                       int64_t T, int64_t S, int64_t D, int64_t stride_q, int64_t stride_k, int64_t heads,
                       float alpha_qk, float alpha_pv, void* stream);

/* One launch for the attention of an incremental decoding step (torch_int/models/opt.py:128-190 with T new
 * tokens and a KV cache): appends k_new / v_new ([BH, T, D] packed) at positions S-T .. S-1 of the cache buffers
 * ([BH, cap, D], S positions after the append; pass NULL for both to attend over a cache that already holds
 * them), then ctx[bh, t, :] = s8(alpha_pv * sum_s p[t, s] * v[s, :]) with p = round(127 * softmax(max(alpha_qk *
 * q.k^T + mask, FLT_MIN_NEG))) -- the same arithmetic, bit for bit, as ti_bmm_s8t_s8n_f32t, ti_attn_softmax_q and
 * ti_bmm_s8t_s8t_s8t chained.  mask is fp32 [BH/heads, 1, T, S] or NULL; probs_out ([BH, T, S] int8) receives the
 * quantised probabilities when not NULL.  Limits: 1 <= T <= 4, D a multiple of 16 up to 128 (OPT-2.7B: 80), and the scores of one
 * (batch, head) must fit the LDS: ti_decode_attn_supported(T, S, D) says whether a shape is accepted. */
int ti_decode_attn_supported(int64_t T, int64_t S, int64_t D);
int ti_decode_attn_s8(const int8_t* q, const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf,
                      const float* mask, int8_t* ctx, int8_t* probs_out, int64_t BH, int64_t T, int64_t D, int64_t cap,
                      int64_t S, int64_t heads, float alpha_qk, float alpha_pv, void* stream);

/* ti_decode_attn_s8 for a launch that is recorded once (HIP graph capture) and replayed while the cache grows: the
 * number of positions after the append is read from device memory (*s_dev, T <= *s_dev <= S_max) when the kernel
 * runs, S_max is the largest value it will ever hold (the launch is sized for it; S_max <= cap).  No mask, no
 * probabilities out; k_new / v_new are appended at positions *s_dev - T .. *s_dev - 1.  Same arithmetic and bits as
 * ti_decode_attn_s8 with S = *s_dev.  No counterpart in the reference (its decode step is re-issued from Python). */
int ti_decode_attn_s8_devlen(const int8_t* q, const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf,
                             int8_t* ctx, int64_t BH, int64_t T, int64_t D, int64_t cap, int64_t S_max,
                             const int32_t* s_dev, int64_t heads, float alpha_qk, float alpha_pv, void* stream);

/* probs[bh, t, :] = int8 round(127 * softmax(max(alpha * q[bh, t, :] . k[bh, :, :]^T + mask, most negative float)))
 * in one launch: ti_bmm_s8t_s8n_f32t followed by ti_attn_softmax_q (torch_int/models/opt.py:137-178) without the
 * fp32 score tensor in between; the same bits.  q is [BH, T, D] with stride_q elements between batches, k is
 * [BH, S, D] with stride_k, rows packed; mask fp32 [BH/heads, 1, T, S] or NULL; probs [BH, T, S] packed.
 * Limits: S a multiple of 16 in [16, 4096] and D a multiple of 16 up to 128:
 * ti_attn_qk_softmax_q_supported(T, S, D) says whether a shape is accepted. */
int ti_attn_qk_softmax_q_supported(int64_t T, int64_t S, int64_t D);
int ti_attn_qk_softmax_q(const int8_t* q, const int8_t* k, const float* mask, int8_t* probs, int64_t BH, int64_t T,
                         int64_t S, int64_t D, int64_t stride_q, int64_t stride_k, int64_t heads, float alpha,
                         void* stream);

/* Classes of an additive attention mask, an optional accelerator for the two prefill entry points above (no
 * counterpart in the reference).  classes[b][i][j] describes the mask values of batch b, query rows 64 i .. 64 i + 63,
 * keys 256 j .. 256 j + 255: 1 = all of them are +-0 (the kernels then do not read them), 2 = all of them are one
 * and the same value, -1e30 or below (the row-maximum sweep of the long-prefill kernel then takes that value instead
 * of loading keys and multiplying), 0 = anything else.  ti_attn_mask_classes fills the array (one read of the mask;
 * ti_attn_mask_classes_bytes = its size, 0 when the shape takes none), once per mask: every head and every layer that
 * adds the same mask shares it.  The _mc entry points are ti_attn_qk_softmax_q / ti_attn_prefill_s8 with that
 * array (NULL = none); the bits of the results do not depend on it.  Under a causal mask only the tiles on the
 * diagonal are class 0, which removes most of the mask traffic and half of the first sweep. */
int64_t ti_attn_mask_classes_bytes(int64_t batch, int64_t T, int64_t S);
int ti_attn_mask_classes(const float* mask, uint8_t* classes, int64_t batch, int64_t T, int64_t S, void* stream);
int ti_attn_qk_softmax_q_mc(const int8_t* q, const int8_t* k, const float* mask, const uint8_t* mask_classes,
                            int8_t* probs, int64_t BH, int64_t T, int64_t S, int64_t D, int64_t stride_q,
                            int64_t stride_k, int64_t heads, float alpha, void* stream);
int ti_attn_prefill_s8_mc(const int8_t* q, const int8_t* k, const int8_t* vt, const float* mask,
                          const uint8_t* mask_classes, int8_t* ctx, int64_t BH, int64_t T, int64_t S, int64_t D,
                          int64_t stride_q, int64_t stride_k, int64_t heads, float alpha_qk, float alpha_pv, void* stream);

/* One decode step of one decoder layer (torch_int/models/opt.py:202-299, Int8OPTDecoderLayer.forward, with one new token
 * per sequence and a KV cache) from one call: LayerNormQ, the q/k/v projections, the cache append and the attention,
 * out_proj, the residual update fused with the second LayerNormQ, fc1 (ReLU) and fc2 added into the residual
 * stream.  Each step is the entry point above that the modules call for it (ti_add_layernorm_q[_f16[_xf32]],
 * ti_linear_a8_w8_b8_o8_group, ti_decode_attn_s8, ti_linear_a8_w8_bfp32_ofp32[_acc], ti_linear_relu_a8_w8_b8_o8,
 * ti_add_f16_xf32), with the same arguments: the values are theirs; what the call saves is the host time of eight
 * trips through the caller's language.  hidden is the residual stream [B, 1, embed] (fp32, or fp16 with half = 1: then
 * the LayerNorm parameters are fp16 too), updated in place; mask fp32 [B, 1, 1, S] or NULL; k_buf / v_buf the cache
 * buffers [B, heads, cap, head_dim] holding S - 1 positions, S after the call; scratch: device memory of
 * ti_opt_decoder_layer_decode_scratch_bytes(B, embed, ffn) bytes on a 256-byte boundary (the layers of a model can
 * share it: calls on one stream run one after the other).  B <= 16. */
typedef struct TiOptDecodeLayer {
  int64_t embed, heads, head_dim, ffn;
  int32_t half;                 /* 1: residual stream and LayerNorm parameters are fp16 */
  float ln1_eps, ln2_eps;
  const void *ln1_gamma, *ln1_beta, *ln2_gamma, *ln2_beta;
  const int8_t *wq, *wk, *wv;   /* [embed, embed] */
  const int8_t *bq, *bk, *bv;   /* [embed] */
  float alpha_q, alpha_k, alpha_v, beta_q, beta_k, beta_v;
  float alpha_qk, alpha_pv;     /* scales of the two attention products */
  const int8_t* wo;             /* out_proj [embed, embed], fp32 bias, beta = 1 */
  const float* bo;
  float alpha_o;
  const int8_t* w1;             /* fc1 [ffn, embed], int8 bias */
  const int8_t* b1;
  float alpha_1, beta_1;
  const int8_t* w2;             /* fc2 [embed, ffn], fp32 bias, beta = 1 */
  const float* b2;
  float alpha_2;
} TiOptDecodeLayer;
int64_t ti_opt_decoder_layer_decode_scratch_bytes(int64_t B, int64_t embed, int64_t ffn);
int ti_opt_decoder_layer_decode(const TiOptDecodeLayer* layer, void* hidden, const float* mask, int8_t* k_buf,
                                int8_t* v_buf, int64_t B, int64_t cap, int64_t S, void* scratch, int64_t scratch_bytes,
                                void* stream);

/* The same for a prefill (Int8OPTDecoderLayer.forward, torch_int/models/opt.py:202-299, on T > 16 tokens per sequence
 * without a cache): LayerNormQ, the q/k/v projections stored head-major (one grouped launch where
 * ti_linear_group_is_one_launch says so, else three calls with the workspace), V transposed, the one-launch prefill
 * attention with the head merge (ti_attn_prefill_s8_mc), out_proj, the residual update fused with the second
 * LayerNormQ, fc1 (ReLU), fc2 added into the residual stream -- the entry points and arguments of the module path, so
 * its values.  hidden [B, T, embed] is updated in place; mask fp32 [B, 1, T, T] or NULL, mask_classes its class array
 * (ti_attn_mask_classes) or NULL; k_out / v_out receive the key and value rows [B, heads, T, head_dim] (the cache the
 * decode steps continue).  T a multiple of 16 that ti_attn_prefill_supported(T, T, head_dim) accepts, B * T <= 4096
 * (larger prefills are bound by their kernels, not by the host).  scratch:
 * ti_opt_decoder_layer_prefill_scratch_bytes(B * T, embed, ffn) bytes on a 256-byte boundary; workspace: the split-K
 * workspace of the linears (ti_linear_workspace_bytes of the largest of them, or NULL). */
int64_t ti_opt_decoder_layer_prefill_scratch_bytes(int64_t rows, int64_t embed, int64_t ffn);
int ti_opt_decoder_layer_prefill(const TiOptDecodeLayer* layer, void* hidden, const float* mask,
                                 const uint8_t* mask_classes, int8_t* k_out, int8_t* v_out, int64_t B, int64_t T,
                                 void* scratch, int64_t scratch_bytes, void* workspace, int64_t workspace_bytes,
                                 void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TORCH_INT_HIP_H */

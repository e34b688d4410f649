// Shared declarations for the gfx950 INT8 kernels: error reporting, vector
// types and the fp32 epilogues every GEMM/BMM kernel applies to its int32
// accumulators.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/torch_int_hip.h"

namespace ti {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Records a formatted reason for the calling thread and returns `code`.
int fail(int code, const char* fmt, ...);

// ---------------------------------------------------------------- epilogues
// Kinds of output transform.  The *_BIAS kinds read a per-column bias.
enum EpiKind : int {
  EPI_S32_BIAS = 0,    // out = acc + bias                      (int32, wrapping)
  EPI_S32_SCALED = 1,  // out = sat_s32(rint(fma(a, acc, b*bias)))
  EPI_F32_BIAS = 2,    // out = fma(a, acc, b*bias)             (fp32 bias)
  EPI_S8_BIAS = 3,     // out = s8(rint(clamp(fma(a, acc, b*bias))))
  EPI_S8_RELU = 4,     // out = s8(rint(min(max(fma(..), 0), 127)))
  EPI_F32_SCALE = 5,   // out = a * acc
  EPI_S8_SCALE = 6,    // out = s8(rint(clamp(a * acc)))
  EPI_S32_RAW = 7,     // out = acc
  EPI_F32_BIAS_ACC = 8,  // out = out + fma(a, acc, b*bias)   (fp32; adds into the tensor already there)
};

// round-half-even then v_cvt_i32_f32, which saturates to int32 and maps NaN to 0
__device__ __forceinline__ int rne_sat_s32(float t) {
  const float r = __builtin_rintf(t);
  int o;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(o) : "v"(r));
  return o;
}

// s8(rint(clamp(t, lo, 127))): rounding first and clamping the integer gives the same
// value for every finite t (the bounds are integers), one VALU op cheaper.
template <int LO>
__device__ __forceinline__ int rne_clamp(float t) {
  int i = rne_sat_s32(t);
  i = i < LO ? LO : i;
  i = i > 127 ? 127 : i;
  return i;
}
__device__ __forceinline__ int rne_s8(float t) { return rne_clamp<-128>(t); }

template <int KIND>
struct Epi;

template <>
struct Epi<EPI_S32_BIAS> {
  using Out = int32_t;
  using Bias = int32_t;
  static constexpr bool kHasBias = true;
  static constexpr bool kAccumulate = false;
  // the "bias term" is carried as raw bits so one code path serves all kinds
  static __device__ __forceinline__ float bias_term(Bias b, float) { return __int_as_float(b); }
  static __device__ __forceinline__ Out apply(int acc, float bt, float) {
    return (int32_t)((uint32_t)acc + (uint32_t)__float_as_int(bt));
  }
};
template <>
struct Epi<EPI_S32_SCALED> {
  using Out = int32_t;
  using Bias = int32_t;
  static constexpr bool kHasBias = true;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias b, float beta) { return beta * (float)b; }
  static __device__ __forceinline__ Out apply(int acc, float bt, float alpha) {
    return rne_sat_s32(__builtin_fmaf(alpha, (float)acc, bt));
  }
};
template <>
struct Epi<EPI_F32_BIAS> {
  using Out = float;
  using Bias = float;
  static constexpr bool kHasBias = true;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias b, float beta) { return beta * b; }
  static __device__ __forceinline__ Out apply(int acc, float bt, float alpha) {
    return __builtin_fmaf(alpha, (float)acc, bt);
  }
};
template <>
struct Epi<EPI_S8_BIAS> {
  using Out = int8_t;
  using Bias = int8_t;
  static constexpr bool kHasBias = true;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias b, float beta) { return beta * (float)(int)b; }
  // the output value as an int in [-128, 127] (for epilogues that pack bytes themselves)
  static __device__ __forceinline__ int apply_int(int acc, float bt, float alpha) {
    return rne_s8(__builtin_fmaf(alpha, (float)acc, bt));
  }
  static __device__ __forceinline__ Out apply(int acc, float bt, float alpha) { return (int8_t)apply_int(acc, bt, alpha); }
};
template <>
struct Epi<EPI_S8_RELU> {
  using Out = int8_t;
  using Bias = int8_t;
  static constexpr bool kHasBias = true;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias b, float beta) { return beta * (float)(int)b; }
  static __device__ __forceinline__ int apply_int(int acc, float bt, float alpha) {
    // relu then clamp == integer clamp to [0, 127] after rounding (NaN -> 0 either way)
    return rne_clamp<0>(__builtin_fmaf(alpha, (float)acc, bt));
  }
  static __device__ __forceinline__ Out apply(int acc, float bt, float alpha) { return (int8_t)apply_int(acc, bt, alpha); }
};
template <>
struct Epi<EPI_F32_SCALE> {
  using Out = float;
  using Bias = float;
  static constexpr bool kHasBias = false;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias, float) { return 0.0f; }
  static __device__ __forceinline__ Out apply(int acc, float, float alpha) { return alpha * (float)acc; }
};
template <>
struct Epi<EPI_S8_SCALE> {
  using Out = int8_t;
  using Bias = int8_t;
  static constexpr bool kHasBias = false;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias, float) { return 0.0f; }
  static __device__ __forceinline__ int apply_int(int acc, float, float alpha) { return rne_s8(alpha * (float)acc); }
  static __device__ __forceinline__ Out apply(int acc, float bt, float alpha) { return (int8_t)apply_int(acc, bt, alpha); }
};
template <>
struct Epi<EPI_S32_RAW> {
  using Out = int32_t;
  using Bias = int32_t;
  static constexpr bool kHasBias = false;
  static constexpr bool kAccumulate = false;
  static __device__ __forceinline__ float bias_term(Bias, float) { return 0.0f; }
  static __device__ __forceinline__ Out apply(int acc, float, float) { return acc; }
};

template <>
struct Epi<EPI_F32_BIAS_ACC> {
  using Out = float;
  using Bias = float;
  static constexpr bool kHasBias = true;
  static constexpr bool kAccumulate = true;  // the stores add to what the output already holds
  static __device__ __forceinline__ float bias_term(Bias b, float beta) { return beta * b; }
  static __device__ __forceinline__ Out apply(int acc, float bt, float alpha) {
    return __builtin_fmaf(alpha, (float)acc, bt);
  }
};

// `fresh` for the ordinary kinds; `*where + fresh` (one fp32 add, the linear's own result rounded first)
// for the accumulate-into-output kind.
template <class E>
__device__ __forceinline__ typename E::Out merge_old(typename E::Out fresh, const typename E::Out* where) {
  if constexpr (E::kAccumulate)
    return *where + fresh;
  else
    return fresh;
}

// Problem description handed to every GEMM kernel.  A is [batch, M, K], B is
// [batch, N, K], C is [batch, M, N], all packed; bias is [N] (shared by batches).
struct GemmParams {
  const int8_t* A;
  const int8_t* B;
  const void* bias;
  void* C;
  int M, N, K, batch;
  int lda, ldb;                         // bytes between consecutive rows of A and B (>= K)
  long long strideA, strideB, strideC;  // elements between consecutive batches
  float alpha, beta;
  // Head-major output (out_d > 0): row m = (b, t) with t < out_T, column n = (h, dd) with dd < out_d is
  // stored as element [b][h][t][dd] of a packed [M/out_T, N/out_d, out_T, out_d] tensor -- the layout the
  // attention products want, written by the projection itself.  0 = plain row-major [M, N].  8-bit outputs only.
  int out_T = 0, out_d = 0;
  // Head-major output of a problem that is the last rows of a larger one: row m of this problem is row m + m_base
  // of the whole (plain row-major output needs no such field: C points at the first row).
  int m_base = 0;
  // Tile rows an XCD's run of tiles walks down before it moves to the next tile column (see tile_of_workgroup).
  int band = 8;
  // gemm_pipe_kernel: all tiles of a batch on one XCD (see decode_item there)
  int group_batches = 0;
  // Split-K inside one launch (the FUSED form of the 16x16-block kernel): K is the length of one slice, strideA and
  // strideB step from slice to slice; `parts` holds splits x tiles parked accumulator tiles, `arrivals` one zeroed
  // counter per (tile, wave), `xcc_seen` one zeroed word per tile in which the workgroups of the tile mark the XCC
  // they run on, xcc_error = host-mapped word that is set when two of them differ.
  int splits = 1;
  // Split-K of a batched product (the pipelined kernels): batch index b of the launch is (problem b / kslices,
  // K slice b % kslices); problems are strideA / strideB apart, slices strideAk / strideBk (K is one slice's length).
  int kslices = 1;
  long long strideAk = 0, strideBk = 0;
  void* parts = nullptr;
  int* arrivals = nullptr;
  unsigned* xcc_seen = nullptr;
  int* xcc_error = nullptr;
};

// First byte of the A / B operand of batch index b of a launch.
__device__ __forceinline__ const int8_t* a_of_batch(const GemmParams& p, int b) {
  if (p.kslices > 1) {
    const int bb = b / p.kslices;
    return p.A + (long long)bb * p.strideA + (long long)(b - bb * p.kslices) * p.strideAk;
  }
  return p.A + (long long)b * p.strideA;
}
__device__ __forceinline__ const int8_t* b_of_batch(const GemmParams& p, int b) {
  if (p.kslices > 1) {
    const int bb = b / p.kslices;
    return p.B + (long long)bb * p.strideB + (long long)(b - bb * p.kslices) * p.strideBk;
  }
  return p.B + (long long)b * p.strideB;
}

// Offset of output element (m, n) of one batch; consecutive n stay consecutive inside a head, so vector
// stores of VEC columns starting at a multiple of VEC are unaffected when out_d % VEC == 0.
__device__ __forceinline__ long long out_index(const GemmParams& p, int m, int n) {
  if (p.out_d == 0) return (long long)m * p.N + n;
  m += p.m_base;
  const int b = m / p.out_T, t = m - b * p.out_T;
  const int h = n / p.out_d, dd = n - h * p.out_d;
  return (((long long)b * (p.N / p.out_d) + h) * p.out_T + t) * p.out_d + dd;
}

// Up to four linears that share the activation matrix and the shape (the q/k/v projections of one
// attention block) run as one launch: problem i has its own weight, bias, output and scales.
struct GemmGroup {
  const int8_t* B[4];
  const void* bias[4];
  void* C[4];
  float alpha[4], beta[4];
  int count;
};
int launch_gemm_group_s8(const GemmParams& shape, const GemmGroup& grp, hipStream_t stream);

// Launchers (gemm_s8.hip).  `kind` is an EpiKind.  Returns a TI_* status.
int launch_gemm(int kind, const GemmParams& p, void* workspace, long long workspace_bytes,
                hipStream_t stream);
long long gemm_workspace_bytes(long long M, long long N, long long K);
int gemm_group_is_one_launch(long long M, long long N, long long K, int count);
int gemm_row_split(long long M, long long N, long long K);
long long bmm_workspace_bytes(long long batch, long long M, long long N, long long K);  // split-K scratch of a batched product  // rows a linear cuts off its end and runs as a second problem
void allow_fused_split_probe(bool allow);  // per thread: may a GEMM call run the one-time placement probe?
int warm_fused_split(void* stream);        // run that probe now (1 = the one-launch split-K is usable on this device)
int fused_split_faulted();                 // 1 = a one-launch split-K on the current device flagged a misplaced workgroup
int fused_flag_action(int state, int flag, bool enabled, long long counters, long long max_counters);
int fused_slot_for_test(long long* table, unsigned* live_mask, int cap, long long stream, unsigned busy_mask, int* fresh);
int set_fused_split(int enable);  // one-launch split-K on (1) / off (0) / unchanged (-1); returns the previous setting
const char* last_gemm_kernel();  // kernel family of the calling thread's last launch_gemm ("" before the first)

// ln_q.hip
int launch_dq_add_layernorm_q(const int32_t* in, float scale, const float* res, const float* gamma,
                              const float* beta, float eps, float* r_out, int8_t* q_out,
                              long long rows, long long H, hipStream_t stream);

int launch_add_layernorm_q(const float* x, float* residual, const float* gamma, const float* beta, float eps,
                           int8_t* q_out, long long rows, long long H, hipStream_t stream);

int launch_dq_add_layernorm_q_f16(const int32_t* in, float scale, const void* res, const void* gamma, const void* beta,
                                  float eps, void* r_out, int8_t* q_out, long long rows, long long H,
                                  hipStream_t stream);
int launch_add_f16_xf32(const float* x, void* residual, long long n, hipStream_t stream);
int launch_add_layernorm_q_f16_xf32(const float* x, void* residual, const void* gamma, const void* beta, float eps,
                                    int8_t* q_out, long long rows, long long H, hipStream_t stream);
int launch_add_layernorm_q_f16(const void* x, void* residual, const void* gamma, const void* beta, float eps,
                               int8_t* q_out, long long rows, long long H, hipStream_t stream);

// softmax_q.hip
int launch_attn_softmax_q(const float* scores, const float* mask, int8_t* out, long long batch, long long heads,
                          long long T, long long S, hipStream_t stream);

// permute.hip
int launch_permute_0213_s8(const int8_t* src, int8_t* dst, long long B, long long X, long long Y, long long D,
                           hipStream_t stream);
int launch_transpose_last2_s8(const int8_t* src, int8_t* dst, long long B, long long R, long long C,
                              hipStream_t stream);
bool attn_qk_softmax_q_supported(long long T, long long S, long long D);
bool attn_prefill_supported(long long T, long long S, long long D);
int launch_attn_qk_softmax_q(const int8_t* q, const int8_t* k, const float* mask, int8_t* probs, long long BH,
                             long long T, long long S, long long D, long long stride_q, long long stride_k,
                             long long heads, float alpha, const int8_t* vt, int8_t* ctx, float alpha_pv,
                             hipStream_t stream, const unsigned char* mask_classes = nullptr);
long long attn_mask_classes_bytes(long long batch, long long T, long long S);
int launch_attn_mask_classes(const float* mask, unsigned char* cls, long long batch, long long T, long long S,
                             hipStream_t stream);
bool decode_attn_supported(long long T, long long S, long long D);
int launch_decode_attn_s8(const int8_t* q, const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf,
                          const float* mask, int8_t* ctx, int8_t* probs_out, long long BH, long long T, long long D,
                          long long cap, long long S, long long heads, float alpha_qk, float alpha_pv,
                          hipStream_t stream, const int* s_dev = nullptr);
int launch_kv_append_s8(const int8_t* knew, const int8_t* vnew, int8_t* kbuf, int8_t* vbuf, long long BH, long long T,
                        long long D, long long cap, long long S, hipStream_t stream);

// diag_mfma.hip
int launch_diag_mfma_loop(int mode, const int8_t* data, long long iters, int* sink, hipStream_t stream);
long long diag_mfma_loop_ops(long long iters);
int launch_diag_store_loop(float* out, long long M, long long N, int workgroups, int reps, hipStream_t stream);
int launch_diag_read_loop(int mode, const int8_t* data, long long N, long long K, int* sink, hipStream_t stream);
int launch_diag_copy_loop(int mode, const int8_t* data, long long iters, int* sink, hipStream_t stream);
long long diag_copy_loop_bytes(long long iters);
int launch_diag_mix_loop(int shape, int parts, const int8_t* data, long long iters, int* sink, hipStream_t stream);
long long diag_mix_loop_ops(int shape, long long iters);

// bmm_rowmajor.hip
int launch_bmm_s8t_s8t_s8t(const int8_t* a, const int8_t* b, int8_t* c, long long batch, long long M, long long N,
                           long long K, long long stride_b, float alpha, hipStream_t stream);

}  // namespace ti

// extern "C" surface of libtorch_int_hip.so: argument validation and dispatch.
// Declarations and the contract of each entry point live in
// include/torch_int_hip.h.
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include "ti_common.h"

// Split-K scratch of ti_linear_a8_w8_b8_o8_noalloc: int32 partial products [slices][M][N].  One copy of the
// array lives on every GPU the library runs on, from the moment the code object is loaded there until the
// process ends.  In host code this name is only a handle for hipGetSymbolAddress; kernels and copies get the
// device address that scratch_address() returns.  (No `used` attribute here: with it the device compiler emits
// the array before it has seen the host code that names it, keeps the symbol local to the code object, and the
// runtime's lookup in hipGetSymbolAddress aborts the process.)
static __device__ __align__(256) unsigned char scratch[TI_NOALLOC_SCRATCH_BYTES];

namespace ti {

static thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

// Device address of `scratch` on the current device (each GPU has its own copy at its own address), looked
// up once per device.  Racing first calls store the same value.
static constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

static int scratch_address(const char* op, void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TI_ERR_NO_DEVICE, "%s: hipGetDevice: %s", op, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(TI_ERR_NO_DEVICE, "%s: device index %d is beyond the %d devices the scratch table covers", op, dev,
                kMaxDevices);
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(TI_ERR_NO_DEVICE, "%s: hipGetSymbolAddress(scratch) on device %d: %s", op, dev,
                  hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return TI_OK;
}

static int check_dims(const char* op, int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (batch < 0 || M < 0 || N < 0 || K < 0)
    return fail(TI_ERR_INVALID_ARG, "%s: negative dimension (batch=%lld M=%lld N=%lld K=%lld)", op,
                (long long)batch, (long long)M, (long long)N, (long long)K);
  const int64_t lim = 0x7fffffffLL;
  if (M > lim || N > lim || K > lim || batch > 65535 || M * K > lim || N * K > lim)
    return fail(TI_ERR_INVALID_ARG,
                "%s: size beyond kernel limits (batch<=65535, M*K and N*K < 2^31 per batch; got batch=%lld "
                "M=%lld N=%lld K=%lld)",
                op, (long long)batch, (long long)M, (long long)N, (long long)K);
  return TI_OK;
}

static int check_ptr(const char* op, const char* name, const void* p, size_t align, bool needed) {
  if (!needed) return TI_OK;
  if (p == nullptr) return fail(TI_ERR_INVALID_ARG, "%s: %s is NULL", op, name);
  if (reinterpret_cast<uintptr_t>(p) % align)
    return fail(TI_ERR_ALIGNMENT, "%s: %s is not aligned to %zu bytes", op, name, align);
  return TI_OK;
}

static int run_gemm(const char* op, int kind, const void* a, const void* b, const void* bias, size_t bias_elt,
                    void* c, size_t out_elt, int64_t batch, int64_t M, int64_t N, int64_t K, float alpha,
                    float beta, void* ws, int64_t ws_bytes, void* stream, int64_t stride_a = 0,
                    int64_t stride_b = 0, int64_t out_T = 0, int64_t out_d = 0) {
  g_err[0] = 0;
  if (int rc = check_dims(op, batch, M, N, K)) return rc;
  // batch strides (elements between consecutive batches of a / b); 0 = packed
  if (stride_a == 0) stride_a = M * K;
  if (stride_b == 0) stride_b = N * K;
  if (stride_a < M * K || stride_b < N * K)
    return fail(TI_ERR_INVALID_ARG, "%s: batch strides (%lld, %lld) are smaller than one batch (%lld, %lld)", op,
                (long long)stride_a, (long long)stride_b, (long long)(M * K), (long long)(N * K));
  const bool nonempty = batch > 0 && M > 0 && N > 0;
  if (int rc = check_ptr(op, "input", a, 1, nonempty && K > 0)) return rc;
  if (int rc = check_ptr(op, "weight", b, 1, nonempty && K > 0)) return rc;
  if (int rc = check_ptr(op, "bias", bias, bias_elt ? bias_elt : 1, nonempty && bias_elt > 0)) return rc;
  if (int rc = check_ptr(op, "output", c, out_elt, nonempty)) return rc;
  if (ws_bytes < 0) return fail(TI_ERR_INVALID_ARG, "%s: negative workspace size", op);
  GemmParams p;
  p.A = static_cast<const int8_t*>(a);
  p.B = static_cast<const int8_t*>(b);
  p.bias = bias;
  p.C = c;
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.batch = (int)batch;
  p.lda = (int)K;
  p.ldb = (int)K;
  p.strideA = stride_a;
  p.strideB = stride_b;
  p.strideC = M * N;
  p.alpha = alpha;
  p.beta = beta;
  if (out_T != 0 || out_d != 0) {
    if (out_T <= 0 || out_d <= 0 || M % out_T != 0 || N % out_d != 0 || out_d % 16 != 0)
      return fail(TI_ERR_INVALID_ARG,
                  "%s: head-major output needs T > 0 dividing M and head_dim > 0 dividing N, a multiple of 16 "
                  "(got M=%lld N=%lld T=%lld head_dim=%lld)",
                  op, (long long)M, (long long)N, (long long)out_T, (long long)out_d);
    p.out_T = (int)out_T;
    p.out_d = (int)out_d;
  }
  return launch_gemm(kind, p, ws, ws_bytes, static_cast<hipStream_t>(stream));
}

}  // namespace ti

using namespace ti;

extern "C" {

int ti_version(void) { return 100; }

const char* ti_last_error(void) { return g_err; }

int ti_init(void) {
  g_err[0] = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(TI_ERR_NO_DEVICE, "hipGetDevice: %s", hipGetErrorString(e));
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return fail(TI_ERR_NO_DEVICE, "hipGetDeviceProperties: %s", hipGetErrorString(e));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(TI_ERR_NO_DEVICE, "device %d is %s; this library holds gfx950 code only", dev, prop.gcnArchName);
  void* ptr = nullptr;  // resolve the no-allocation entry point's scratch here, outside any capture or hot loop
  if (int rc = scratch_address("ti_init", &ptr)) return rc;
  (void)warm_fused_split(nullptr);  // and probe the workgroup placement the one-launch split-K relies on
  return TI_OK;
}

int64_t ti_linear_workspace_bytes(int64_t M, int64_t N, int64_t K) { return gemm_workspace_bytes(M, N, K); }
int ti_linear_row_split(int64_t M, int64_t N, int64_t K) { return gemm_row_split(M, N, K); }
int ti_linear_group_is_one_launch(int64_t M, int64_t N, int64_t K, int count) {
  return M > 0 && N > 0 && K > 0 && count > 0 ? gemm_group_is_one_launch(M, N, K, count) : 0;
}

int ti_linear_a8_w8_b32_o32(const int8_t* x, const int8_t* w, const int32_t* bias, int32_t* out, int64_t M,
                            int64_t N, int64_t K, void* ws, int64_t ws_bytes, void* stream) {
  return run_gemm("linear_a8_w8_b32_o32", EPI_S32_BIAS, x, w, bias, 4, out, 4, 1, M, N, K, 1.0f, 1.0f, ws,
                  ws_bytes, stream);
}

int ti_linear_a8_w8_b32_o32_with_scaling(const int8_t* x, const int8_t* w, const int32_t* bias, int32_t* out,
                                         int64_t M, int64_t N, int64_t K, float alpha, float beta, void* ws,
                                         int64_t ws_bytes, void* stream) {
  return run_gemm("linear_a8_w8_b32_o32_with_scaling", EPI_S32_SCALED, x, w, bias, 4, out, 4, 1, M, N, K, alpha,
                  beta, ws, ws_bytes, stream);
}

int ti_linear_a8_w8_bfp32_ofp32(const int8_t* x, const int8_t* w, const float* bias, float* out, int64_t M,
                                int64_t N, int64_t K, float alpha, float beta, void* ws, int64_t ws_bytes,
                                void* stream) {
  return run_gemm("linear_a8_w8_bfp32_ofp32", EPI_F32_BIAS, x, w, bias, 4, out, 4, 1, M, N, K, alpha, beta, ws,
                  ws_bytes, stream);
}

int ti_linear_a8_w8_bfp32_ofp32_acc(const int8_t* x, const int8_t* w, const float* bias, float* inout, int64_t M,
                                    int64_t N, int64_t K, float alpha, float beta, void* ws, int64_t ws_bytes,
                                    void* stream) {
  return run_gemm("linear_a8_w8_bfp32_ofp32_acc", EPI_F32_BIAS_ACC, x, w, bias, 4, inout, 4, 1, M, N, K, alpha, beta,
                  ws, ws_bytes, stream);
}

int ti_linear_a8_w8_b8_o8(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out, int64_t M,
                          int64_t N, int64_t K, float alpha, float beta, void* ws, int64_t ws_bytes,
                          void* stream) {
  return run_gemm("linear_a8_w8_b8_o8", EPI_S8_BIAS, x, w, bias, 1, out, 1, 1, M, N, K, alpha, beta, ws,
                  ws_bytes, stream);
}

int ti_linear_a8_w8_b8_o8_noalloc(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out, int64_t M,
                                  int64_t N, int64_t K, float alpha, float beta, void* stream) {
  const char* op = "linear_a8_w8_b8_o8_noalloc";
  g_err[0] = 0;
  if (int rc = check_dims(op, 1, M, N, K)) return rc;
  const int64_t need = gemm_workspace_bytes(M, N, K);
  if (need > (int64_t)TI_NOALLOC_SCRATCH_BYTES)
    return fail(TI_ERR_INVALID_ARG,
                "%s: M=%lld N=%lld K=%lld needs %lld bytes of split-K scratch, the built-in buffer holds %lld; "
                "call ti_linear_a8_w8_b8_o8 with a workspace of your own",
                op, (long long)M, (long long)N, (long long)K, (long long)need, (long long)TI_NOALLOC_SCRATCH_BYTES);
  void* ws = nullptr;
  if (need > 0) {
    if (int rc = scratch_address(op, &ws)) return rc;
  }
  // the partial products are written in full before they are read: nothing to clear.  The one-launch split-K is
  // taken only on a device where its one-time probe (which allocates) has already run, e.g. through ti_init().
  allow_fused_split_probe(false);
  const int rc = run_gemm(op, EPI_S8_BIAS, x, w, bias, 1, out, 1, 1, M, N, K, alpha, beta, ws, need > 0 ? need : 0,
                          stream);
  allow_fused_split_probe(true);
  return rc;
}

int ti_linear_a8_w8_b8_o8_heads(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out, int64_t M,
                                int64_t N, int64_t K, float alpha, float beta, int64_t T, int64_t head_dim,
                                void* ws, int64_t ws_bytes, void* stream) {
  return run_gemm("linear_a8_w8_b8_o8_heads", EPI_S8_BIAS, x, w, bias, 1, out, 1, 1, M, N, K, alpha, beta, ws,
                  ws_bytes, stream, 0, 0, T, head_dim);
}

static int linear_group(const char* op, const int8_t* x, const int8_t* const* w, const int8_t* const* bias,
                        int8_t* const* out, const float* alpha, const float* beta, int64_t count, int64_t M, int64_t N,
                        int64_t K, int64_t T, int64_t head_dim, void* stream) {
  g_err[0] = 0;
  if (count < 0 || count > 4) return fail(TI_ERR_INVALID_ARG, "%s: 0 to 4 problems per group, got %lld", op, (long long)count);
  if (int rc = check_dims(op, 1, M, N, K)) return rc;
  const bool nonempty = count > 0 && M > 0 && N > 0;
  if (!nonempty) return TI_OK;
  if (w == nullptr || bias == nullptr || out == nullptr || alpha == nullptr || beta == nullptr)
    return fail(TI_ERR_INVALID_ARG, "%s: a per-problem array is NULL", op);
  if (int rc = check_ptr(op, "input", x, 1, K > 0)) return rc;
  GemmGroup grp{};
  grp.count = (int)count;
  for (int i = 0; i < count; ++i) {
    if (int rc = check_ptr(op, "weight", w[i], 1, K > 0)) return rc;
    if (int rc = check_ptr(op, "bias", bias[i], 1, true)) return rc;
    if (int rc = check_ptr(op, "output", out[i], 1, true)) return rc;
    grp.B[i] = w[i];
    grp.bias[i] = bias[i];
    grp.C[i] = out[i];
    grp.alpha[i] = alpha[i];
    grp.beta[i] = beta[i];
  }
  GemmParams p;
  p.A = x;
  p.B = grp.B[0];
  p.bias = grp.bias[0];
  p.C = grp.C[0];
  p.M = (int)M;
  p.N = (int)N;
  p.K = (int)K;
  p.batch = 1;
  p.lda = (int)K;
  p.ldb = (int)K;
  p.strideA = M * K;
  p.strideB = N * K;
  p.strideC = M * N;
  p.alpha = grp.alpha[0];
  p.beta = grp.beta[0];
  p.out_T = (int)T;
  p.out_d = (int)head_dim;
  return launch_gemm_group_s8(p, grp, static_cast<hipStream_t>(stream));
}

int ti_linear_a8_w8_b8_o8_group(const int8_t* x, const int8_t* const* w, const int8_t* const* bias, int8_t* const* out,
                                const float* alpha, const float* beta, int64_t count, int64_t M, int64_t N,
                                int64_t K, void* stream) {
  return linear_group("linear_a8_w8_b8_o8_group", x, w, bias, out, alpha, beta, count, M, N, K, 0, 0, stream);
}

int ti_linear_a8_w8_b8_o8_group_heads(const int8_t* x, const int8_t* const* w, const int8_t* const* bias,
                                      int8_t* const* out, const float* alpha, const float* beta, int64_t count,
                                      int64_t M, int64_t N, int64_t K, int64_t T, int64_t head_dim, void* stream) {
  const char* op = "linear_a8_w8_b8_o8_group_heads";
  g_err[0] = 0;
  if (T <= 0 || head_dim <= 0 || M % T != 0 || N % head_dim != 0 || head_dim % 16 != 0)
    return fail(TI_ERR_INVALID_ARG, "%s: M=%lld must be a multiple of T=%lld, N=%lld of head_dim=%lld, head_dim of 16",
                op, (long long)M, (long long)T, (long long)N, (long long)head_dim);
  return linear_group(op, x, w, bias, out, alpha, beta, count, M, N, K, T, head_dim, stream);
}

int ti_linear_relu_a8_w8_b8_o8(const int8_t* x, const int8_t* w, const int8_t* bias, int8_t* out, int64_t M,
                               int64_t N, int64_t K, float alpha, float beta, void* ws, int64_t ws_bytes,
                               void* stream) {
  return run_gemm("linear_relu_a8_w8_b8_o8", EPI_S8_RELU, x, w, bias, 1, out, 1, 1, M, N, K, alpha, beta, ws,
                  ws_bytes, stream);
}

int ti_bmm_s8t_s8n_f32t(const int8_t* a, const int8_t* b, float* c, int64_t batch, int64_t M, int64_t N,
                        int64_t K, float alpha, void* stream) {
  return run_gemm("bmm_s8t_s8n_f32t", EPI_F32_SCALE, a, b, nullptr, 0, c, 4, batch, M, N, K, alpha, 0.0f,
                  nullptr, 0, stream);
}

int ti_bmm_s8t_s8n_s8t(const int8_t* a, const int8_t* b, int8_t* c, int64_t batch, int64_t M, int64_t N,
                       int64_t K, float alpha, void* stream) {
  return run_gemm("bmm_s8t_s8n_s8t", EPI_S8_SCALE, a, b, nullptr, 0, c, 1, batch, M, N, K, alpha, 0.0f, nullptr,
                  0, stream);
}

int ti_bmm_s8t_s8n_s32t(const int8_t* a, const int8_t* b, int32_t* c, int64_t batch, int64_t M, int64_t N,
                        int64_t K, void* stream) {
  return run_gemm("bmm_s8t_s8n_s32t", EPI_S32_RAW, a, b, nullptr, 0, c, 4, batch, M, N, K, 1.0f, 0.0f, nullptr,
                  0, stream);
}

int64_t ti_bmm_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K) {
  if (batch <= 0 || M <= 0 || N <= 0 || K <= 0) return 0;
  return bmm_workspace_bytes(batch, M, N, K);
}

int ti_bmm_s8t_s8n_f32t_ws(const int8_t* a, const int8_t* b, float* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                           float alpha, void* ws, int64_t ws_bytes, void* stream) {
  return run_gemm("bmm_s8t_s8n_f32t", EPI_F32_SCALE, a, b, nullptr, 0, c, 4, batch, M, N, K, alpha, 0.0f, ws, ws_bytes,
                  stream);
}

int ti_bmm_s8t_s8n_s8t_ws(const int8_t* a, const int8_t* b, int8_t* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                          float alpha, void* ws, int64_t ws_bytes, void* stream) {
  return run_gemm("bmm_s8t_s8n_s8t", EPI_S8_SCALE, a, b, nullptr, 0, c, 1, batch, M, N, K, alpha, 0.0f, ws, ws_bytes,
                  stream);
}

int ti_bmm_s8t_s8n_s32t_ws(const int8_t* a, const int8_t* b, int32_t* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                           void* ws, int64_t ws_bytes, void* stream) {
  return run_gemm("bmm_s8t_s8n_s32t", EPI_S32_RAW, a, b, nullptr, 0, c, 4, batch, M, N, K, 1.0f, 0.0f, ws, ws_bytes,
                  stream);
}

int ti_dq_add_layernorm_q(const int32_t* input, float input_scale, const float* residual, const float* gamma,
                          const float* beta, float eps, float* r_out, int8_t* q_out, int64_t rows, int64_t H,
                          void* stream) {
  g_err[0] = 0;
  const char* op = "dq_add_layernorm_q";
  if (rows < 0 || H < 0) return fail(TI_ERR_INVALID_ARG, "%s: negative size (rows=%lld H=%lld)", op,
                                     (long long)rows, (long long)H);
  if (rows > 0x7fffffffLL || H > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "%s: rows and H must be below 2^31", op);
  const bool nonempty = rows > 0 && H > 0;
  if (int rc = check_ptr(op, "input", input, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "residual", residual, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "gamma", gamma, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "beta", beta, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "residual_out", r_out, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "q_out", q_out, 1, nonempty)) return rc;
  return launch_dq_add_layernorm_q(input, input_scale, residual, gamma, beta, eps, r_out, q_out, rows, H,
                                   static_cast<hipStream_t>(stream));
}

int ti_add_layernorm_q(const float* x, float* residual, const float* gamma, const float* beta, float eps,
                       int8_t* q_out, int64_t rows, int64_t H, void* stream) {
  g_err[0] = 0;
  const char* op = "add_layernorm_q";
  if (rows < 0 || H < 0 || rows > 0x7fffffffLL || H > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "%s: rows and H must be in [0, 2^31) (rows=%lld H=%lld)", op, (long long)rows,
                (long long)H);
  const bool nonempty = rows > 0 && H > 0;
  if (int rc = check_ptr(op, "x", x, 4, nonempty && x != nullptr)) return rc;
  if (int rc = check_ptr(op, "residual", residual, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "gamma", gamma, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "beta", beta, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "q_out", q_out, 1, nonempty)) return rc;
  return launch_add_layernorm_q(x, residual, gamma, beta, eps, q_out, rows, H, static_cast<hipStream_t>(stream));
}

int ti_dq_add_layernorm_q_f16(const int32_t* input, float input_scale, const void* residual, const void* gamma,
                              const void* beta, float eps, void* r_out, int8_t* q_out, int64_t rows, int64_t H,
                              void* stream) {
  g_err[0] = 0;
  const char* op = "dq_add_layernorm_q_f16";
  if (rows < 0 || H < 0 || rows > 0x7fffffffLL || H > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "%s: rows and H must be in [0, 2^31) (rows=%lld H=%lld)", op, (long long)rows,
                (long long)H);
  const bool nonempty = rows > 0 && H > 0;
  if (int rc = check_ptr(op, "input", input, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "residual", residual, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "gamma", gamma, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "beta", beta, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "residual_out", r_out, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "q_out", q_out, 1, nonempty)) return rc;
  return launch_dq_add_layernorm_q_f16(input, input_scale, residual, gamma, beta, eps, r_out, q_out, rows, H,
                                       static_cast<hipStream_t>(stream));
}

int ti_add_layernorm_q_f16(const void* x, void* residual, const void* gamma, const void* beta, float eps, int8_t* q_out,
                           int64_t rows, int64_t H, void* stream) {
  g_err[0] = 0;
  const char* op = "add_layernorm_q_f16";
  if (rows < 0 || H < 0 || rows > 0x7fffffffLL || H > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "%s: rows and H must be in [0, 2^31) (rows=%lld H=%lld)", op, (long long)rows,
                (long long)H);
  const bool nonempty = rows > 0 && H > 0;
  if (int rc = check_ptr(op, "x", x, 2, nonempty && x != nullptr)) return rc;
  if (int rc = check_ptr(op, "residual", residual, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "gamma", gamma, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "beta", beta, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "q_out", q_out, 1, nonempty)) return rc;
  return launch_add_layernorm_q_f16(x, residual, gamma, beta, eps, q_out, rows, H, static_cast<hipStream_t>(stream));
}

int ti_add_f16_xf32(const float* x, void* residual, int64_t n, void* stream) {
  g_err[0] = 0;
  const char* op = "add_f16_xf32";
  if (n < 0) return fail(TI_ERR_INVALID_ARG, "%s: n must not be negative (got %lld)", op, (long long)n);
  if (int rc = check_ptr(op, "x", x, 4, n > 0)) return rc;
  if (int rc = check_ptr(op, "residual", residual, 2, n > 0)) return rc;
  return launch_add_f16_xf32(x, residual, n, static_cast<hipStream_t>(stream));
}

int ti_add_layernorm_q_f16_xf32(const float* x, void* residual, const void* gamma, const void* beta, float eps,
                                int8_t* q_out, int64_t rows, int64_t H, void* stream) {
  g_err[0] = 0;
  const char* op = "add_layernorm_q_f16_xf32";
  if (rows < 0 || H < 0 || rows > 0x7fffffffLL || H > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "%s: rows and H must be in [0, 2^31) (rows=%lld H=%lld)", op, (long long)rows,
                (long long)H);
  const bool nonempty = rows > 0 && H > 0;
  if (int rc = check_ptr(op, "x", x, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "residual", residual, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "gamma", gamma, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "beta", beta, 2, nonempty)) return rc;
  if (int rc = check_ptr(op, "q_out", q_out, 1, nonempty)) return rc;
  return launch_add_layernorm_q_f16_xf32(x, residual, gamma, beta, eps, q_out, rows, H, static_cast<hipStream_t>(stream));
}

int ti_attn_softmax_q(const float* scores, const float* mask, int8_t* probs, int64_t batch, int64_t heads, int64_t T,
                      int64_t S, void* stream) {
  g_err[0] = 0;
  const char* op = "attn_softmax_q";
  if (batch < 0 || heads < 0 || T < 0 || S < 0 || T > 0x7fffffffLL || S > 0x7fffffffLL || heads > 0x7fffffffLL ||
      batch > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31)", op);
  const bool nonempty = batch > 0 && heads > 0 && T > 0 && S > 0;
  if (int rc = check_ptr(op, "scores", scores, 4, nonempty)) return rc;
  if (int rc = check_ptr(op, "mask", mask, 4, nonempty && mask != nullptr)) return rc;
  if (int rc = check_ptr(op, "probs", probs, 1, nonempty)) return rc;
  return launch_attn_softmax_q(scores, mask, probs, batch, heads, T, S, static_cast<hipStream_t>(stream));
}

const char* ti_last_kernel(void) { return last_gemm_kernel(); }

int ti_fused_splitk(int enable) { return set_fused_split(enable); }
int ti_fused_splitk_faulted(void) { return fused_split_faulted(); }
int ti_selftest_fused_flag_action(int state, int flag, int enabled, int64_t counters, int64_t max_counters) {
  return fused_flag_action(state, flag, enabled != 0, counters, max_counters);
}
int ti_selftest_fused_slot(int64_t* table, uint32_t* live_mask, int cap, int64_t stream, uint32_t busy_mask,
                           int* fresh) {
  static_assert(sizeof(long long) == sizeof(int64_t) && sizeof(unsigned) == sizeof(uint32_t), "plain forwards");
  return fused_slot_for_test(reinterpret_cast<long long*>(table), reinterpret_cast<unsigned*>(live_mask), cap, stream,
                             busy_mask, fresh);
}

int64_t ti_diag_mfma_loop_ops(int64_t iters) { return iters > 0 ? diag_mfma_loop_ops(iters) : 0; }

int ti_diag_mfma_loop(int mode, const int8_t* data, int64_t data_bytes, int64_t iters, int32_t* sink, void* stream) {
  g_err[0] = 0;
  const char* op = "diag_mfma_loop";
  if (iters < 2 || iters > (1 << 30) || (iters & 1))
    return fail(TI_ERR_INVALID_ARG, "%s: iters must be even, in [2, 2^30] (got %lld)", op, (long long)iters);
  if (data_bytes < (1 << 20))
    return fail(TI_ERR_INVALID_ARG, "%s: data must hold at least 1 MiB (got %lld bytes)", op, (long long)data_bytes);
  if (int rc = check_ptr(op, "data", data, 16, true)) return rc;
  if (int rc = check_ptr(op, "sink", sink, 4, true)) return rc;
  return launch_diag_mfma_loop(mode, data, iters, sink, static_cast<hipStream_t>(stream));
}

int ti_diag_store_loop(float* out, int64_t M, int64_t N, int workgroups, int reps, void* stream) {
  g_err[0] = 0;
  const char* op = "diag_store_loop";
  if (M < 256 || N < 160 || M % 256 != 0 || N % 160 != 0 || M * N > (1ll << 31))
    return fail(TI_ERR_INVALID_ARG, "%s: M must be a multiple of 256, N of 160, M * N at most 2^31 (got %lld x %lld)", op,
                (long long)M, (long long)N);
  if (workgroups < 1 || workgroups > 65536 || reps < 1 || reps > 65536)
    return fail(TI_ERR_INVALID_ARG, "%s: workgroups and reps must be in [1, 65536] (got %d, %d)", op, workgroups, reps);
  if (int rc = check_ptr(op, "out", out, 16, true)) return rc;
  return launch_diag_store_loop(out, M, N, workgroups, reps, static_cast<hipStream_t>(stream));
}

int64_t ti_diag_copy_loop_bytes(int64_t iters) { return iters > 0 ? diag_copy_loop_bytes(iters) : 0; }

int ti_diag_copy_loop(int mode, const int8_t* data, int64_t data_bytes, int64_t iters, int32_t* sink, void* stream) {
  g_err[0] = 0;
  const char* op = "diag_copy_loop";
  if (iters < 1 || iters > (1 << 30))
    return fail(TI_ERR_INVALID_ARG, "%s: iters must be in [1, 2^30] (got %lld)", op, (long long)iters);
  if (data_bytes < (2 << 20))
    return fail(TI_ERR_INVALID_ARG, "%s: data must hold at least 2 MiB (got %lld bytes)", op, (long long)data_bytes);
  if (int rc = check_ptr(op, "data", data, 16, true)) return rc;
  if (int rc = check_ptr(op, "sink", sink, 4, true)) return rc;
  return launch_diag_copy_loop(mode, data, iters, sink, static_cast<hipStream_t>(stream));
}

int ti_diag_read_loop(int mode, const int8_t* data, int64_t N, int64_t K, int32_t* sink, void* stream) {
  g_err[0] = 0;
  const char* op = "diag_read_loop";
  if (int rc = check_ptr(op, "data", data, 16, true)) return rc;
  if (int rc = check_ptr(op, "sink", sink, 4, true)) return rc;
  return launch_diag_read_loop(mode, data, N, K, sink, static_cast<hipStream_t>(stream));
}

int64_t ti_diag_mix_loop_ops(int shape, int64_t iters) { return iters > 0 ? diag_mix_loop_ops(shape, iters) : 0; }

int ti_diag_mix_loop(int shape, int parts, const int8_t* data, int64_t data_bytes, int64_t iters, int32_t* sink,
                     void* stream) {
  g_err[0] = 0;
  const char* op = "diag_mix_loop";
  if (iters < 1 || iters > (1 << 30))
    return fail(TI_ERR_INVALID_ARG, "%s: iters must be in [1, 2^30] (got %lld)", op, (long long)iters);
  if (data_bytes < (3 << 20))
    return fail(TI_ERR_INVALID_ARG, "%s: data must hold at least 3 MiB (got %lld bytes)", op, (long long)data_bytes);
  if (int rc = check_ptr(op, "data", data, 16, true)) return rc;
  if (int rc = check_ptr(op, "sink", sink, 4, true)) return rc;
  return launch_diag_mix_loop(shape, parts, data, iters, sink, static_cast<hipStream_t>(stream));
}

int ti_bmm_s8t_s8n_f32t_strided(const int8_t* a, const int8_t* b, float* c, int64_t batch, int64_t M, int64_t N,
                                int64_t K, int64_t stride_a, int64_t stride_b, float alpha, void* stream) {
  return run_gemm("bmm_s8t_s8n_f32t_strided", EPI_F32_SCALE, a, b, nullptr, 0, c, 4, batch, M, N, K, alpha, 0.0f,
                  nullptr, 0, stream, stride_a, stride_b);
}

int ti_bmm_s8t_s8t_s8t(const int8_t* a, const int8_t* b, int8_t* c, int64_t batch, int64_t M, int64_t N, int64_t K,
                       int64_t stride_b, float alpha, void* stream) {
  g_err[0] = 0;
  const char* op = "bmm_s8t_s8t_s8t";
  if (int rc = check_dims(op, batch, M, N, K)) return rc;
  if (stride_b == 0) stride_b = K * N;
  if (stride_b < K * N)
    return fail(TI_ERR_INVALID_ARG, "%s: batch stride %lld is smaller than one K x N matrix (%lld)", op,
                (long long)stride_b, (long long)(K * N));
  const bool nonempty = batch > 0 && M > 0 && N > 0;
  if (int rc = check_ptr(op, "a", a, 1, nonempty && K > 0)) return rc;
  if (int rc = check_ptr(op, "b", b, 1, nonempty && K > 0)) return rc;
  if (int rc = check_ptr(op, "c", c, 1, nonempty)) return rc;
  return launch_bmm_s8t_s8t_s8t(a, b, c, batch, M, N, K, stride_b, alpha, static_cast<hipStream_t>(stream));
}

int ti_permute_0213_s8(const int8_t* src, int8_t* dst, int64_t B, int64_t X, int64_t Y, int64_t D, void* stream) {
  g_err[0] = 0;
  const char* op = "permute_0213_s8";
  const int64_t lim = 0x7fffffffLL;
  if (B < 0 || X < 0 || Y < 0 || D < 0 || X > lim || Y > lim || D > lim || B > lim)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31)", op);
  const bool nonempty = B > 0 && X > 0 && Y > 0 && D > 0;
  if (int rc = check_ptr(op, "src", src, 1, nonempty)) return rc;
  if (int rc = check_ptr(op, "dst", dst, 1, nonempty)) return rc;
  return launch_permute_0213_s8(src, dst, B, X, Y, D, static_cast<hipStream_t>(stream));
}

int ti_kv_append_s8(const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf, int64_t BH, int64_t T,
                    int64_t D, int64_t cap, int64_t S, void* stream) {
  g_err[0] = 0;
  const char* op = "kv_append_s8";
  const int64_t lim = 0x7fffffffLL;
  if (BH < 0 || T < 0 || D < 0 || cap < 0 || S < 0 || BH > lim || T > lim || D > lim || cap > lim)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31)", op);
  if (S + T > cap) return fail(TI_ERR_INVALID_ARG, "%s: %lld + %lld positions do not fit a capacity of %lld", op,
                               (long long)S, (long long)T, (long long)cap);
  const bool nonempty = BH > 0 && T > 0 && D > 0;
  if (int rc = check_ptr(op, "k_new", k_new, 1, nonempty)) return rc;
  if (int rc = check_ptr(op, "v_new", v_new, 1, nonempty)) return rc;
  if (int rc = check_ptr(op, "k_buf", k_buf, 1, nonempty)) return rc;
  if (int rc = check_ptr(op, "v_buf", v_buf, 1, nonempty)) return rc;
  return launch_kv_append_s8(k_new, v_new, k_buf, v_buf, BH, T, D, cap, S, static_cast<hipStream_t>(stream));
}

int ti_attn_qk_softmax_q_supported(int64_t T, int64_t S, int64_t D) {
  return attn_qk_softmax_q_supported(T, S, D) ? 1 : 0;
}
int ti_attn_prefill_supported(int64_t T, int64_t S, int64_t D) { return attn_prefill_supported(T, S, D) ? 1 : 0; }

int64_t ti_attn_mask_classes_bytes(int64_t batch, int64_t T, int64_t S) { return attn_mask_classes_bytes(batch, T, S); }

int ti_attn_mask_classes(const float* mask, uint8_t* classes, int64_t batch, int64_t T, int64_t S, void* stream) {
  g_err[0] = 0;
  const char* op = "attn_mask_classes";
  if (batch < 0 || T < 0 || S < 0) return fail(TI_ERR_INVALID_ARG, "%s: negative size", op);
  if (batch == 0 || T == 0) return TI_OK;
  if (int rc = check_ptr(op, "mask", mask, 16, true)) return rc;
  if (int rc = check_ptr(op, "classes", classes, 1, true)) return rc;
  return launch_attn_mask_classes(mask, classes, batch, T, S, static_cast<hipStream_t>(stream));
}

int ti_attn_qk_softmax_q(const int8_t* q, const int8_t* k, const float* mask, int8_t* probs, int64_t BH, int64_t T,
                         int64_t S, int64_t D, int64_t stride_q, int64_t stride_k, int64_t heads, float alpha,
                         void* stream) {
  return ti_attn_qk_softmax_q_mc(q, k, mask, nullptr, probs, BH, T, S, D, stride_q, stride_k, heads, alpha, stream);
}

int ti_attn_qk_softmax_q_mc(const int8_t* q, const int8_t* k, const float* mask, const uint8_t* mask_classes,
                            int8_t* probs, int64_t BH, int64_t T, int64_t S, int64_t D, int64_t stride_q,
                            int64_t stride_k, int64_t heads, float alpha, void* stream) {
  g_err[0] = 0;
  const char* op = "attn_qk_softmax_q";
  const int64_t lim = 0x7fffffffLL;
  if (BH < 0 || T < 0 || S < 0 || D < 0 || heads < 1 || BH > lim || T > lim || heads > lim)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31) and heads >= 1", op);
  if (BH % heads != 0) return fail(TI_ERR_INVALID_ARG, "%s: BH = %lld is not a multiple of heads = %lld", op,
                                   (long long)BH, (long long)heads);
  if (BH == 0 || T == 0) return TI_OK;
  if (!attn_qk_softmax_q_supported(T, S, D))
    return fail(TI_ERR_INVALID_ARG, "%s: unsupported shape T=%lld S=%lld head_dim=%lld (needs S a multiple of 16 in "
                "[16, 4096] and head_dim a multiple of 16 up to 128)", op,
                (long long)T, (long long)S, (long long)D);
  if (stride_q < T * D || stride_k < S * D || stride_q % 16 != 0 || stride_k % 16 != 0)
    return fail(TI_ERR_INVALID_ARG, "%s: batch strides (%lld, %lld) must be multiples of 16 and cover one matrix", op,
                (long long)stride_q, (long long)stride_k);
  if (int rc = check_ptr(op, "q", q, 16, true)) return rc;
  if (int rc = check_ptr(op, "k", k, 16, true)) return rc;
  if (int rc = check_ptr(op, "mask", mask, 16, mask != nullptr)) return rc;
  if (int rc = check_ptr(op, "probs", probs, 16, true)) return rc;
  return launch_attn_qk_softmax_q(q, k, mask, probs, BH, T, S, D, stride_q, stride_k, heads, alpha, nullptr, nullptr,
                                  0.0f, static_cast<hipStream_t>(stream), mask_classes);
}

int ti_attn_prefill_s8(const int8_t* q, const int8_t* k, const int8_t* vt, const float* mask, int8_t* ctx, int64_t BH,
                       int64_t T, int64_t S, int64_t D, int64_t stride_q, int64_t stride_k, int64_t heads,
                       float alpha_qk, float alpha_pv, void* stream) {
  return ti_attn_prefill_s8_mc(q, k, vt, mask, nullptr, ctx, BH, T, S, D, stride_q, stride_k, heads, alpha_qk, alpha_pv,
                               stream);
}

int ti_attn_prefill_s8_mc(const int8_t* q, const int8_t* k, const int8_t* vt, const float* mask,
                          const uint8_t* mask_classes, int8_t* ctx, int64_t BH, int64_t T, int64_t S, int64_t D,
                          int64_t stride_q, int64_t stride_k, int64_t heads, float alpha_qk, float alpha_pv, void* stream) {
  g_err[0] = 0;
  const char* op = "attn_prefill_s8";
  const int64_t lim = 0x7fffffffLL;
  if (BH < 0 || T < 0 || S < 0 || D < 0 || heads < 1 || BH > lim || T > lim || heads > lim)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31) and heads >= 1", op);
  if (BH % heads != 0) return fail(TI_ERR_INVALID_ARG, "%s: BH = %lld is not a multiple of heads = %lld", op,
                                   (long long)BH, (long long)heads);
  if (BH == 0 || T == 0) return TI_OK;
  if (!attn_prefill_supported(T, S, D))
    return fail(TI_ERR_INVALID_ARG, "%s: unsupported shape T=%lld S=%lld head_dim=%lld (needs S a multiple of 16 in "
                "[16, 4096] and head_dim a multiple of 16 up to 128)",
                op, (long long)T, (long long)S, (long long)D);
  if (stride_q < T * D || stride_k < S * D || stride_q % 16 != 0 || stride_k % 16 != 0)
    return fail(TI_ERR_INVALID_ARG, "%s: batch strides (%lld, %lld) must be multiples of 16 and cover one matrix", op,
                (long long)stride_q, (long long)stride_k);
  if (int rc = check_ptr(op, "q", q, 16, true)) return rc;
  if (int rc = check_ptr(op, "k", k, 16, true)) return rc;
  if (int rc = check_ptr(op, "vt", vt, 16, true)) return rc;
  if (int rc = check_ptr(op, "mask", mask, 16, mask != nullptr)) return rc;
  if (int rc = check_ptr(op, "ctx", ctx, 4, true)) return rc;
  return launch_attn_qk_softmax_q(q, k, mask, nullptr, BH, T, S, D, stride_q, stride_k, heads, alpha_qk, vt, ctx,
                                  alpha_pv, static_cast<hipStream_t>(stream), mask_classes);
}

int ti_decode_attn_supported(int64_t T, int64_t S, int64_t D) { return decode_attn_supported(T, S, D) ? 1 : 0; }

int ti_decode_attn_s8(const int8_t* q, const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf,
                      const float* mask, int8_t* ctx, int8_t* probs_out, int64_t BH, int64_t T, int64_t D, int64_t cap,
                      int64_t S, int64_t heads, float alpha_qk, float alpha_pv, void* stream) {
  g_err[0] = 0;
  const char* op = "decode_attn_s8";
  const int64_t lim = 0x7fffffffLL;
  if (BH < 0 || T < 0 || D < 0 || cap < 0 || S < 0 || heads < 1 || BH > lim || cap > lim || heads > lim)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31) and heads >= 1", op);
  if (BH % heads != 0) return fail(TI_ERR_INVALID_ARG, "%s: BH = %lld is not a multiple of heads = %lld", op,
                                   (long long)BH, (long long)heads);
  if ((k_new == nullptr) != (v_new == nullptr))
    return fail(TI_ERR_INVALID_ARG, "%s: k_new and v_new must both be given or both be NULL", op);
  if (S > cap) return fail(TI_ERR_INVALID_ARG, "%s: %lld positions do not fit a capacity of %lld", op, (long long)S,
                           (long long)cap);
  if (k_new != nullptr && S < T)
    return fail(TI_ERR_INVALID_ARG, "%s: S = %lld counts the %lld appended positions", op, (long long)S, (long long)T);
  if (BH == 0) return TI_OK;
  if (!decode_attn_supported(T, S, D))
    return fail(TI_ERR_INVALID_ARG, "%s: unsupported shape T=%lld S=%lld head_dim=%lld (needs 1 <= T <= 4, head_dim a multiple of 16 up "
                "to 128, S >= 1 and scores that fit the LDS)", op, (long long)T, (long long)S, (long long)D);
  if (int rc = check_ptr(op, "q", q, 16, true)) return rc;
  if (int rc = check_ptr(op, "k_new", k_new, 16, k_new != nullptr)) return rc;
  if (int rc = check_ptr(op, "v_new", v_new, 16, v_new != nullptr)) return rc;
  if (int rc = check_ptr(op, "k_buf", k_buf, 16, true)) return rc;
  if (int rc = check_ptr(op, "v_buf", v_buf, 16, true)) return rc;
  if (int rc = check_ptr(op, "mask", mask, 4, mask != nullptr)) return rc;
  if (int rc = check_ptr(op, "ctx", ctx, 1, true)) return rc;
  return launch_decode_attn_s8(q, k_new, v_new, k_buf, v_buf, mask, ctx, probs_out, BH, T, D, cap, S, heads, alpha_qk,
                               alpha_pv, static_cast<hipStream_t>(stream));
}

int ti_decode_attn_s8_devlen(const int8_t* q, const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf,
                             int8_t* ctx, int64_t BH, int64_t T, int64_t D, int64_t cap, int64_t S_max,
                             const int32_t* s_dev, int64_t heads, float alpha_qk, float alpha_pv, void* stream) {
  g_err[0] = 0;
  const char* op = "decode_attn_s8_devlen";
  const int64_t lim = 0x7fffffffLL;
  if (BH < 0 || T < 0 || D < 0 || cap < 0 || S_max < 0 || heads < 1 || BH > lim || cap > lim || heads > lim)
    return fail(TI_ERR_INVALID_ARG, "%s: sizes must be in [0, 2^31) and heads >= 1", op);
  if (BH % heads != 0) return fail(TI_ERR_INVALID_ARG, "%s: BH = %lld is not a multiple of heads = %lld", op,
                                   (long long)BH, (long long)heads);
  if (k_new == nullptr || v_new == nullptr)
    return fail(TI_ERR_INVALID_ARG, "%s: k_new and v_new must be given", op);
  if (S_max > cap) return fail(TI_ERR_INVALID_ARG, "%s: %lld positions do not fit a capacity of %lld", op,
                               (long long)S_max, (long long)cap);
  if (S_max < T) return fail(TI_ERR_INVALID_ARG, "%s: S_max = %lld counts the %lld appended positions", op,
                             (long long)S_max, (long long)T);
  if (BH == 0) return TI_OK;
  if (!decode_attn_supported(T, S_max, D))
    return fail(TI_ERR_INVALID_ARG, "%s: unsupported shape T=%lld S_max=%lld head_dim=%lld (needs 1 <= T <= 4, head_dim a multiple of 16 "
                "up to 128 and scores that fit the LDS)", op, (long long)T, (long long)S_max, (long long)D);
  if (int rc = check_ptr(op, "q", q, 16, true)) return rc;
  if (int rc = check_ptr(op, "k_new", k_new, 16, true)) return rc;
  if (int rc = check_ptr(op, "v_new", v_new, 16, true)) return rc;
  if (int rc = check_ptr(op, "k_buf", k_buf, 16, true)) return rc;
  if (int rc = check_ptr(op, "v_buf", v_buf, 16, true)) return rc;
  if (int rc = check_ptr(op, "ctx", ctx, 1, true)) return rc;
  if (int rc = check_ptr(op, "s_dev", s_dev, 4, true)) return rc;
  return launch_decode_attn_s8(q, k_new, v_new, k_buf, v_buf, nullptr, ctx, nullptr, BH, T, D, cap, S_max, heads,
                               alpha_qk, alpha_pv, static_cast<hipStream_t>(stream), s_dev);
}

int ti_transpose_last2_s8(const int8_t* src, int8_t* dst, int64_t B, int64_t R, int64_t C, void* stream) {
  g_err[0] = 0;
  const char* op = "transpose_last2_s8";
  const int64_t lim = 0x7fffffffLL;
  if (B < 0 || R < 0 || C < 0 || R > lim || C > lim || B > 65535 || (R + 63) / 64 > 65535)
    return fail(TI_ERR_INVALID_ARG, "%s: needs 0 <= B <= 65535, R < 2^22, C < 2^31", op);
  const bool nonempty = B > 0 && R > 0 && C > 0;
  if (int rc = check_ptr(op, "src", src, 1, nonempty)) return rc;
  if (int rc = check_ptr(op, "dst", dst, 1, nonempty)) return rc;
  return launch_transpose_last2_s8(src, dst, B, R, C, static_cast<hipStream_t>(stream));
}

// One decoder layer of a decode step: the seven (fp16 stream: eight) calls an Int8OPTDecoderLayer makes for one new
// token per sequence, issued from one C call.  Each step IS the public entry point the Python modules call, with
// the arguments they pass, so the values are theirs.
int64_t ti_opt_decoder_layer_decode_scratch_bytes(int64_t B, int64_t embed, int64_t ffn) {
  if (B <= 0 || embed <= 0 || ffn <= 0) return 0;
  auto up = [](int64_t n) { return (n + 255) / 256 * 256; };
  return 5 * up(B * embed) + up(4 * B * embed) + up(B * ffn);
}

int ti_opt_decoder_layer_decode(const TiOptDecodeLayer* L, void* hidden, const float* mask, int8_t* k_buf, int8_t* v_buf,
                                int64_t B, int64_t cap, int64_t S, void* scratch, int64_t scratch_bytes, void* stream) {
  g_err[0] = 0;
  const char* op = "opt_decoder_layer_decode";
  if (L == nullptr) return fail(TI_ERR_INVALID_ARG, "%s: no layer description", op);
  const int64_t E = L->embed, H = L->heads, d = L->head_dim, F = L->ffn;
  if (E <= 0 || H <= 0 || d <= 0 || F <= 0 || H * d != E)
    return fail(TI_ERR_INVALID_ARG, "%s: needs embed = heads * head_dim > 0 and ffn > 0 (got %lld, %lld x %lld, %lld)", op,
                (long long)E, (long long)H, (long long)d, (long long)F);
  if (B < 0 || B > 16) return fail(TI_ERR_INVALID_ARG, "%s: 0 to 16 sequences, one new token each (got %lld)", op, (long long)B);
  if (B == 0) return TI_OK;
  if (int rc = check_ptr(op, "hidden", hidden, L->half ? 2 : 4, true)) return rc;
  if (int rc = check_ptr(op, "scratch", scratch, 256, true)) return rc;
  if (scratch_bytes < ti_opt_decoder_layer_decode_scratch_bytes(B, E, F))
    return fail(TI_ERR_INVALID_ARG, "%s: scratch of %lld bytes, needs %lld", op, (long long)scratch_bytes,
                (long long)ti_opt_decoder_layer_decode_scratch_bytes(B, E, F));
  auto up = [](int64_t n) { return (n + 255) / 256 * 256; };
  char* at = static_cast<char*>(scratch);
  auto take = [&](int64_t bytes) {
    char* r = at;
    at += up(bytes);
    return r;
  };
  int8_t* x = reinterpret_cast<int8_t*>(take(B * E));      // LayerNorm-quantised input of the projections, then of fc1
  int8_t* q = reinterpret_cast<int8_t*>(take(B * E));
  int8_t* k = reinterpret_cast<int8_t*>(take(B * E));
  int8_t* v = reinterpret_cast<int8_t*>(take(B * E));
  int8_t* ctx = reinterpret_cast<int8_t*>(take(B * E));
  float* f32 = reinterpret_cast<float*>(take(4 * B * E));   // output of out_proj, then (fp16 stream) of fc2
  int8_t* h = reinterpret_cast<int8_t*>(take(B * F));
  int rc;
  // self_attn_layer_norm
  rc = L->half ? ti_add_layernorm_q_f16(nullptr, hidden, L->ln1_gamma, L->ln1_beta, L->ln1_eps, x, B, E, stream)
               : ti_add_layernorm_q(nullptr, static_cast<float*>(hidden), static_cast<const float*>(L->ln1_gamma),
                                    static_cast<const float*>(L->ln1_beta), L->ln1_eps, x, B, E, stream);
  if (rc) return rc;
  // q, k, v projections
  const int8_t* w3[3] = {L->wq, L->wk, L->wv};
  const int8_t* b3[3] = {L->bq, L->bk, L->bv};
  int8_t* o3[3] = {q, k, v};
  const float a3[3] = {L->alpha_q, L->alpha_k, L->alpha_v};
  const float be3[3] = {L->beta_q, L->beta_k, L->beta_v};
  if ((rc = ti_linear_a8_w8_b8_o8_group(x, w3, b3, o3, a3, be3, 3, B, E, E, stream))) return rc;
  // cache append + attention; [B, 1, E] rows are [B * heads, 1, head_dim] as they lie
  if ((rc = ti_decode_attn_s8(q, k, v, k_buf, v_buf, mask, ctx, nullptr, B * H, 1, d, cap, S, H, L->alpha_qk, L->alpha_pv,
                              stream)))
    return rc;
  // out_proj, then the residual update fused with final_layer_norm
  if ((rc = ti_linear_a8_w8_bfp32_ofp32(ctx, L->wo, L->bo, f32, B, E, E, L->alpha_o, 1.0f, nullptr, 0, stream))) return rc;
  rc = L->half ? ti_add_layernorm_q_f16_xf32(f32, hidden, L->ln2_gamma, L->ln2_beta, L->ln2_eps, x, B, E, stream)
               : ti_add_layernorm_q(f32, static_cast<float*>(hidden), static_cast<const float*>(L->ln2_gamma),
                                    static_cast<const float*>(L->ln2_beta), L->ln2_eps, x, B, E, stream);
  if (rc) return rc;
  // fc1 (ReLU), fc2 added into the residual stream
  if ((rc = ti_linear_relu_a8_w8_b8_o8(x, L->w1, L->b1, h, B, F, E, L->alpha_1, L->beta_1, nullptr, 0, stream))) return rc;
  if (L->half) {
    if ((rc = ti_linear_a8_w8_bfp32_ofp32(h, L->w2, L->b2, f32, B, E, F, L->alpha_2, 1.0f, nullptr, 0, stream))) return rc;
    return ti_add_f16_xf32(f32, hidden, B * E, stream);
  }
  return ti_linear_a8_w8_bfp32_ofp32_acc(h, L->w2, L->b2, static_cast<float*>(hidden), B, E, F, L->alpha_2, 1.0f, nullptr, 0,
                                         stream);
}

// One decoder layer of a prefill (no cache yet): the launches an Int8OPTDecoderLayer makes for T > 16 tokens per
// sequence when its attention takes the one-launch prefill kernel, issued from one C call through the public entry
// points, with the arguments the modules pass.
int64_t ti_opt_decoder_layer_prefill_scratch_bytes(int64_t rows, int64_t embed, int64_t ffn) {
  if (rows <= 0 || embed <= 0 || ffn <= 0) return 0;
  auto up = [](int64_t n) { return (n + 255) / 256 * 256; };
  return 4 * up(rows * embed) + up(4 * rows * embed) + up(rows * ffn);
}

int ti_opt_decoder_layer_prefill(const TiOptDecodeLayer* L, void* hidden, const float* mask, const uint8_t* mask_classes,
                                 int8_t* k_out, int8_t* v_out, int64_t B, int64_t T, void* scratch, int64_t scratch_bytes,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
  g_err[0] = 0;
  const char* op = "opt_decoder_layer_prefill";
  if (L == nullptr) return fail(TI_ERR_INVALID_ARG, "%s: no layer description", op);
  const int64_t E = L->embed, H = L->heads, d = L->head_dim, F = L->ffn;
  if (E <= 0 || H <= 0 || d <= 0 || F <= 0 || H * d != E)
    return fail(TI_ERR_INVALID_ARG, "%s: needs embed = heads * head_dim > 0 and ffn > 0 (got %lld, %lld x %lld, %lld)", op,
                (long long)E, (long long)H, (long long)d, (long long)F);
  if (B < 0 || T < 0 || B > 65535 || T > 4096) return fail(TI_ERR_INVALID_ARG, "%s: needs 0 <= B <= 65535, 0 <= T <= 4096", op);
  const int64_t M = B * T;
  if (M == 0) return TI_OK;
  if (M > 4096) return fail(TI_ERR_INVALID_ARG, "%s: up to 4096 tokens in all (got %lld x %lld)", op, (long long)B, (long long)T);
  if (!attn_prefill_supported(T, T, d))
    return fail(TI_ERR_INVALID_ARG, "%s: %lld tokens per sequence at head size %lld: needs a multiple of 16 up to 4096 and a "
                "head size that is a multiple of 16 up to 128", op, (long long)T, (long long)d);
  if (int rc = check_ptr(op, "hidden", hidden, L->half ? 2 : 4, true)) return rc;
  if (int rc = check_ptr(op, "k_out", k_out, 16, true)) return rc;
  if (int rc = check_ptr(op, "v_out", v_out, 16, true)) return rc;
  if (int rc = check_ptr(op, "scratch", scratch, 256, true)) return rc;
  if (scratch_bytes < ti_opt_decoder_layer_prefill_scratch_bytes(M, E, F))
    return fail(TI_ERR_INVALID_ARG, "%s: scratch of %lld bytes, needs %lld", op, (long long)scratch_bytes,
                (long long)ti_opt_decoder_layer_prefill_scratch_bytes(M, E, F));
  auto up = [](int64_t n) { return (n + 255) / 256 * 256; };
  char* at = static_cast<char*>(scratch);
  auto take = [&](int64_t bytes) {
    char* r = at;
    at += up(bytes);
    return r;
  };
  int8_t* x = reinterpret_cast<int8_t*>(take(M * E));     // LayerNorm-quantised input of the projections, then of fc1
  int8_t* q = reinterpret_cast<int8_t*>(take(M * E));     // [B, heads, T, head_dim]
  int8_t* vt = reinterpret_cast<int8_t*>(take(M * E));    // [B * heads, head_dim, T]
  int8_t* ctx = reinterpret_cast<int8_t*>(take(M * E));   // [B, T, embed]
  float* f32 = reinterpret_cast<float*>(take(4 * M * E)); // output of out_proj, then (fp16 stream) of fc2
  int8_t* h = reinterpret_cast<int8_t*>(take(M * F));
  int rc;
  rc = L->half ? ti_add_layernorm_q_f16(nullptr, hidden, L->ln1_gamma, L->ln1_beta, L->ln1_eps, x, M, E, stream)
               : ti_add_layernorm_q(nullptr, static_cast<float*>(hidden), static_cast<const float*>(L->ln1_gamma),
                                    static_cast<const float*>(L->ln1_beta), L->ln1_eps, x, M, E, stream);
  if (rc) return rc;
  // q, k, v stored head-major by the projections themselves: one grouped launch where the library has one, else one
  // call per projection with the split-K workspace (the choice the attention module makes)
  const int8_t* w3[3] = {L->wq, L->wk, L->wv};
  const int8_t* b3[3] = {L->bq, L->bk, L->bv};
  int8_t* o3[3] = {q, k_out, v_out};
  const float a3[3] = {L->alpha_q, L->alpha_k, L->alpha_v};
  const float be3[3] = {L->beta_q, L->beta_k, L->beta_v};
  if (ti_linear_group_is_one_launch(M, E, E, 3)) {
    if ((rc = ti_linear_a8_w8_b8_o8_group_heads(x, w3, b3, o3, a3, be3, 3, M, E, E, T, d, stream))) return rc;
  } else {
    for (int i = 0; i < 3; ++i)
      if ((rc = ti_linear_a8_w8_b8_o8_heads(x, w3[i], b3[i], o3[i], M, E, E, a3[i], be3[i], T, d, workspace,
                                             workspace_bytes, stream)))
        return rc;
  }
  // V transposed, then the whole attention with the head merge
  if ((rc = ti_transpose_last2_s8(v_out, vt, B * H, T, d, stream))) return rc;
  if ((rc = ti_attn_prefill_s8_mc(q, k_out, vt, mask, mask_classes, ctx, B * H, T, T, d, T * d, T * d, H, L->alpha_qk,
                                  L->alpha_pv, stream)))
    return rc;
  if ((rc = ti_linear_a8_w8_bfp32_ofp32(ctx, L->wo, L->bo, f32, M, E, E, L->alpha_o, 1.0f, workspace, workspace_bytes,
                                        stream)))
    return rc;
  rc = L->half ? ti_add_layernorm_q_f16_xf32(f32, hidden, L->ln2_gamma, L->ln2_beta, L->ln2_eps, x, M, E, stream)
               : ti_add_layernorm_q(f32, static_cast<float*>(hidden), static_cast<const float*>(L->ln2_gamma),
                                    static_cast<const float*>(L->ln2_beta), L->ln2_eps, x, M, E, stream);
  if (rc) return rc;
  if ((rc = ti_linear_relu_a8_w8_b8_o8(x, L->w1, L->b1, h, M, F, E, L->alpha_1, L->beta_1, workspace, workspace_bytes,
                                       stream)))
    return rc;
  if (L->half) {
    if ((rc = ti_linear_a8_w8_bfp32_ofp32(h, L->w2, L->b2, f32, M, E, F, L->alpha_2, 1.0f, workspace, workspace_bytes,
                                          stream)))
      return rc;
    return ti_add_f16_xf32(f32, hidden, M * E, stream);
  }
  return ti_linear_a8_w8_bfp32_ofp32_acc(h, L->w2, L->b2, static_cast<float*>(hidden), M, E, F, L->alpha_2, 1.0f, workspace,
                                         workspace_bytes, stream);
}

}  // extern "C"

// Host-side entry of the INT8 GEMM family: dispatch over the epilogue kinds (each kind's kernels are
// compiled in a translation unit of their own, gemm_s8_kinds.hip with -DTI_KIND=n), the grouped q/k/v
// launches, the split-K slice GEMM and the workspace query.
#include "gemm_s8_impl.h"

namespace ti {

long long gemm_workspace_bytes(long long M, long long N, long long K) {
  const int s = choose_splits(M, N, K);
  return s > 1 ? (long long)s * M * N * 4 : 0;
}

// one per epilogue kind (EpiKind value n), each in its own translation unit
int launch_gemm_kind_0(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_1(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_2(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_3(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_4(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_5(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_6(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_7(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);
int launch_gemm_kind_8(const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream);

thread_local const char* g_last_kernel = "";
const char* last_gemm_kernel() { return g_last_kernel; }

int launch_splitk_raw(int tile, const GemmParams& q, hipStream_t stream) {
  if (tile == SPLIT_128) return launch_pipe<PipeCfg<128, 128, 2, 2, 4, EPI_S32_RAW, false>>(q, stream);
  if (tile == SPLIT_256x160) return launch_pipe16q<Pipe16QCfg<256, 160, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x80) return launch_pipe16q<Pipe16QCfg<128, 80, 4, 1, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x160) return launch_pipe16q<Pipe16QCfg<128, 160, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x288) return launch_pipe16q<Pipe16QCfg<128, 288, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_256x288) return launch_pipe16q<Pipe16QCfg<256, 288, 4, 2, EPI_S32_RAW>>(q, stream);
  if (q.K % QBK == 0) return launch_pipe2<Pipe2Cfg<256, 256, 2, 4, EPI_S32_RAW, false>>(q, stream);
  return launch_pipe<PipeCfg<256, 256, 2, 4, 4, EPI_S32_RAW, false>>(q, stream);
}

// q/k/v-style group of s8 linears.  Decode shapes (M <= 16, K % 1024 == 0, enough strips) take one launch
// of the streaming kernel over all the weights; anything else runs problem by problem.
int launch_gemm_group_s8(const GemmParams& shape, const GemmGroup& grp, hipStream_t stream) {
  constexpr int KIND = EPI_S8_BIAS;
  if (shape.M == 0 || shape.N == 0 || grp.count == 0) return TI_OK;
  bool ptr_ok = (reinterpret_cast<uintptr_t>(shape.A) & 15) == 0;
  for (int i = 0; i < grp.count; ++i) ptr_ok = ptr_ok && (reinterpret_cast<uintptr_t>(grp.B[i]) & 15) == 0;
  const bool aligned = ptr_ok && (shape.K % SBK == 0) && shape.K > 0;
  const int spb = (shape.N + 15) / 16;
  const long long strips = (long long)spb * grp.count;
  if (aligned && shape.M <= 16 && strips >= 256) {
    g_last_kernel = "stream_group";
    const int cus = num_cus();
    auto launch = [&](auto kern, int rows, int per_cu) -> int {
      const int lds = 2 * rows * SBK + S_RED;
      static std::atomic<unsigned long long> lds_ok{0};
      if (int rc = allow_lds(kern, lds, lds_ok)) return rc;
      const long long slots = (long long)cus * per_cu;
      hipLaunchKernelGGL(kern, dim3((unsigned)(strips < slots ? strips : slots)), dim3(256), lds, stream, shape, spb,
                         (int)strips, grp);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
      return TI_OK;
    };
    if (shape.M == 1) return launch(gemm_stream_kernel<KIND, 1, 2, true>, 17, 4);
    if (shape.M <= 4) return launch(gemm_stream_kernel<KIND, 4, 2, true>, 20, 3);
    return launch(gemm_stream_kernel<KIND, 16, 2, true>, 32, 2);
  }
  // Prefill shapes whose width the 256x160 or 256x288 tiles divide: the problems are the batches of one
  // persistent launch, so the pipeline fill and the epilogue of one projection overlap the next one's work.
  if (ptr_ok && shape.M > 128 && shape.K % QBK == 0 && shape.K >= QBK && grp.count > 1 && shape.lda == shape.K &&
      shape.ldb == shape.K) {
    const long long cus = num_cus();
    auto fill = [&](long long tiles) { return (double)tiles / (double)(((tiles + cus - 1) / cus) * cus); };
    const long long rows256 = (shape.M + 255) / 256;
    const double e160 = shape.N % 160 == 0 ? 0.88 * fill(rows256 * (shape.N / 160) * grp.count) : 0.0;
    const double e288 = shape.N % 288 == 0 ? 0.95 * fill(rows256 * (shape.N / 288) * grp.count) : 0.0;
    if (e160 > 0.0 || e288 > 0.0) {
      GemmParams q = shape;
      q.batch = grp.count;
      if (e160 >= e288) {
        g_last_kernel = "pipe16_256x160_group";
        return launch_pipe16q<Pipe16QCfg<256, 160, 4, 2, KIND, true>>(q, stream, grp);
      }
      g_last_kernel = "pipe16_256x288_group";
      return launch_pipe16q<Pipe16QCfg<256, 288, 4, 2, KIND, true>>(q, stream, grp);
    }
  }
  for (int i = 0; i < grp.count; ++i) {
    GemmParams q = shape;
    q.B = grp.B[i];
    q.bias = grp.bias[i];
    q.C = grp.C[i];
    q.alpha = grp.alpha[i];
    q.beta = grp.beta[i];
    if (int rc = launch_gemm_kind_3(q, nullptr, 0, stream)) return rc;
  }
  return TI_OK;
}

int launch_gemm(int kind, const GemmParams& p, void* ws, long long ws_bytes, hipStream_t stream) {
  if (p.M == 0 || p.N == 0 || p.batch == 0) return TI_OK;
  switch (kind) {
    case EPI_S32_BIAS: return launch_gemm_kind_0(p, ws, ws_bytes, stream);
    case EPI_S32_SCALED: return launch_gemm_kind_1(p, ws, ws_bytes, stream);
    case EPI_F32_BIAS: return launch_gemm_kind_2(p, ws, ws_bytes, stream);
    case EPI_S8_BIAS: return launch_gemm_kind_3(p, ws, ws_bytes, stream);
    case EPI_S8_RELU: return launch_gemm_kind_4(p, ws, ws_bytes, stream);
    case EPI_F32_SCALE: return launch_gemm_kind_5(p, ws, ws_bytes, stream);
    case EPI_S8_SCALE: return launch_gemm_kind_6(p, ws, ws_bytes, stream);
    case EPI_S32_RAW: return launch_gemm_kind_7(p, ws, ws_bytes, stream);
    case EPI_F32_BIAS_ACC: return launch_gemm_kind_8(p, ws, ws_bytes, stream);
  }
  return fail(TI_ERR_INVALID_ARG, "unknown epilogue kind %d", kind);
}

}  // namespace ti

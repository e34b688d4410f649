// Host-side entry of the INT8 GEMM family: dispatch over the epilogue kinds (each kind's kernels are
// compiled in a translation unit of their own, gemm_s8_kinds.hip with -DTI_KIND=n), the grouped q/k/v
// launches, the split-K slice GEMM and the workspace query.
#include <cstdlib>
#include <mutex>

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

// ---------------------------------------------------------------------------
// State of the one-launch split-K (the FUSED form of gemm_pipe16q_kernel), per device.
//
// Arrival counters: zero when the code object is loaded, and every launch leaves them zero (the wave that arrives
// last puts its counter back).  Launches on one stream run one after the other, so each stream that uses the
// fused form gets a block of counters of its own (kFusedStreams of them per device; further streams take the
// two-launch form).
//
// Placement: the fused form needs all workgroups whose ids are congruent mod 8 to run on one XCD.  That is how the
// hardware deals workgroups out (round robin over the XCDs; the XCD of workgroup 0 depends on the queue).  A probe
// launch records the XCC id register of 256 workgroups once per device; unless it shows one XCC per residue class,
// eight different ones, the fused form stays off.  Every fused launch checks itself as well: the workgroups of a
// tile mark their XCC in a word of the tile, and one that finds another XCC's mark raises a flag in host memory;
// the flag is looked at before every later launch and turns the fused form off with an error.
static constexpr int kFusedStreams = 8;
static constexpr int kFusedCounters = 32768;            // per stream: tiles x waves
static constexpr int kFusedTiles = kFusedCounters / 8;  // per stream: one XCC word per tile
static __device__ __align__(256) int g_fused_arrivals[kFusedStreams * (kFusedCounters + kFusedTiles)];

__global__ void xcc_probe_kernel(unsigned* out) {
  if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf;  // HW_REG_XCC_ID
}

struct FusedDevice {
  std::mutex lock;
  int state = 0;  // 0 = not probed yet, 1 = usable, -1 = off
  int* arrivals = nullptr;
  int* host_words = nullptr;  // [0] = the misplacement flag, [1 .. 256] = the probe's output
  int* host_words_dev = nullptr;
  hipStream_t streams[kFusedStreams] = {};
  int nstreams = 0;
};
static FusedDevice g_fused[64];

// -1 = not decided yet: the environment variable TORCH_INT_FUSED_SPLITK=0 switches the form off
static std::atomic<int> g_fused_on{-1};

int set_fused_split(int enable) {
  int before = g_fused_on.load(std::memory_order_relaxed);
  if (before < 0) {
    const char* v = getenv("TORCH_INT_FUSED_SPLITK");
    before = !(v && v[0] == '0');
  }
  if (enable >= 0) g_fused_on.store(enable ? 1 : 0, std::memory_order_relaxed);
  else g_fused_on.store(before, std::memory_order_relaxed);
  return before;
}
static bool fused_enabled() { return set_fused_split(-1) != 0; }

// The first use on a device allocates 1 KB of host memory and synchronises; a thread that must not allocate (the
// entry point that promises it) clears this around its call and then only uses a device that is ready.
static thread_local bool g_fused_may_probe = true;
void allow_fused_split_probe(bool allow) { g_fused_may_probe = allow; }

// counters < 0: only make the current device ready (the probe), on `stream`
int fused_split_prepare(hipStream_t stream, long long counters, GemmParams& q) {
  if (!fused_enabled() || counters > kFusedCounters) return 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  FusedDevice& d = g_fused[dev];
  std::lock_guard<std::mutex> guard(d.lock);
  if (d.state == 0) {
    if (!g_fused_may_probe) return 0;
    // first use on this device: not while the stream records a graph (the probe allocates and synchronises)
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      return 0;
    }
    d.state = -1;
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_fused_arrivals)) != hipSuccess || sym == nullptr) return 0;
    if (hipHostMalloc(reinterpret_cast<void**>(&d.host_words), 257 * sizeof(int), hipHostMallocMapped) != hipSuccess)
      return 0;
    if (hipHostGetDevicePointer(reinterpret_cast<void**>(&d.host_words_dev), d.host_words, 0) != hipSuccess)
      return 0;
    for (int i = 0; i < 257; ++i) d.host_words[i] = -1;
    d.host_words[0] = 0;
    hipLaunchKernelGGL(xcc_probe_kernel, dim3(256), dim3(64), 0, stream,
                       reinterpret_cast<unsigned*>(d.host_words_dev + 1));
    if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) return 0;
    unsigned seen = 0;
    for (int i = 0; i < 256; ++i) {
      const int xcc = d.host_words[1 + i];
      if (xcc < 0 || xcc > 15 || xcc != d.host_words[1 + (i & 7)]) return 0;
    }
    for (int i = 0; i < 8; ++i) {
      const unsigned xcc = (unsigned)d.host_words[1 + i];
      if (seen & (1u << xcc)) return 0;  // two residue classes on one XCD: not the placement this needs
      seen |= 1u << xcc;
    }
    d.arrivals = static_cast<int*>(sym);
    d.state = 1;
  }
  if (d.state != 1) return 0;
  if (*reinterpret_cast<volatile int*>(d.host_words) != 0) {
    d.state = -1;  // a workgroup of an earlier fused launch ran on an unexpected XCD: its result cannot be trusted
    return -fail(TI_ERR_LAUNCH, "an earlier one-launch split-K GEMM found a workgroup on an unexpected XCD and its "
                                "result cannot be trusted; the form is now switched off (TORCH_INT_FUSED_SPLITK=0 "
                                "avoids it from the start)");
  }
  if (counters < 0) return 1;
  int slot = -1;
  for (int i = 0; i < d.nstreams; ++i)
    if (d.streams[i] == stream) slot = i;
  if (slot < 0) {
    if (d.nstreams == kFusedStreams) return 0;
    slot = d.nstreams++;
    d.streams[slot] = stream;
  }
  q.arrivals = d.arrivals + (long long)slot * (kFusedCounters + kFusedTiles);
  q.xcc_seen = reinterpret_cast<unsigned*>(q.arrivals + kFusedCounters);
  q.xcc_error = d.host_words_dev;
  return 1;
}

int warm_fused_split(void* stream) {
  GemmParams unused;
  const int rc = fused_split_prepare(static_cast<hipStream_t>(stream), -1, unused);
  return rc > 0 ? 1 : 0;
}

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
    // widths that only 128 divides (OPT-6.7B: 4096): 256x128 tiles, unless one problem at a time fills the CUs
    // with 256x256 tiles as well (three 2048x4096x4096: 98 -> 93 us, at 512 rows 57 -> 28 us; 2048x7168x7168
    // stays with three launches, 277 against 283 us)
    const double e256_alone = fill(rows256 * ((shape.N + 255) / 256));
    double e128 = shape.N % 128 == 0 ? 0.87 * fill(rows256 * (shape.N / 128) * grp.count) : 0.0;
    if (e128 < 0.5 || e128 <= e256_alone) e128 = 0.0;
    if (e160 > 0.0 || e288 > 0.0 || e128 > 0.0) {
      GemmParams q = shape;
      q.batch = grp.count;
      if (e160 >= e288 && e160 >= e128) {
        g_last_kernel = "pipe16_256x160_group";
        return launch_pipe16q<Pipe16QCfg<256, 160, 4, 2, KIND, true>>(q, stream, grp);
      }
      if (e288 >= e128) {
        g_last_kernel = "pipe16_256x288_group";
        return launch_pipe16q<Pipe16QCfg<256, 288, 4, 2, KIND, true>>(q, stream, grp);
      }
      g_last_kernel = "pipe16_256x128_group";
      return launch_pipe16q<Pipe16QCfg<256, 128, 4, 2, KIND, true>>(q, stream, grp);
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

// Host-side entry of the INT8 GEMM family: dispatch over the epilogue kinds (each kind's kernels are
// compiled in a translation unit of their own, gemm_s8_kinds.hip with -DTI_KIND=n), the grouped q/k/v
// launches, the split-K slice GEMM and the workspace query.
#include <cstdlib>
#include <mutex>

#include "gemm_s8_impl.h"

namespace ti {

long long gemm_workspace_bytes(long long M, long long N, long long K) {
  if (M > 1024) {  // the rows beyond the last multiple of 256 as a small problem of their own (row_split_rows)
    long long need = 0;
    const int r = row_split_rows(M, N, K, &need);
    if (r <= 0) return 0;
    // the first rows are a problem of their own too: at exactly 1024 of them they may split K themselves
    const long long head = M - r <= 1024 ? gemm_workspace_bytes(M - r, N, K) : 0;
    return head > need ? head : need;
  }
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

int gemm_row_split(long long M, long long N, long long K) { return row_split_rows(M, N, K); }

long long bmm_workspace_bytes(long long batch, long long M, long long N, long long K) {
  if (batch == 1) return gemm_workspace_bytes(M, N, K);  // one problem: the linears' split-K forms
  const int s = batched_splits(batch, M, N, K);
  return s > 1 ? (long long)s * batch * M * N * 4 : 0;
}

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
  bool live[kFusedStreams] = {};
  bool pinned[kFusedStreams] = {};  // a launch with this slot's counters was recorded into a graph: never handed on
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

// Runs the placement probe on `stream` (which must not be capturing) and waits for it: true when the 256 probe
// workgroups show one XCC per residue class of the workgroup id mod 8, eight different ones.
static bool probe_placement(FusedDevice& d, hipStream_t stream) {
  for (int i = 0; i < 256; ++i) d.host_words[1 + i] = -1;
  hipLaunchKernelGGL(xcc_probe_kernel, dim3(256), dim3(64), 0, stream, reinterpret_cast<unsigned*>(d.host_words_dev + 1));
  if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) return false;
  unsigned seen = 0;
  for (int i = 0; i < 256; ++i) {
    const int xcc = d.host_words[1 + i];
    if (xcc < 0 || xcc > 15 || xcc != d.host_words[1 + (i & 7)]) return false;
  }
  for (int i = 0; i < 8; ++i) {
    const unsigned xcc = (unsigned)d.host_words[1 + i];
    if (seen & (1u << xcc)) return false;  // two residue classes on one XCD: not the placement this needs
    seen |= 1u << xcc;
  }
  return true;
}

static bool is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) {
    (void)hipGetLastError();
    return true;  // unknown: treat as capturing (no probe, no registration)
  }
  return capturing != hipStreamCaptureStatusNone;
}

// 1 when a one-launch split-K GEMM on the current device has found a workgroup on an unexpected XCD (the output of
// that call cannot be trusted), 0 otherwise.  Reads one word of host memory; meaningful once the launches in
// question have finished.
int fused_split_faulted() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  FusedDevice& d = g_fused[dev];
  std::lock_guard<std::mutex> guard(d.lock);
  return d.host_words != nullptr && *reinterpret_cast<volatile int*>(d.host_words) != 0 ? 1 : 0;
}

// Decision logic of the fused form's bookkeeping, free of HIP calls so that it can be tested on the CPU.
// `flag` is the misplacement word, `state` the device state (0 not probed, 1 usable, -1 off).  Returns the action:
//   0 = take the two-launch form, 1 = go on (probe / slot lookup), -1 = report the misplacement and switch off.
int fused_flag_action(int state, int flag, bool enabled, long long counters, long long max_counters) {
  if (flag != 0 && state != 0) return -1;  // reported by whichever GEMM call comes next, fused or not
  if (!enabled || counters > max_counters) return 0;
  if (state < 0) return 0;
  return 1;
}

// Slot of `stream` among the `cap` slots of a device (`live[i]` = slot i holds a registered stream, `busy(i)` =
// that stream still has work queued): the stream's own slot, else a vacant one, else the first whose stream is
// idle (its counters are zero again: every launch leaves them zero), else -1.  `fresh` is set when the stream was
// not registered before.  Free of HIP calls so that it can be tested on the CPU.
template <class Busy>
static int pick_stream_slot(hipStream_t* streams, bool* live, int cap, hipStream_t stream, Busy busy, bool& fresh) {
  fresh = false;
  for (int i = 0; i < cap; ++i)
    if (live[i] && streams[i] == stream) return i;
  fresh = true;
  int slot = -1;
  for (int i = 0; i < cap && slot < 0; ++i)
    if (!live[i]) slot = i;
  for (int i = 0; i < cap && slot < 0; ++i)
    if (!busy(i)) slot = i;
  if (slot >= 0) {
    streams[slot] = stream;
    live[slot] = true;
  }
  return slot;
}

// CPU-testable face of pick_stream_slot: streams are plain integers, bit i of live_mask / busy_mask describes
// slot i; returns the slot and updates table / live_mask.
int fused_slot_for_test(long long* table, unsigned* live_mask, int cap, long long stream, unsigned busy_mask,
                        int* fresh) {
  hipStream_t tmp[32];
  bool live[32];
  if (cap > 32) cap = 32;
  for (int i = 0; i < cap; ++i) {
    tmp[i] = reinterpret_cast<hipStream_t>(table[i]);
    live[i] = (*live_mask >> i) & 1u;
  }
  bool f = false;
  const int slot = pick_stream_slot(tmp, live, cap, reinterpret_cast<hipStream_t>(stream),
                                    [&](int i) { return ((busy_mask >> i) & 1u) != 0; }, f);
  *live_mask = 0;
  for (int i = 0; i < cap; ++i) {
    table[i] = reinterpret_cast<long long>(tmp[i]);
    if (live[i]) *live_mask |= 1u << i;
  }
  *fresh = f ? 1 : 0;
  return slot;
}

static const char* kMisplacedMsg =
    "an earlier one-launch split-K GEMM on this device found a workgroup on an unexpected XCD and its result cannot "
    "be trusted (re-run it); the form is now switched off (TORCH_INT_FUSED_SPLITK=0 avoids it from the start)";

// Reports (once) a misplacement that an earlier fused launch on the current device flagged: TI_OK or TI_ERR_LAUNCH.
// Called at the start of every GEMM launch, whatever kernel it will take.
int fused_split_check() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return TI_OK;
  FusedDevice& d = g_fused[dev];
  if (d.host_words == nullptr) return TI_OK;  // never used here (written under the lock, before any fused launch)
  std::lock_guard<std::mutex> guard(d.lock);
  if (d.state == 1 && *reinterpret_cast<volatile int*>(d.host_words) != 0) {
    d.state = -1;
    return fail(TI_ERR_LAUNCH, "%s", kMisplacedMsg);
  }
  return TI_OK;
}

// counters == 0: only make the current device and `stream` ready (the probe)
int fused_split_prepare(hipStream_t stream, long long counters, GemmParams& q) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  FusedDevice& d = g_fused[dev];
  std::lock_guard<std::mutex> guard(d.lock);
  const int flag = d.host_words != nullptr ? *reinterpret_cast<volatile int*>(d.host_words) : 0;
  const int action = fused_flag_action(d.state, flag, fused_enabled(), counters, kFusedCounters);
  if (action < 0) {
    if (d.state == 1) {
      d.state = -1;
      return -fail(TI_ERR_LAUNCH, "%s", kMisplacedMsg);
    }
    return 0;  // already reported
  }
  if (action == 0) return 0;
  bool probed_now = false;  // the device's first probe ran on `stream` just now and vouches for it
  if (d.state == 0) {
    if (!g_fused_may_probe) return 0;
    // first use on this device: not while the stream records a graph (the probe allocates and synchronises)
    if (is_capturing(stream)) return 0;
    d.state = -1;
    void* sym = nullptr;
    if (hipGetSymbolAddress(&sym, HIP_SYMBOL(g_fused_arrivals)) != hipSuccess || sym == nullptr) return 0;
    if (hipHostMalloc(reinterpret_cast<void**>(&d.host_words), 257 * sizeof(int), hipHostMallocMapped) != hipSuccess) {
      d.host_words = nullptr;
      return 0;
    }
    d.host_words[0] = 0;
    if (hipHostGetDevicePointer(reinterpret_cast<void**>(&d.host_words_dev), d.host_words, 0) != hipSuccess)
      return 0;
    if (!probe_placement(d, stream)) return 0;
    d.arrivals = static_cast<int*>(sym);
    d.state = 1;
    probed_now = true;
  }
  bool fresh = false;
  const int slot = pick_stream_slot(d.streams, d.live, kFusedStreams, stream,
                                    [&](int i) { return d.pinned[i] || hipStreamQuery(d.streams[i]) == hipErrorNotReady; },
                                    fresh);
  (void)hipGetLastError();  // a query of a destroyed stream leaves an error behind; the slot counts as idle
  if (slot < 0) return 0;
  if (fresh && !probed_now) {
    // a stream seen for the first time: the XCD on which its workgroup 0 starts may differ, and a stream made with
    // a CU mask may not deal workgroups out this way at all, so the probe runs on it once (it synchronises the
    // stream, so not during a capture or from a caller that must not wait: the slot is given back then)
    if (!g_fused_may_probe || is_capturing(stream) || !probe_placement(d, stream)) {
      d.live[slot] = false;
      return 0;
    }
  } else if (!d.pinned[slot] && is_capturing(stream)) {
    d.pinned[slot] = true;  // the recording keeps these counters for as long as the graph lives
  }
  q.arrivals = d.arrivals + (long long)slot * (kFusedCounters + kFusedTiles);
  q.xcc_seen = reinterpret_cast<unsigned*>(q.arrivals + kFusedCounters);
  q.xcc_error = d.host_words_dev;
  return 1;
}

int warm_fused_split(void* stream) {
  GemmParams unused;
  const int rc = fused_split_prepare(static_cast<hipStream_t>(stream), 0, unused);
  return rc > 0 ? 1 : 0;
}

int launch_splitk_raw(int tile, const GemmParams& q, hipStream_t stream) {
  if (tile == SPLIT_128) return launch_pipe<PipeCfg<128, 128, 2, 2, 4, EPI_S32_RAW, false>>(q, stream);
  if (tile == SPLIT_256x160) return launch_pipe16q<Pipe16QCfg<256, 160, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x80) return launch_pipe16q<Pipe16QCfg<128, 80, 4, 1, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x160) return launch_pipe16q<Pipe16QCfg<128, 160, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x288) return launch_pipe16q<Pipe16QCfg<128, 288, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_128x192) return launch_pipe16q<Pipe16QCfg<128, 192, 4, 2, EPI_S32_RAW>>(q, stream);
  if (tile == SPLIT_256x288) return launch_pipe16q<Pipe16QCfg<256, 288, 4, 2, EPI_S32_RAW>>(q, stream);
  if (q.K % QBK == 0) return launch_pipe2<Pipe2Cfg<256, 256, 2, 4, EPI_S32_RAW, false>>(q, stream);
  return launch_pipe<PipeCfg<256, 256, 2, 4, 4, EPI_S32_RAW, false>>(q, stream);
}

// Tile width of the one persistent launch that runs a group of `count` [M,K] x [N,K] s8 linears at prefill sizes
// (160, 288 or 128), or 0 when the problems run one after the other.
static int group_prefill_tile(long long M, long long N, long long K, int count) {
  if (!(M > 128 && K % QBK == 0 && K >= QBK && count > 1)) return 0;
  const long long cus = num_cus();
  auto fill = [&](long long tiles) { return (double)tiles / (double)(((tiles + cus - 1) / cus) * cus); };
  const long long rows256 = (M + 255) / 256;
  const double e160 = N % 160 == 0 ? 0.88 * fill(rows256 * (N / 160) * count) : 0.0;
  const double e288 = N % 288 == 0 ? 0.95 * fill(rows256 * (N / 288) * count) : 0.0;
  // widths that only 128 divides (OPT-6.7B: 4096): 256x128 tiles, unless one problem at a time fills the CUs
  // with 256x256 tiles as well (three 2048x4096x4096: 98 -> 93 us, at 512 rows 57 -> 28 us; 2048x7168x7168
  // stays with three launches, 277 against 283 us)
  const double e256_alone = fill(rows256 * ((N + 255) / 256));
  double e128 = N % 128 == 0 ? 0.87 * fill(rows256 * (N / 128) * count) : 0.0;
  if (e128 < 0.5 || e128 <= e256_alone) e128 = 0.0;
  const double e = e160 > e288 ? (e160 > e128 ? e160 : e128) : (e288 > e128 ? e288 : e128);
  if (e <= 0.0) return 0;
  // Up to 1024 rows a problem may have a one-round tiling of its own that needs no workspace (128x80, 128x192 or
  // 256x192 tiles over the whole of K): when the cost model prices the problems one after the other below the
  // grouped launch, they run that way (three 512x12288x12288: 260 us grouped on 256x128 tiles, 250 us apart;
  // three 512x5120x5120 stay grouped).  Times as row_split_rows prices a tiling.
  if (M <= 1024) {
    int tile = 0;
    double t_one = -1.0;
    const int splits = choose_splits(M, N, K, &tile, &t_one);
    if (splits == 1 && t_one > 0.0 && (tile == SPLIT_128x80 || tile == SPLIT_128x192 || tile == SPLIT_256x192)) {
      const double t_group = (double)count * M * N * (double)(K / 64) * 0.85 / (65536.0 * (double)cus * e) + 8.0;
      if ((double)count * t_one < t_group) return 0;
    }
  }
  return e160 >= e288 && e160 >= e128 ? 160 : e288 >= e128 ? 288 : 128;
}

// Whether a group call of that shape is ONE launch (the streaming kernel at decode sizes, a tiled kernel at prefill
// sizes) rather than a loop over the problems; a caller that holds a split-K workspace does better with separate
// calls in the second case.
int gemm_group_is_one_launch(long long M, long long N, long long K, int count) {
  if (M <= 16) return K % SBK == 0 ? 1 : 0;
  return group_prefill_tile(M, N, K, count) != 0 ? 1 : 0;
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
  if (aligned && gemv_takes(shape) && strips >= 256) {
    g_last_kernel = "gemv_group";
    return launch_gemv<KIND, true>(shape, grp, grp.count, stream);
  }
  if (aligned && shape.M <= 16 && strips >= 256) {
    g_last_kernel = "stream_group";
    const int cus = num_cus();
    auto launch = [&](auto kern, int stages, int rows, int per_cu) -> int {
      const int lds = stages * rows * SBK + S_RED;
      static std::atomic<unsigned long long> lds_ok{0};
      if (int rc = allow_lds(kern, lds, lds_ok)) return rc;
      const long long slots = (long long)cus * per_cu;
      hipLaunchKernelGGL(kern, dim3((unsigned)(strips < slots ? strips : slots)), dim3(256), lds, stream, shape, spb,
                         (int)strips, grp);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
      return TI_OK;
    };
    const bool deep = stream_deep_pipeline(shape.M, strips, cus);
    if (shape.M == 1)
      return deep ? launch(gemm_stream_kernel<KIND, 1, 3, true>, 3, 17, 2)
                  : launch(gemm_stream_kernel<KIND, 1, 2, true>, 2, 17, 3);
    if (shape.M <= 4) return launch(gemm_stream_kernel<KIND, 4, 2, true>, 2, 20, 3);
    return deep ? launch(gemm_stream_kernel<KIND, 16, 3, true>, 3, 32, 1)
                : launch(gemm_stream_kernel<KIND, 16, 2, true>, 2, 32, 2);
  }
  // Prefill shapes whose width the 256x160, 256x288 or 256x128 tiles divide: the problems are the batches of one
  // persistent launch, so the pipeline fill and the epilogue of one projection overlap the next one's work.
  if (ptr_ok && shape.lda == shape.K && shape.ldb == shape.K) {
    const int tile = group_prefill_tile(shape.M, shape.N, shape.K, grp.count);
    if (tile != 0) {
      GemmParams q = shape;
      q.batch = grp.count;
      if (tile == 160) {
        g_last_kernel = "pipe16_256x160_group";
        return launch_pipe16q<Pipe16QCfg<256, 160, 4, 2, KIND, true>>(q, stream, grp);
      }
      if (tile == 288) {
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
  if (int rc = fused_split_check()) return rc;
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

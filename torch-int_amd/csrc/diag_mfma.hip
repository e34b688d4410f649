// Diagnostic, not part of any operator: loops that issue the instruction mix of the tiled INT8 GEMM mainloop
// on operands that never change, to measure what the matrix pipe sustains on this board with a given operand
// pattern (the caller fills `data`: a constant byte, or uniformly random bytes).  No result is produced; the
// accumulators are only folded into a value that is never stored unless it hits a magic number.
//
// One workgroup of 8 waves per CU, two waves per SIMD, as the 256x256-tile kernel runs.  Per step a wave issues
// 16 v_mfma_i32_32x32x32_i8 (a 128x64 wave tile over 64 bytes of K) and, depending on the mode,
//   mode 0  nothing else                                       -> the matrix pipe alone
//   mode 1  + 12 ds_read_b128 fragment reads, waited for       -> operands fed from LDS
//   mode 2  + 4 x 1 KiB global->LDS copies from a source that stays in L2 (1 MiB shared by all
//             workgroups), a wait that leaves the newest three steps of copies in flight, and a
//             workgroup barrier                                 -> the whole mainloop without the epilogue
#include "ti_common.h"

namespace ti {

#define TI_GLOBAL_AS __attribute__((address_space(1)))
#define TI_LDS_AS __attribute__((address_space(3)))

static constexpr int kDiagLds = 128 * 1024;

template <int MODE>
__global__ __launch_bounds__(512, 2) void mfma_loop_kernel(const int8_t* __restrict__ data, int iters, int* sink) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const char* g = reinterpret_cast<const char*>(data);
  // the lower half of the LDS holds the bytes the fragment reads fetch; the upper half receives the copies
  for (int i = threadIdx.x; i < 65536 / 16; i += 512)
    *reinterpret_cast<v4i*>(smem + i * 16) = *reinterpret_cast<const v4i*>(g + (size_t)i * 16);
  __syncthreads();
  v16i acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0;
  v4i a[2][8], b[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      a[s][r] = *reinterpret_cast<const v4i*>(g + ((size_t)(wave * 12 + r) * 64 + lane) * 16 + s * 131072);
#pragma unroll
    for (int r = 0; r < 4; ++r)
      b[s][r] = *reinterpret_cast<const v4i*>(g + ((size_t)(wave * 12 + 8 + r) * 64 + lane) * 16 + s * 131072);
  }
  const int rd_base = lane * 16 + (wave & 3) * 1024;
  const size_t goff = (size_t)(blockIdx.x % 8) * 131072 + wave * 4096 + lane * 16;  // 1 MiB in all: stays in L2
#define TI_MF(ai, bi, ci, S) \
  asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[ci]) : "v"(a[S][ai]), "v"(b[S][bi]))
#define TI_RD(dst, off)                                                                          \
  if (MODE >= 1) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(rd_base), "n"(off))
#define TI_STEP(S, T)                                                                                          \
  {                                                                                                            \
    if (MODE == 2) {                                                                                           \
      _Pragma("unroll") for (int j = 0; j < 4; ++j) __builtin_amdgcn_global_load_lds(                         \
          (const TI_GLOBAL_AS void*)(g + goff + j * 1024),                                                     \
          (TI_LDS_AS void*)((TI_LDS_AS char*)smem + 65536 + (S * 8 + wave) * 4096 + j * 1024), 16, 0, 0); \
    }                                                                                                          \
    TI_MF(0, 0, 0, S); TI_RD(a[T][0], 0);     TI_MF(1, 0, 1, S); TI_RD(a[T][1], 4096);                         \
    TI_MF(2, 0, 2, S); TI_RD(a[T][2], 8192);  TI_MF(3, 0, 3, S); TI_RD(a[T][3], 12288);                        \
    TI_MF(0, 1, 4, S); TI_RD(b[T][0], 16384); TI_MF(1, 1, 5, S); TI_RD(b[T][1], 20480);                        \
    TI_MF(2, 1, 6, S); TI_RD(a[T][4], 24576); TI_MF(3, 1, 7, S); TI_RD(a[T][5], 28672);                        \
    TI_MF(4, 2, 0, S); TI_RD(a[T][6], 32768); TI_MF(5, 2, 1, S); TI_RD(a[T][7], 36864);                        \
    TI_MF(6, 2, 2, S); TI_RD(b[T][2], 40960); TI_MF(7, 2, 3, S); TI_RD(b[T][3], 45056);                        \
    TI_MF(4, 3, 4, S); TI_MF(5, 3, 5, S); TI_MF(6, 3, 6, S); TI_MF(7, 3, 7, S);                                \
    if (MODE >= 1) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                          \
    if (MODE == 2) asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory");                              \
  }
  for (int it = 0; it < iters; it += 2) {
    TI_STEP(0, 1)
    TI_STEP(1, 0)
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  int s = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += acc[i][j];
  if (s == 0x12345678) sink[0] = 1;
#undef TI_STEP
#undef TI_RD
#undef TI_MF
}

static int diag_grid() {
  int dev = 0, count = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || count <= 0)
    count = 256;
  return count;
}

long long diag_mfma_loop_ops(long long iters) {
  // workgroups x 8 waves x steps x 16 instructions x (32 x 32 x 32 multiply-adds = 2 ops each)
  return (long long)diag_grid() * 8 * iters * 16 * 65536;
}

template <int MODE>
static int launch_mfma_loop(const int8_t* data, int iters, int* sink, hipStream_t stream) {
  auto kern = mfma_loop_kernel<MODE>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     kDiagLds);
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(diag_grid()), dim3(512), kDiagLds, stream, data, iters, sink);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "mfma loop launch: %s", hipGetErrorString(e));
  return TI_OK;
}

int launch_diag_mfma_loop(int mode, const int8_t* data, long long iters, int* sink, hipStream_t stream) {
  switch (mode) {
    case 0: return launch_mfma_loop<0>(data, (int)iters, sink, stream);
    case 1: return launch_mfma_loop<1>(data, (int)iters, sink, stream);
    case 2: return launch_mfma_loop<2>(data, (int)iters, sink, stream);
  }
  return fail(TI_ERR_INVALID_ARG, "diag_mfma_loop: mode must be 0, 1 or 2 (got %d)", mode);
}

// Store-rate diagnostic: `workgroups` workgroups of 8 waves write fp32 tiles of 256 x 160 of a row-major [M, N]
// matrix exactly as the 256x160 GEMM kernel's epilogue does (a wave owns 64 x 80, one 16-byte store per lane covers
// 16 rows x 64 bytes), `reps` times over the tiles blockIdx.x, + gridDim.x, ...; nothing else.  Every element
// written is 1.0f.  With few workgroups it measures what one CU can store, with one per CU the whole chip.
__global__ __launch_bounds__(512, 2) void store_loop_kernel(float* __restrict__ out, int N, int tiles_n, int tiles,
                                                            int reps) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1, r = lane & 15, g = lane >> 4;
  const v4f one = {1.0f, 1.0f, 1.0f, 1.0f};
  for (int rep = 0; rep < reps; ++rep)
    for (int t = blockIdx.x; t < tiles; t += gridDim.x) {
      const int tm = t / tiles_n, tn = t - tm * tiles_n;
      float* base = out + (size_t)(tm * 256 + wm * 64) * N + tn * 160 + wn * 80;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 5; ++j) *reinterpret_cast<v4f*>(base + (size_t)(i * 16 + r) * N + j * 16 + 4 * g) = one;
    }
}

int launch_diag_store_loop(float* out, long long M, long long N, int workgroups, int reps, hipStream_t stream) {
  const int tiles_n = (int)(N / 160), tiles = (int)(M / 256) * tiles_n;
  hipLaunchKernelGGL(store_loop_kernel, dim3(workgroups), dim3(512), 0, stream, out, (int)N, tiles_n,
                     tiles, reps);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "store loop launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// Copy-rate diagnostic: what one CU moves from the L2 with the GEMM mainloop's access pattern and nothing else.  One
// workgroup of 8 waves per CU; per step a wave fetches six row pieces of 128 contiguous bytes per 8-lane group (48 KiB
// per workgroup and step, a 256x160 tile's K step) from rows 5120 bytes apart, two steps in flight; the 2 MiB source is
// shared by all workgroups and stays in the L2.
//   mode 0  global->LDS copies (global_load_lds_dwordx4) into three rotating LDS stages
//   mode 1  16-byte loads into registers, folded with xor
static constexpr int kCopyPieces = 6, kCopyPitch = 5120;
template <int MODE>
__global__ __launch_bounds__(512) void copy_loop_kernel(const int8_t* __restrict__ data, int iters, int* sink) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const char* src[kCopyPieces];
#pragma unroll
  for (int j = 0; j < kCopyPieces; ++j)
    src[j] = reinterpret_cast<const char*>(data) + (size_t)((wave * kCopyPieces + j) * 8 + lane / 8) * kCopyPitch +
             (lane % 8) * 16;
  v4i acc = {0, 0, 0, 0};
  int koff = 0;
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
      TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + (it % 3) * (8 * kCopyPieces * 1024) + wave * kCopyPieces * 1024;
#pragma unroll
      for (int j = 0; j < kCopyPieces; ++j)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[j] + koff), (TI_LDS_AS void*)(dst + j * 1024),
                                         16, 0, 0);
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kCopyPieces) : "memory");
    } else {
      v4i v[kCopyPieces];
#pragma unroll
      for (int j = 0; j < kCopyPieces; ++j) v[j] = *reinterpret_cast<const v4i*>(src[j] + koff);
#pragma unroll
      for (int j = 0; j < kCopyPieces; ++j) acc ^= v[j];
    }
    koff = koff + 256 > kCopyPitch ? 0 : koff + 128;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (acc[0] + acc[1] + acc[2] + acc[3] == 0x12345678 || (iters < 0 && smem[threadIdx.x] == 77)) sink[0] = 1;
}

// Read-rate diagnostic: one pass over a weight matrix [N][K] of int8 with nothing but the loads, for the ceilings of
// the HBM-bound kernels (the streaming GEMM above all).
//   mode 0  flat: every workgroup reads 4 KiB pieces (256 lanes x 16 bytes), four in flight per lane, grid-stride
//   mode 1  the same with non-temporal loads
//   mode 2  the streaming GEMM's copy pipeline without its arithmetic: a workgroup of four waves owns strips of 16
//           rows and walks K in blocks of 1 KiB per row (one global->LDS copy instruction per row and block, waves
//           1..3 copy), three LDS stages, one wait and one barrier per block, non-temporal copies
//   mode 3  mode 2 with the default cache policy
template <bool NT>
__global__ __launch_bounds__(256) void read_flat_kernel(const v4i* __restrict__ src, long long n16, int* sink) {
  v4i acc = {0, 0, 0, 0};
  const long long stride = (long long)gridDim.x * 1024;
  for (long long i = (long long)blockIdx.x * 1024 + threadIdx.x; i < n16; i += stride) {
    v4i v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const v4i* a = src + i + u * 256;
      v[u] = i + u * 256 < n16 ? (NT ? __builtin_nontemporal_load(a) : *a) : v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u];
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x12345678) sink[0] = 1;
}

template <int AUX>
__global__ __launch_bounds__(256) void read_strips_kernel(const char* __restrict__ w, int N, int K, int* sink) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  constexpr int S = 3, STAGE = 16 * 1024, NCOPY = 6;  // 3 copying waves x 6 row copies >= 16 rows
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int strips = N / 16, KB = K / 1024;
  int my = 0;
  for (int s = blockIdx.x; s < strips; s += gridDim.x) ++my;
  if (my == 0) return;  // the same for every wave of the workgroup, before the first barrier
  const int G = my * KB;
  const int cw = wave > 0 ? wave - 1 : 0;
  int c_s = blockIdx.x, c_kb = 0, c_g = 0, live = 1;
  auto issue = [&]() {
    TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + (c_g % S) * STAGE;
    const char* base = w + (size_t)c_s * 16 * K + (size_t)c_kb * 1024 + lane * 16;
#pragma unroll
    for (int i = 0; i < NCOPY; ++i) {
      int q = cw + 3 * i;
      q = q < 16 ? q : 15;
      __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(base + (size_t)q * K), (TI_LDS_AS void*)(dst + q * 1024),
                                       16, 0, AUX);
    }
    c_kb += live;
    ++c_g;
    if (live && c_kb == KB) {  // past the last strip the final block is copied again: the wait count never changes
      if (c_g < G) {
        c_kb = 0;
        c_s += gridDim.x;
      } else {
        live = 0;
        c_kb = KB - 1;
      }
    }
  };
  if (wave > 0)
    for (int i = 0; i < S - 1; ++i) issue();
  int acc = 0;
  for (int g = 0; g < G; ++g) {
    if (wave > 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((S - 2) * NCOPY) : "memory");
    asm volatile("s_barrier" ::: "memory");
    if (wave > 0) issue();
    acc ^= *reinterpret_cast<const int*>(smem + (g % S) * STAGE + threadIdx.x * 4);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  if (acc == 0x12345678) sink[0] = 1;
}

int launch_diag_read_loop(int mode, const int8_t* data, long long N, long long K, int* sink, hipStream_t stream) {
  if (mode < 0 || mode > 3) return fail(TI_ERR_INVALID_ARG, "diag_read_loop: mode must be 0 ... 3 (got %d)", mode);
  if (N < 16 || N % 16 != 0 || K < 1024 || K % 1024 != 0 || N > (1 << 24) || K > (1 << 24))
    return fail(TI_ERR_INVALID_ARG, "diag_read_loop: N must be a multiple of 16 and K a multiple of 1024 (got %lld, %lld)",
                N, K);
  const int cus = diag_grid();
  if (mode <= 1) {
    auto kern = mode == 0 ? read_flat_kernel<false> : read_flat_kernel<true>;
    hipLaunchKernelGGL(kern, dim3(cus * 4), dim3(256), 0, stream, reinterpret_cast<const v4i*>(data), N * K / 16, sink);
  } else {
    auto kern = mode == 2 ? read_strips_kernel<2> : read_strips_kernel<0>;
    const int lds = 3 * 16 * 1024 + 29 * 1024;  // padded to 77 KiB: two workgroups per CU, as the GEMM kernel has
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
    const long long strips = N / 16, slots = 2LL * cus;
    hipLaunchKernelGGL(kern, dim3((unsigned)(strips < slots ? strips : slots)), dim3(256), lds, stream,
                       reinterpret_cast<const char*>(data), (int)N, (int)K, sink);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "read loop launch: %s", hipGetErrorString(e));
  return TI_OK;
}

long long diag_copy_loop_bytes(long long iters) { return (long long)diag_grid() * 8 * kCopyPieces * 1024 * iters; }

int launch_diag_copy_loop(int mode, const int8_t* data, long long iters, int* sink, hipStream_t stream) {
  if (mode != 0 && mode != 1) return fail(TI_ERR_INVALID_ARG, "diag_copy_loop: mode must be 0 or 1 (got %d)", mode);
  const int lds = mode == 0 ? 3 * 8 * kCopyPieces * 1024 : 0;
  auto kern = mode == 0 ? copy_loop_kernel<0> : copy_loop_kernel<1>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     3 * 8 * kCopyPieces * 1024);
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(diag_grid()), dim3(512), lds, stream, data, (int)iters, sink);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "copy loop launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// Instruction-mix diagnostic for the 16x16-block GEMM kernels: one workgroup per CU runs `iters` K steps of nothing
// but the instructions a wave of the real kernel issues per step, on operands that change every step (the LDS
// region the fragment reads fetch is filled from `data`), with no dependence on what the copies deliver:
//   shape 0  the 256x160 tile: 8 waves, each 40 v_mfma_i32_16x16x64_i8, 18 ds_read_b128, 7 global->LDS copies of 1 KiB
//   shape 1  the 128x80 tile:  4 waves, each 20 MFMAs, 14 reads, 7 copies
// `parts` is a bit set: 1 the MFMAs, 2 the fragment reads, 4 the copies (L2-resident source, two steps in flight) and
// their wait, 8 the workgroup barrier.  The time of parts = 15 is the floor of the kernel's K step on this board.
template <int WAVES, int NM, int NR, int NC, int PARTS>
__global__ __launch_bounds__(WAVES * 64) void mix_loop_kernel(const int8_t* __restrict__ data, int iters, int* sink) {
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const char* g = reinterpret_cast<const char*>(data);
  for (int i = threadIdx.x; i < 2048; i += WAVES * 64)
    *reinterpret_cast<v4i*>(smem + i * 16) = *reinterpret_cast<const v4i*>(g + (size_t)i * 16);
  __syncthreads();
  const char* src = g + (size_t)(blockIdx.x % 8) * 262144 + (size_t)wave * 8 * kCopyPitch + (lane >> 3) * kCopyPitch +
                    (lane & 7) * 16;
  v4i acc[10], f[14];
#pragma unroll
  for (int i = 0; i < 10; ++i) acc[i] = v4i{0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 14; ++i) f[i] = v4i{lane, i, wave, 1};
  const int rd = lane * 16 + (wave & 3) * 8192;
  int koff = 0;
  for (int it = 0; it < iters; ++it) {
    if (PARTS & 4) {
      TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + 32768 + (it & 1) * (WAVES * NC * 1024) + wave * NC * 1024;
#pragma unroll
      for (int j = 0; j < NC; ++j)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src + koff + j * 8 * kCopyPitch),
                                         (TI_LDS_AS void*)(dst + j * 1024), 16, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NM; ++i) {
      if (PARTS & 1)
        asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[i % 10]) : "v"(f[i % 7]), "v"(f[7 + i % 7]));
      if ((PARTS & 2) && i < NR)
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(f[i % 14]) : "v"(rd), "n"((i % 8) * 1024));
    }
    if (PARTS & 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NC) : "memory");  // two steps in flight, as the kernel
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (PARTS & 8) asm volatile("s_barrier" ::: "memory");
    koff = (koff + 128) & 4095;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  int s = 0;
#pragma unroll
  for (int i = 0; i < 10; ++i) s += acc[i][0] + acc[i][3];
#pragma unroll
  for (int i = 0; i < 14; ++i) s += f[i][1];
  if (s == 0x12345678) sink[0] = 1;
}

long long diag_mix_loop_ops(int shape, long long iters) {
  return (long long)diag_grid() * (shape == 0 ? 8 * 40 : 4 * 20) * iters * 32768;
}

template <int WAVES, int NM, int NR, int NC, int PARTS>
static int launch_mix(const int8_t* data, int iters, int* sink, hipStream_t stream) {
  auto kern = mix_loop_kernel<WAVES, NM, NR, NC, PARTS>;
  constexpr int lds = 32768 + 2 * WAVES * NC * 1024;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, dim3(diag_grid()), dim3(WAVES * 64), lds, stream, data, iters, sink);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "mix loop launch: %s", hipGetErrorString(e));
  return TI_OK;
}

int launch_diag_mix_loop(int shape, int parts, const int8_t* data, long long iters, int* sink, hipStream_t stream) {
#define TI_MIX(P)                                                                                 \
  case P:                                                                                         \
    return shape == 0 ? launch_mix<8, 40, 18, 7, P>(data, (int)iters, sink, stream)               \
                      : launch_mix<4, 20, 14, 7, P>(data, (int)iters, sink, stream)
  if (shape != 0 && shape != 1) return fail(TI_ERR_INVALID_ARG, "diag_mix_loop: shape must be 0 or 1 (got %d)", shape);
  switch (parts) {
    TI_MIX(1); TI_MIX(2); TI_MIX(3); TI_MIX(4); TI_MIX(5); TI_MIX(6); TI_MIX(7); TI_MIX(8);
    TI_MIX(9); TI_MIX(10); TI_MIX(11); TI_MIX(12); TI_MIX(13); TI_MIX(14); TI_MIX(15);
  }
#undef TI_MIX
  return fail(TI_ERR_INVALID_ARG, "diag_mix_loop: parts must be in [1, 15] (got %d)", parts);
}

}  // namespace ti

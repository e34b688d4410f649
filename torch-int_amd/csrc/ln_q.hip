// dq_add_layernorm_q for gfx950: dequantise an int32 tensor, add it to the fp32
// residual stream, LayerNorm over the last dimension and quantise to int8, in
// one pass over HBM (13 bytes per element: 4 in + 4 residual in + 4 residual
// out + 1 int8 out).
//
// The residual stream, gamma and beta are fp32 or, all three, fp16 (element type T).  With fp16 the arithmetic
// stays fp32 and rounds where a chain of torch ops on fp16 tensors rounds: the int32 input is converted to fp16
// first (torch.add casts it to the common dtype; magnitudes from 65520 up become infinity), the updated residual
// is rounded to fp16 before it is normalised (LayerNorm sees the stored tensor), and the LayerNorm output is
// rounded to fp16 before it is rounded to an integer.  9 bytes per element then.
//
// One 256-lane workgroup per row.  The row lives in registers between the
// three phases (sum, sum of squared deviations, normalise), so each input
// byte is read once.  The fp32 reduction order is fixed:
//   chunk c (elements 4c..4c+3) belongs to lane c % 256; a lane adds its
//   elements in ascending order; wavefronts combine with a xor butterfly
//   (offsets 32..1); the four wavefront sums are added left to right.
#include <type_traits>

#include "ti_common.h"

namespace ti {

__device__ __forceinline__ float wave_butterfly_sum(float s) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) s = s + __shfl_xor(s, off, 64);
  return s;
}

__device__ __forceinline__ float block_sum_256(float s, float* red) {
  s = wave_butterfly_sum(s);
  const int wave = threadIdx.x >> 6;
  __syncthreads();  // previous use of red[] is over
  if ((threadIdx.x & 63) == 0) red[wave] = s;
  __syncthreads();
  return ((red[0] + red[1]) + red[2]) + red[3];
}

typedef _Float16 v4h __attribute__((ext_vector_type(4)));

// four consecutive elements (chunk c) of a row as fp32 / stored from fp32
__device__ __forceinline__ v4f load4(const float* row, int c) { return reinterpret_cast<const v4f*>(row)[c]; }
__device__ __forceinline__ v4f load4(const _Float16* row, int c) {
  const v4h h = reinterpret_cast<const v4h*>(row)[c];
  return v4f{(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
}
__device__ __forceinline__ void store4(float* row, int c, v4f v) { reinterpret_cast<v4f*>(row)[c] = v; }
__device__ __forceinline__ void store4(_Float16* row, int c, v4f v) {
  reinterpret_cast<v4h*>(row)[c] = v4h{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
}
// The value a tensor of element type T holds after the fp32 value `x` is stored to it (round to nearest even
// for fp16).  The empty asm keeps the fp32 result of the preceding operation a value of its own: without it the
// compiler merges an fma and the conversion into one mixed-precision instruction that rounds the exact sum
// straight to fp16, which differs from "fp32 operation, then conversion" when the fp32 result is a tie.
template <class T>
__device__ __forceinline__ float as_stored(float x) {
  if constexpr (sizeof(T) == 2) asm volatile("" : "+v"(x));
  return (float)(T)x;
}

__device__ __forceinline__ int pack_s8x4(float y0, float y1, float y2, float y3) {
  unsigned b0 = (unsigned char)(int8_t)rne_s8(y0);
  unsigned b1 = (unsigned char)(int8_t)rne_s8(y1);
  unsigned b2 = (unsigned char)(int8_t)rne_s8(y2);
  unsigned b3 = (unsigned char)(int8_t)rne_s8(y3);
  return (int)(b0 | (b1 << 8) | (b2 << 16) | (b3 << 24));
}

// What is normalised: MODE_DQ_ADD  r = res + scale * float(in)   (int32 in; dq_add_layernorm_q)
//                     MODE_ADD     r = res + x                   (fp32 x passed through `in`)
//                     MODE_PLAIN   r = x                         (fp32 x passed through `res`; r is not stored)
//                     MODE_ADD_F32 r = res + T(x)                (fp32 x added to a stream of another type T:
//                                                                 `residual.add_(x.to(residual.dtype))`)
enum LnMode : int { MODE_DQ_ADD = 0, MODE_ADD = 1, MODE_PLAIN = 2, MODE_ADD_F32 = 3 };

// H % 4 == 0, H <= NC * 1024, all row starts 16-byte aligned.
// EARLY: gamma and beta are fetched together with the row instead of after the two reductions; with only
// a few rows in flight (decode) the kernel is a chain of memory latencies and this removes one of them,
// with many rows the extra registers would only cost occupancy.
template <int NC, int MODE, bool EARLY, class T>
__global__ __launch_bounds__(256) void ln_q_rows_kernel(const void* __restrict__ in, float scale,
                                                        const T* res,  // may alias r_out
                                                        const T* __restrict__ gamma,
                                                        const T* __restrict__ beta, float eps,
                                                        T* r_out, int8_t* __restrict__ q_out, int H) {
  __shared__ float red[4];
  const long long row = blockIdx.x;
  const int t = threadIdx.x;
  const int nchunks = H >> 2;
  const v4i* in4 = reinterpret_cast<const v4i*>(static_cast<const int32_t*>(in) + row * H);  // MODE_DQ_ADD
  const T* x_row = static_cast<const T*>(in) + row * H;                                        // MODE_ADD
  const float* xf32_row = static_cast<const float*>(in) + row * H;                             // MODE_ADD_F32
  const T* res_row = res + row * H;
  T* rout_row = r_out + row * H;
  int* q4 = reinterpret_cast<int*>(q_out + row * H);

  v4f ge[EARLY ? NC : 1], be[EARLY ? NC : 1];
  if constexpr (EARLY) {
#pragma unroll
    for (int i = 0; i < NC; ++i) {
      const int c = t + i * 256;
      if (c < nchunks) {
        ge[i] = load4(gamma, c);
        be[i] = load4(beta, c);
      }
    }
  }
  v4f r[NC];
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = t + i * 256;
    if (c < nchunks) {
      v4f a = load4(res_row, c);
      v4f v;
      if (MODE == MODE_DQ_ADD) {
        v4i x = in4[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = as_stored<T>(__builtin_fmaf(scale, as_stored<T>((float)x[j]), a[j]));
      } else if (MODE == MODE_ADD) {
        v4f x = load4(x_row, c);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = as_stored<T>(a[j] + x[j]);
      } else if (MODE == MODE_ADD_F32) {
        v4f x = load4(xf32_row, c);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = as_stored<T>(a[j] + as_stored<T>(x[j]));
      } else {
        v = a;
      }
      r[i] = v;
      if (MODE != MODE_PLAIN) store4(rout_row, c, v);
#pragma unroll
      for (int j = 0; j < 4; ++j) s = s + v[j];
    }
  }
  const float fH = (float)H;
  const float mu = block_sum_256(s, red) / fH;
  float s2 = 0.0f;
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = t + i * 256;
    if (c < nchunks) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float d = r[i][j] - mu;
        float sq = d * d;
        s2 = s2 + sq;
      }
    }
  }
  const float var = block_sum_256(s2, red) / fH;
  const float rstd = 1.0f / __builtin_sqrtf(var + eps);
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int c = t + i * 256;
    if (c < nchunks) {
      v4f g, b;
      if constexpr (EARLY) {
        g = ge[i];
        b = be[i];
      } else {
        g = load4(gamma, c);
        b = load4(beta, c);
      }
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) y[j] = as_stored<T>(__builtin_fmaf((r[i][j] - mu) * rstd, g[j], b[j]));
      q4[c] = pack_s8x4(y[0], y[1], y[2], y[3]);
    }
  }
}

// Any H and alignment: same reduction tree, scalar accesses, the row is
// recomputed from the inputs in each phase instead of being kept in registers.
template <class T>
__global__ __launch_bounds__(256) void ln_q_rows_generic_kernel(const void* __restrict__ in, float scale,
                                                                const T* res, const T* __restrict__ gamma,
                                                                const T* __restrict__ beta, float eps,
                                                                T* r_out, int8_t* __restrict__ q_out, int H,
                                                                int mode) {
  __shared__ float red[4];
  const long long row = blockIdx.x;
  const int t = threadIdx.x;
  const int32_t* x = static_cast<const int32_t*>(in) + row * H;
  const T* xf = static_cast<const T*>(in) + row * H;
  const float* xf32 = static_cast<const float*>(in) + row * H;
  const T* a = res + row * H;
  T* ro = r_out + row * H;
  int8_t* q = q_out + row * H;
  const int nchunks = (H + 3) >> 2;
  auto value = [&](int i) {
    if (mode == MODE_DQ_ADD) return as_stored<T>(__builtin_fmaf(scale, as_stored<T>((float)x[i]), (float)a[i]));
    if (mode == MODE_ADD) return as_stored<T>((float)a[i] + (float)xf[i]);
    if (mode == MODE_ADD_F32) return as_stored<T>((float)a[i] + as_stored<T>(xf32[i]));
    return (float)a[i];
  };
  float s = 0.0f;
  for (int c = t; c < nchunks; c += 256)
    for (int j = 0; j < 4; ++j) {
      const int i = c * 4 + j;
      if (i < H) s = s + value(i);
    }
  const float fH = (float)H;
  const float mu = block_sum_256(s, red) / fH;
  float s2 = 0.0f;
  for (int c = t; c < nchunks; c += 256)
    for (int j = 0; j < 4; ++j) {
      const int i = c * 4 + j;
      if (i < H) {
        float d = value(i) - mu;
        float sq = d * d;
        s2 = s2 + sq;
      }
    }
  const float var = block_sum_256(s2, red) / fH;
  const float rstd = 1.0f / __builtin_sqrtf(var + eps);
  // r_out may alias res: each element is read (above and here) only by the
  // lane that writes it, and the write comes last.
  for (int c = t; c < nchunks; c += 256)
    for (int j = 0; j < 4; ++j) {
      const int i = c * 4 + j;
      if (i < H) {
        float v = value(i);
        float y = as_stored<T>(__builtin_fmaf((v - mu) * rstd, (float)gamma[i], (float)beta[i]));
        if (mode != MODE_PLAIN) ro[i] = (T)v;
        q[i] = (int8_t)rne_s8(y);
      }
    }
}

template <int NC, class T>
static void launch_rows(int mode, const void* in, float scale, const T* res, const T* gamma, const T* beta, float eps,
                        T* r_out, int8_t* q_out, long long rows, int H, hipStream_t stream) {
  const dim3 grid((unsigned)rows), block(256);
  const bool early = rows <= 64;  // fewer rows than CUs: latency-bound
#define TI_LN_LAUNCH(MODE)                                                                                        \
  if (early)                                                                                                      \
    hipLaunchKernelGGL((ln_q_rows_kernel<NC, MODE, true, T>), grid, block, 0, stream, in, scale, res, gamma, beta, eps, \
                       r_out, q_out, H);                                                                          \
  else                                                                                                            \
    hipLaunchKernelGGL((ln_q_rows_kernel<NC, MODE, false, T>), grid, block, 0, stream, in, scale, res, gamma, beta, eps, \
                       r_out, q_out, H)
  if (mode == MODE_DQ_ADD) {
    TI_LN_LAUNCH(MODE_DQ_ADD);
  } else if (mode == MODE_ADD) {
    TI_LN_LAUNCH(MODE_ADD);
  } else if (mode == MODE_ADD_F32) {
    if constexpr (!std::is_same<T, float>::value) {  // for an fp32 stream this is MODE_ADD
      TI_LN_LAUNCH(MODE_ADD_F32);
    }
  } else {
    TI_LN_LAUNCH(MODE_PLAIN);
  }
#undef TI_LN_LAUNCH
}

template <class T>
static int launch_ln_mode(int mode, const void* in, float scale, const T* res, const T* gamma, const T* beta, float eps,
                          T* r_out, int8_t* q_out, long long rows, long long H, hipStream_t stream) {
  if (rows == 0 || H == 0) return TI_OK;
  // a chunk of four elements is one load: 16 bytes of fp32, 8 bytes of fp16 (16 bytes of the int32 input)
  constexpr uintptr_t kAlign = 4 * sizeof(T) - 1;
  auto al = [](const void* p, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(p) & mask) == 0; };
  const uintptr_t in_mask = mode == MODE_DQ_ADD || mode == MODE_ADD_F32 ? 15 : kAlign;
  const bool fast = (H % 4 == 0) && H <= 16 * 1024 && (mode == MODE_PLAIN || al(in, in_mask)) && al(res, kAlign) &&
                    al(gamma, kAlign) && al(beta, kAlign) && (mode == MODE_PLAIN || al(r_out, kAlign)) && al(q_out, 3);
  const int h = (int)H;
  if (fast) {
    const int nc = (int)((H + 1023) / 1024);
#define TI_LN_CASE(n)                                                                                \
  case n:                                                                                            \
    launch_rows<n, T>(mode, in, scale, res, gamma, beta, eps, r_out, q_out, rows, h, stream);        \
    break;
    switch (nc) {
      TI_LN_CASE(1) TI_LN_CASE(2) TI_LN_CASE(3) TI_LN_CASE(4) TI_LN_CASE(5) TI_LN_CASE(6) TI_LN_CASE(7)
      TI_LN_CASE(8) TI_LN_CASE(9) TI_LN_CASE(10) TI_LN_CASE(11) TI_LN_CASE(12) TI_LN_CASE(13)
      TI_LN_CASE(14) TI_LN_CASE(15) TI_LN_CASE(16)
    }
#undef TI_LN_CASE
  } else {
    hipLaunchKernelGGL(ln_q_rows_generic_kernel<T>, dim3((unsigned)rows), dim3(256), 0, stream, in, scale, res, gamma,
                       beta, eps, r_out, q_out, h, mode);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "layernorm_q launch: %s", hipGetErrorString(e));
  return TI_OK;
}

int launch_dq_add_layernorm_q(const int32_t* in, float scale, const float* res, const float* gamma,
                              const float* beta, float eps, float* r_out, int8_t* q_out, long long rows,
                              long long H, hipStream_t stream) {
  return launch_ln_mode<float>(MODE_DQ_ADD, in, scale, res, gamma, beta, eps, r_out, q_out, rows, H, stream);
}

// x == nullptr: q = LayerNormQ(residual); else residual += x (in place) and q = LayerNormQ(residual).
int launch_add_layernorm_q(const float* x, float* residual, const float* gamma, const float* beta, float eps,
                           int8_t* q_out, long long rows, long long H, hipStream_t stream) {
  if (x == nullptr)
    return launch_ln_mode<float>(MODE_PLAIN, nullptr, 1.0f, residual, gamma, beta, eps, nullptr, q_out, rows, H, stream);
  return launch_ln_mode<float>(MODE_ADD, x, 1.0f, residual, gamma, beta, eps, residual, q_out, rows, H, stream);
}

// The same two operations on an fp16 residual stream with fp16 gamma and beta (pointers to IEEE binary16).
int launch_dq_add_layernorm_q_f16(const int32_t* in, float scale, const void* res, const void* gamma, const void* beta,
                                  float eps, void* r_out, int8_t* q_out, long long rows, long long H,
                                  hipStream_t stream) {
  using H16 = _Float16;
  return launch_ln_mode<H16>(MODE_DQ_ADD, in, scale, static_cast<const H16*>(res), static_cast<const H16*>(gamma),
                             static_cast<const H16*>(beta), eps, static_cast<H16*>(r_out), q_out, rows, H, stream);
}

int launch_add_layernorm_q_f16(const void* x, void* residual, const void* gamma, const void* beta, float eps,
                               int8_t* q_out, long long rows, long long H, hipStream_t stream) {
  using H16 = _Float16;
  H16* r = static_cast<H16*>(residual);
  if (x == nullptr)
    return launch_ln_mode<H16>(MODE_PLAIN, nullptr, 1.0f, r, static_cast<const H16*>(gamma),
                               static_cast<const H16*>(beta), eps, nullptr, q_out, rows, H, stream);
  return launch_ln_mode<H16>(MODE_ADD, x, 1.0f, r, static_cast<const H16*>(gamma), static_cast<const H16*>(beta), eps, r,
                             q_out, rows, H, stream);
}

// residual (fp16) += fp16(x), elementwise, for an fp32 x: `residual.add_(x.to(residual.dtype))` in one pass (what the
// decoder layer does with the fp32 output of fc2 on an fp16 stream).  Chunks of four elements; a scalar tail.
__global__ __launch_bounds__(256) void add_f16_xf32_kernel(const float* __restrict__ x, _Float16* residual, long long n,
                                                           bool vec) {
  const long long c = (long long)blockIdx.x * 256 + threadIdx.x;
  if (c * 4 >= n) return;
  if (vec && c * 4 + 4 <= n) {
    const v4f a = reinterpret_cast<const v4f*>(x)[c];
    const v4h h = reinterpret_cast<const v4h*>(residual)[c];
    v4h o;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = (_Float16)as_stored<_Float16>((float)h[j] + as_stored<_Float16>(a[j]));
    reinterpret_cast<v4h*>(residual)[c] = o;
  } else {
    for (long long i = c * 4; i < n && i < c * 4 + 4; ++i)
      residual[i] = (_Float16)as_stored<_Float16>((float)residual[i] + as_stored<_Float16>(x[i]));
  }
}

int launch_add_f16_xf32(const float* x, void* residual, long long n, hipStream_t stream) {
  if (n == 0) return TI_OK;
  const bool vec = (reinterpret_cast<uintptr_t>(x) & 15) == 0 && (reinterpret_cast<uintptr_t>(residual) & 7) == 0;
  const long long chunks = (n + 3) / 4;
  hipLaunchKernelGGL(add_f16_xf32_kernel, dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, stream, x,
                     static_cast<_Float16*>(residual), n, vec);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "add_f16_xf32 launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// residual (fp16) += fp16(x) for an fp32 x, then the LayerNorm-quantiser: `residual.add_(x.to(residual.dtype))`
// followed by LayerNormQ, as the decoder layer does with the fp32 output of out_proj on an fp16 stream.
int launch_add_layernorm_q_f16_xf32(const float* x, void* residual, const void* gamma, const void* beta, float eps,
                                    int8_t* q_out, long long rows, long long H, hipStream_t stream) {
  using H16 = _Float16;
  H16* r = static_cast<H16*>(residual);
  return launch_ln_mode<H16>(MODE_ADD_F32, x, 1.0f, r, static_cast<const H16*>(gamma), static_cast<const H16*>(beta), eps,
                             r, q_out, rows, H, stream);
}

}  // namespace ti

// Row softmax of fp32 attention scores fused with the additive mask, the clamp
// to the most negative finite float and the quantisation to int8
// probabilities (round(127 p)): the op chain between the two attention
// products of an int8 OPT attention block, in one pass over HBM
// (4 bytes read + 1 byte written per element; the mask is shared by all heads
// of a batch and stays in L2).
//
// One wavefront per row; the row lives in registers.  Every arithmetic step is
// a fixed sequence of IEEE fp32 operations (own exp built from fma, fixed
// reduction order), so the result is reproducible bit for bit on any
// implementation that follows the same sequence.
#include "ti_common.h"
#include "softmax_math.h"

namespace ti {

// NV = float4 vectors per lane; S % 4 == 0, S <= NV * 256, 16-byte aligned rows.
// Chunk c (elements 4c..4c+3) belongs to lane c % 64; a lane accumulates its elements in
// ascending order; lanes combine with a xor butterfly (offsets 32..1).
template <int NV>
__global__ __launch_bounds__(256) void attn_softmax_q_kernel(const float* __restrict__ scores,
                                                             const float* __restrict__ mask,
                                                             int8_t* __restrict__ out, long long rows, int T, int S,
                                                             int heads) {
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const int nchunks = S >> 2;
  const v4f* src = reinterpret_cast<const v4f*>(scores + row * S);
  const v4f* msk = nullptr;
  if (mask != nullptr) {
    const long long bh = row / T;
    const long long t = row - bh * T;
    msk = reinterpret_cast<const v4f*>(mask + ((bh / heads) * T + t) * S);
  }
  const float lowest = -3.402823466e+38f;
  v4f v[NV];
  float m = lowest;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      v4f x = src[c];
      if (msk != nullptr) {
        const v4f k = msk[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = x[j] + k[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = x[j] > lowest ? x[j] : lowest;  // -inf (and NaN) -> most negative finite
        m = m > x[j] ? m : x[j];
      }
      v[i] = x;
    }
  }
  m = wave_max(m);
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float e = exp_nonpos(v[i][j] - m);
        v[i][j] = e;
        s = s + e;
      }
    }
  }
  s = wave_sum(s);
  const float scale = 127.0f / s;  // one division per row; probabilities are e * scale
  int* dst = reinterpret_cast<int*>(out + row * S);
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + i * 64;
    if (c < nchunks) {
      unsigned w = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float pq = __builtin_rintf(v[i][j] * scale);  // in [0, 127]
        w |= (unsigned)(int)pq << (8 * j);
      }
      dst[c] = (int)w;
    }
  }
}

// Any S / alignment: same arithmetic and the same reduction order, scalar accesses, three passes.
__global__ __launch_bounds__(256) void attn_softmax_q_generic_kernel(const float* __restrict__ scores,
                                                                     const float* __restrict__ mask,
                                                                     int8_t* __restrict__ out, long long rows, int T,
                                                                     int S, int heads) {
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int lane = threadIdx.x & 63;
  const float* src = scores + row * S;
  const float* msk = nullptr;
  if (mask != nullptr) {
    const long long bh = row / T;
    const long long t = row - bh * T;
    msk = mask + ((bh / heads) * T + t) * S;
  }
  const float lowest = -3.402823466e+38f;
  const int nchunks = (S + 3) >> 2;
  auto value = [&](int i) {
    float x = src[i];
    if (msk != nullptr) x = x + msk[i];
    return x > lowest ? x : lowest;
  };
  float m = lowest;
  for (int c = lane; c < nchunks; c += 64)
    for (int j = 0; j < 4; ++j)
      if (c * 4 + j < S) {
        const float x = value(c * 4 + j);
        m = m > x ? m : x;
      }
  m = wave_max(m);
  float s = 0.0f;
  for (int c = lane; c < nchunks; c += 64)
    for (int j = 0; j < 4; ++j)
      if (c * 4 + j < S) s = s + exp_nonpos(value(c * 4 + j) - m);
  s = wave_sum(s);
  const float scale = 127.0f / s;
  for (int c = lane; c < nchunks; c += 64)
    for (int j = 0; j < 4; ++j)
      if (c * 4 + j < S)
        out[row * S + c * 4 + j] = (int8_t)(int)__builtin_rintf(exp_nonpos(value(c * 4 + j) - m) * scale);
}

int launch_attn_softmax_q(const float* scores, const float* mask, int8_t* out, long long batch, long long heads,
                          long long T, long long S, hipStream_t stream) {
  const long long rows = batch * heads * T;
  if (rows == 0 || S == 0) return TI_OK;
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool fast = (S % 4 == 0) && S <= 16 * 256 && al16(scores) && (mask == nullptr || al16(mask)) &&
                    ((reinterpret_cast<uintptr_t>(out) & 3) == 0);
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  if (fast) {
    const int nv = (int)((S + 255) / 256);
#define TI_SM_CASE(n)                                                                                          \
  case n:                                                                                                      \
    hipLaunchKernelGGL(attn_softmax_q_kernel<n>, grid, block, 0, stream, scores, mask, out, rows, (int)T, (int)S, \
                       (int)heads);                                                                            \
    break;
    switch (nv) {
      TI_SM_CASE(1) TI_SM_CASE(2) TI_SM_CASE(3) TI_SM_CASE(4) TI_SM_CASE(5) TI_SM_CASE(6) TI_SM_CASE(7) TI_SM_CASE(8)
      TI_SM_CASE(9) TI_SM_CASE(10) TI_SM_CASE(11) TI_SM_CASE(12) TI_SM_CASE(13) TI_SM_CASE(14) TI_SM_CASE(15)
      TI_SM_CASE(16)
    }
#undef TI_SM_CASE
  } else {
    hipLaunchKernelGGL(attn_softmax_q_generic_kernel, grid, block, 0, stream, scores, mask, out, rows, (int)T, (int)S,
                       (int)heads);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_softmax_q launch: %s", hipGetErrorString(e));
  return TI_OK;
}

}  // namespace ti

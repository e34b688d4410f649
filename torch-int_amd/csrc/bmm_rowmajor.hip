// c[b, m, n] = s8(rint(clamp(alpha * sum_k a[b, m, k] * bm[b, k, n])))  with bm ROW-major [batch, K, N].
//
// The attention block's P.V product during incremental decoding: P is [batch*heads, 1..16, src]
// and V sits in the KV cache as [batch*heads, src, d].  Reading V in place streams it once with
// full 128-byte rows; the A.B^T entry points would first need V^T (a transposing copy of the
// whole cache per step) and then hit a K = src that is rarely a multiple of 16.  HBM-bound:
// batch*K*N bytes of V, nothing else of any size.
#include "ti_common.h"

namespace ti {

constexpr int RM_KC = 1024;  // bytes of each A row staged in LDS per pass over K
constexpr int RM_BN = 128;   // output columns per workgroup

// 256 threads = 32 column quads x 8 interleaved K slices.  MR rows of A per workgroup.
// FAST: N % 4 == 0 and bm / c are 4-byte aligned, so four columns move as one dword.
template <int MR, bool FAST>
__global__ __launch_bounds__(256) void bmm_rowmajor_kernel(const int8_t* __restrict__ A, const int8_t* __restrict__ B,
                                                           int8_t* __restrict__ C, int M, int N, int K, int tiles_n,
                                                           int groups_m, long long stride_b, float alpha) {
  __shared__ int8_t a_s[MR][RM_KC];
  __shared__ int red[4][MR][RM_BN];
  const int t = threadIdx.x, cq = t & 31, ks = t >> 5, wave = t >> 6;
  const int tn = blockIdx.x % tiles_n;
  const int gm = (blockIdx.x / tiles_n) % groups_m;
  const long long b = blockIdx.x / (tiles_n * groups_m);
  const int n = tn * RM_BN + cq * 4;
  const int m0 = gm * MR;
  int acc[MR][4];
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[m][j] = 0;

  for (int kc0 = 0; kc0 < K; kc0 += RM_KC) {
    const int kc = K - kc0 < RM_KC ? K - kc0 : RM_KC;
    __syncthreads();  // the previous pass has finished reading a_s
#pragma unroll
    for (int m = 0; m < MR; ++m) {
      const bool live = m0 + m < M;
      const int8_t* arow = A + ((b * M + (live ? m0 + m : 0)) * (long long)K + kc0);
      for (int k = t; k < kc; k += 256) a_s[m][k] = live ? arow[k] : (int8_t)0;
    }
    __syncthreads();
    const int8_t* bbase = B + (b * stride_b + kc0 * (long long)N + n);
    constexpr int U = 8;  // rows of bm in flight per thread
    for (int k0 = ks; k0 < kc; k0 += 8 * U) {
      int w[U][4];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = k0 + 8 * u;
        if (FAST) {
          int v = 0;
          if (k < kc && n < N) v = *reinterpret_cast<const int*>(bbase + (long long)k * N);
          w[u][0] = (v << 24) >> 24;
          w[u][1] = (v << 16) >> 24;
          w[u][2] = (v << 8) >> 24;
          w[u][3] = v >> 24;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) w[u][j] = (k < kc && n + j < N) ? (int)bbase[(long long)k * N + j] : 0;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int k = k0 + 8 * u;
        if (k >= kc) break;
#pragma unroll
        for (int m = 0; m < MR; ++m) {
          const int a = a_s[m][k];
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[m][j] += a * w[u][j];
        }
      }
    }
  }
  // the two K slices of a wave meet in its lower half, then the four waves through LDS
#pragma unroll
  for (int m = 0; m < MR; ++m)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[m][j] += __shfl_xor(acc[m][j], 32);
  if ((t & 32) == 0) {
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
      for (int j = 0; j < 4; ++j) red[wave][m][cq * 4 + j] = acc[m][j];
  }
  __syncthreads();
  for (int idx = t; idx < MR * 32; idx += 256) {
    const int m = idx >> 5, q = idx & 31;
    const int nn = tn * RM_BN + q * 4;
    if (m0 + m >= M || nn >= N) continue;
    int8_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int s = red[0][m][q * 4 + j] + red[1][m][q * 4 + j] + red[2][m][q * 4 + j] + red[3][m][q * 4 + j];
      o[j] = Epi<EPI_S8_SCALE>::apply(s, 0.0f, alpha);
    }
    int8_t* dst = C + ((b * M + m0 + m) * (long long)N + nn);
    if (FAST) {
      *reinterpret_cast<unsigned*>(dst) = (unsigned)(unsigned char)o[0] | ((unsigned)(unsigned char)o[1] << 8) |
                                          ((unsigned)(unsigned char)o[2] << 16) | ((unsigned)(unsigned char)o[3] << 24);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (nn + j < N) dst[j] = o[j];
    }
  }
}

template <int MR>
static void launch_rm(bool fast, dim3 grid, hipStream_t stream, const int8_t* a, const int8_t* b, int8_t* c, int M,
                      int N, int K, int tiles_n, int groups_m, long long stride_b, float alpha) {
  if (fast)
    hipLaunchKernelGGL((bmm_rowmajor_kernel<MR, true>), grid, dim3(256), 0, stream, a, b, c, M, N, K, tiles_n,
                       groups_m, stride_b, alpha);
  else
    hipLaunchKernelGGL((bmm_rowmajor_kernel<MR, false>), grid, dim3(256), 0, stream, a, b, c, M, N, K, tiles_n,
                       groups_m, stride_b, alpha);
}

int launch_bmm_s8t_s8t_s8t(const int8_t* a, const int8_t* b, int8_t* c, long long batch, long long M, long long N,
                           long long K, long long stride_b, float alpha, hipStream_t stream) {
  if (batch == 0 || M == 0 || N == 0) return TI_OK;
  const int mr = M == 1 ? 1 : (M <= 4 ? 4 : 16);
  const long long tiles_n = (N + RM_BN - 1) / RM_BN, groups_m = (M + mr - 1) / mr;
  const long long wgs = tiles_n * groups_m * batch;
  if (wgs > 0x7fffffffLL) return fail(TI_ERR_INVALID_ARG, "bmm_s8t_s8t_s8t: too many output tiles (%lld)", wgs);
  const bool fast = (N % 4 == 0) && (stride_b % 4 == 0) && (reinterpret_cast<uintptr_t>(b) % 4 == 0) &&
                    (reinterpret_cast<uintptr_t>(c) % 4 == 0);
  const dim3 grid((unsigned)wgs);
  if (mr == 1)
    launch_rm<1>(fast, grid, stream, a, b, c, (int)M, (int)N, (int)K, (int)tiles_n, (int)groups_m, stride_b, alpha);
  else if (mr == 4)
    launch_rm<4>(fast, grid, stream, a, b, c, (int)M, (int)N, (int)K, (int)tiles_n, (int)groups_m, stride_b, alpha);
  else
    launch_rm<16>(fast, grid, stream, a, b, c, (int)M, (int)N, (int)K, (int)tiles_n, (int)groups_m, stride_b, alpha);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "bmm_s8t_s8t_s8t launch: %s", hipGetErrorString(e));
  return TI_OK;
}

}  // namespace ti

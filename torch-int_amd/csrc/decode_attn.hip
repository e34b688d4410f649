// Attention for incremental decoding in one launch: per (batch, head) one workgroup appends the new
// key / value rows to the KV cache, computes alpha_qk * Q.K^T over the whole cache, turns the scores into
// int8 probabilities (mask, clamp, softmax, *127, round: the arithmetic and the summation order of
// attn_softmax_q) and multiplies them with V as the cache stores it ([len, head_dim] rows).  It replaces
// the append, skinny Q.K^T, softmax and row-major P.V launches of a decode step; the scores and the
// probabilities stay in LDS.  HBM-bound on the 2 * len * head_dim bytes of cache per (batch, head).
//
// 256 threads.  A cache row is read by head_dim/16 adjacent lanes (16 bytes each), so one load
// instruction of a wave covers 64*16/head_dim whole rows; partial dot products meet through lane
// shuffles (integers: any order gives the same bits).
#include "ti_common.h"
#include "softmax_math.h"

namespace ti {

constexpr int DA_MAX_T = 4;         // query rows per (batch, head)
constexpr int DA_LDS_LIMIT = 60 * 1024;

__device__ __forceinline__ int dot16(v4i a, v4i b, int c) {
#pragma unroll
  for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_sdot4(a[i], b[i], c, false);
  return c;
}

// Sum over the LPR (4 or 8) adjacent lanes that share a cache row, through DPP lane permutes: within quads
// (lane ^ 1, lane ^ 2), then across the two quads of an 8-lane group (mirror of the half row).
template <int LPR>
__device__ __forceinline__ int row_sum(int a) {
  a += __builtin_amdgcn_mov_dpp(a, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  a += __builtin_amdgcn_mov_dpp(a, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  if (LPR == 8) a += __builtin_amdgcn_mov_dpp(a, 0x141, 0xf, 0xf, true);  // row_half_mirror
  return a;
}

// Bytes of dynamic LDS: fp32 scores [T][Sp], int8 probabilities [T][Sp], partial outputs [4][T][D].
__host__ __device__ inline long long decode_attn_lds(long long T, long long S, long long D) {
  const long long Sp = (S + 3) / 4 * 4;
  return T * Sp * 4 + T * Sp + 4 * T * D * 4;
}

// NI > 0: the whole cache of the (batch, head) is at most NI row groups per lane and all of its loads are
// issued up front (keys and values, 16 bytes each per lane), so the kernel waits for memory once.
// NI == 0: any length, four row groups in flight at a time.
// PART: the head size in memory is smaller than D, the bytes of a cache row that the lanes cover; the forms for
// head sizes 64 and 128 carry none of its tests.
template <int TQ, int D, int NI, bool PART>
__global__ __launch_bounds__(256) void decode_attn_kernel(const int8_t* __restrict__ q, const int8_t* __restrict__ k_new,
                                                          const int8_t* __restrict__ v_new, int8_t* k_buf,
                                                          int8_t* v_buf, const float* __restrict__ mask,
                                                          int8_t* __restrict__ ctx, int8_t* __restrict__ probs_out,
                                                          int T, int S_arg, long long cap, int heads, float alpha_qk,
                                                          float alpha_pv, const int* __restrict__ s_dev, int dr_arg) {
  const int dr = PART ? dr_arg : D;
  // dr = the head size in memory, a multiple of 16 up to D (64 or 128, the lanes a cache row is spread over):
  // rows of q, the caches and ctx are dr bytes long; the lanes beyond a row hold zeros and store nothing
  // s_dev != nullptr: the number of positions is read from device memory (a launch recorded in a HIP graph is
  // replayed for a cache that has grown meanwhile; S_arg is then the largest length the launch was sized for)
  // (clamped to the contract T <= length <= S_arg: the host cannot check a value it never sees, and a length
  // outside that range would index past the LDS score rows and the cache buffers)
  int S = S_arg;
  if (s_dev != nullptr) {
    S = s_dev[0];
    S = S < T ? T : S;
    S = S > S_arg ? S_arg : S;
  }
  constexpr int LPR = D / 16;    // lanes per cache row
  constexpr int RPW = 64 / LPR;  // rows per wave per load
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int Sp = (S + 3) & ~3;
  float* scores = reinterpret_cast<float*>(smem);                              // [T][Sp]
  int8_t* probs = reinterpret_cast<int8_t*>(smem + (size_t)T * Sp * 4);        // [T][Sp]
  int* red = reinterpret_cast<int*>(smem + (size_t)T * Sp * 5);                // [4][T][D]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rs = lane / LPR, cs = lane % LPR;
  const bool in_row = !PART || cs * 16 < dr;
  const long long bh = blockIdx.x;
  const int S_old = k_new != nullptr ? S - T : S;  // rows below come from the cache, the rest from k_new / v_new
  int8_t* kb = k_buf + bh * cap * dr;
  int8_t* vb = v_buf + bh * cap * dr;
  const int8_t* kn = k_new != nullptr ? k_new + bh * T * dr : nullptr;
  const int8_t* vn = v_new != nullptr ? v_new + bh * T * dr : nullptr;

  // ---- phase 1: scores[t][s] = alpha_qk * (q[t] . k[s]); new key rows go into the cache on the way
  v4i qr[TQ];
#pragma unroll
  for (int t = 0; t < TQ; ++t)
    qr[t] = t < T && in_row ? *reinterpret_cast<const v4i*>(q + (bh * T + t) * dr + cs * 16) : v4i{0, 0, 0, 0};
  constexpr int U = NI > 0 ? NI : 4;  // row groups in flight per wave
  // Rows past the end re-read the last row (their products are never used), so the loads need no branches;
  // rows that come from k_new / v_new are also written into the cache.
  auto load_rows = [&](int base, v4i (&dst)[U], int8_t* buf, const int8_t* fresh) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      int s = base + u * 4 * RPW + rs;
      s = s < S ? s : S - 1;
      const int8_t* src = s < S_old ? buf + (long long)s * dr : fresh + (long long)(s - S_old) * dr;
      dst[u] = in_row ? *reinterpret_cast<const v4i*>(src + cs * 16) : v4i{0, 0, 0, 0};
    }
    if (S_old < S) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int s = base + u * 4 * RPW + rs;
        if (s >= S_old && s < S && in_row) *reinterpret_cast<v4i*>(buf + (long long)s * dr + cs * 16) = dst[u];
      }
    }
  };
  // the additive mask of the rows a lane will score, fetched together with the cache rows
  const float* msk = mask != nullptr ? mask + (bh / heads) * T * (long long)S : nullptr;
  const float lowest = -3.402823466e+38f;
  auto load_mask = [&](int base, float (&mk)[U][TQ]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int s = base + u * 4 * RPW + rs;
#pragma unroll
      for (int t = 0; t < TQ; ++t) mk[u][t] = (msk != nullptr && cs == 0 && s < S && t < T) ? msk[t * (long long)S + s] : 0.0f;
    }
  };
  // what the softmax reads: max(alpha_qk * acc + mask, most negative finite float)
  auto score_rows = [&](int base, v4i (&kv)[U], float (&mk)[U][TQ]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (base + u * 4 * RPW >= S) break;  // the same for every lane of the wave
      const int s = base + u * 4 * RPW + rs;
#pragma unroll
      for (int t = 0; t < TQ; ++t) {
        const int a = row_sum<LPR>(dot16(kv[u], qr[t], 0));
        if (cs == 0 && s < S && t < T) {
          float x = Epi<EPI_F32_SCALE>::apply(a, 0.0f, alpha_qk);
          if (msk != nullptr) x = x + mk[u][t];
          scores[t * Sp + s] = x > lowest ? x : lowest;
        }
      }
    }
  };
  v4i vv[U];
  if constexpr (NI > 0) {
    v4i kv[U];
    float mk[U][TQ];
    load_rows(wave * RPW, kv, kb, kn);
    load_mask(wave * RPW, mk);
    load_rows(wave * RPW, vv, vb, vn);
    score_rows(wave * RPW, kv, mk);
  } else {
    for (int base = wave * RPW; base < S; base += 4 * RPW * U) {
      v4i kv[U];
      float mk[U][TQ];
      load_rows(base, kv, kb, kn);
      load_mask(base, mk);
      score_rows(base, kv, mk);
    }
  }
  __syncthreads();

  // ---- phase 2: int8 probabilities.  The maximum, the exponentials and the rounding use all threads;
  // the sum of a row is taken by one wave in the order of attn_softmax_q (chunk c of four elements belongs
  // to lane c % 64, a lane adds its elements in ascending order, lanes combine with a xor butterfly 32..1).
  float* wmax = reinterpret_cast<float*>(red);  // [4] per row, then [1] scale per row: red is free until phase 3
  for (int t = 0; t < T; ++t) {
    float* row = scores + t * Sp;
    float m = lowest;
    for (int i = tid; i < S; i += 256) m = m > row[i] ? m : row[i];
    m = wave_max(m);
    if (lane == 0) wmax[t * 8 + wave] = m;
  }
  __syncthreads();
  for (int t = 0; t < T; ++t) {
    float* row = scores + t * Sp;
    const float a = wmax[t * 8 + 0], b = wmax[t * 8 + 1], c = wmax[t * 8 + 2], e = wmax[t * 8 + 3];
    const float ab = a > b ? a : b, ce = c > e ? c : e;
    const float m = ab > ce ? ab : ce;
    for (int i = tid; i < S; i += 256) row[i] = exp_nonpos(row[i] - m);
  }
  __syncthreads();
  if (wave < T) {
    const float* row = scores + wave * Sp;
    const int nchunks = (S + 3) >> 2;
    float sum = 0.0f;
    for (int c = lane; c < nchunks; c += 64)
      for (int j = 0; j < 4; ++j)
        if (c * 4 + j < S) sum = sum + row[c * 4 + j];
    sum = wave_sum(sum);
    if (lane == 0) wmax[wave * 8 + 4] = 127.0f / sum;
  }
  __syncthreads();
  for (int t = 0; t < T; ++t) {
    const float* row = scores + t * Sp;
    const float scale = wmax[t * 8 + 4];
    int8_t* po = probs_out != nullptr ? probs_out + (bh * T + t) * (long long)S : nullptr;
    for (int i = tid; i < S; i += 256) {
      const int8_t pq = (int8_t)(int)__builtin_rintf(row[i] * scale);
      probs[t * Sp + i] = pq;
      if (po != nullptr) po[i] = pq;
    }
  }
  __syncthreads();

  // ---- phase 3: ctx[t][n] = s8(alpha_pv * sum_s p[t][s] * v[s][n]); the lane owns columns cs*16 .. +15
  int acc[TQ][16];
#pragma unroll
  for (int t = 0; t < TQ; ++t)
#pragma unroll
    for (int c = 0; c < 16; ++c) acc[t][c] = 0;
  auto weigh_rows = [&](int base) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (base + u * 4 * RPW >= S) break;  // the same for every lane of the wave
      const int s = base + u * 4 * RPW + rs;
#pragma unroll
      for (int t = 0; t < TQ; ++t) {
        if (t >= T) continue;
        const int p = s < S ? (int)probs[t * Sp + s] : 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          const int x = vv[u][w];
          acc[t][4 * w + 0] += p * ((x << 24) >> 24);
          acc[t][4 * w + 1] += p * ((x << 16) >> 24);
          acc[t][4 * w + 2] += p * ((x << 8) >> 24);
          acc[t][4 * w + 3] += p * (x >> 24);
        }
      }
    }
  };
  if constexpr (NI > 0) {
    weigh_rows(wave * RPW);
  } else {
    for (int base = wave * RPW; base < S; base += 4 * RPW * U) {
      load_rows(base, vv, vb, vn);
      weigh_rows(base);
    }
  }
  // the row slots of a wave meet through shuffles, the four waves through LDS
#pragma unroll
  for (int t = 0; t < TQ; ++t)
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      int a = acc[t][c];
#pragma unroll
      for (int off = LPR; off < 64; off <<= 1) a += __shfl_xor(a, off, 64);
      acc[t][c] = a;
    }
  if (rs == 0) {
#pragma unroll
    for (int t = 0; t < TQ; ++t)
      if (t < T) {
#pragma unroll
        for (int c = 0; c < 16; ++c) red[(wave * T + t) * D + cs * 16 + c] = acc[t][c];
      }
  }
  __syncthreads();
  for (int idx = tid; idx < T * D; idx += 256) {
    const int t = idx / D, c = idx - t * D;
    if (!PART || c < dr) {
      const int sum = red[idx] + red[T * D + idx] + red[2 * T * D + idx] + red[3 * T * D + idx];
      ctx[(bh * T + t) * dr + c] = Epi<EPI_S8_SCALE>::apply(sum, 0.0f, alpha_pv);
    }
  }
}

// D = the head size in memory: any multiple of 16 up to 128 (sizes up to 64 run on four lanes per cache row, the
// others on eight)
bool decode_attn_supported(long long T, long long S, long long D) {
  return T >= 1 && T <= DA_MAX_T && S >= 1 && D >= 16 && D <= 128 && D % 16 == 0 &&
         decode_attn_lds(T, S, D <= 64 ? 64 : 128) <= DA_LDS_LIMIT;
}

int launch_decode_attn_s8(const int8_t* q, const int8_t* k_new, const int8_t* v_new, int8_t* k_buf, int8_t* v_buf,
                          const float* mask, int8_t* ctx, int8_t* probs_out, long long BH, long long T, long long D,
                          long long cap, long long S, long long heads, float alpha_qk, float alpha_pv,
                          hipStream_t stream, const int* s_dev) {
  // with s_dev the kernel reads the length from device memory; S is the largest value it may find there (the LDS
  // and the kernel variant are sized for it)
  if (BH == 0) return TI_OK;
  if (!decode_attn_supported(T, S, D))
    return fail(TI_ERR_INVALID_ARG, "decode_attn: unsupported shape (T=%lld S=%lld head_dim=%lld)", T, S, D);
  if (BH > 0x7fffffffLL) return fail(TI_ERR_INVALID_ARG, "decode_attn: too many (batch, head) pairs (%lld)", BH);
  const dim3 grid((unsigned)BH), block(256);
  const int lanes_d = D <= 64 ? 64 : 128;  // the kernel variant: bytes of a cache row that its lanes cover
  const size_t lds = (size_t)decode_attn_lds(T, S, lanes_d);
  // caches of at most 20 row groups per lane (640 positions at head size 128) with one or two query rows take
  // the variant that issues all loads up front
#define TI_DA(TQ, DD, NI)                                                                                              \
  do {                                                                                                                 \
    if (D == DD)                                                                                                       \
      hipLaunchKernelGGL((decode_attn_kernel<TQ, DD, NI, false>), grid, block, lds, stream, q, k_new, v_new, k_buf,    \
                         v_buf, mask, ctx, probs_out, (int)T, (int)S, cap, (int)heads, alpha_qk, alpha_pv, s_dev, (int)D); \
    else                                                                                                               \
      hipLaunchKernelGGL((decode_attn_kernel<TQ, DD, NI, true>), grid, block, lds, stream, q, k_new, v_new, k_buf,     \
                         v_buf, mask, ctx, probs_out, (int)T, (int)S, cap, (int)heads, alpha_qk, alpha_pv, s_dev, (int)D); \
  } while (0)
  const bool resident = T <= 2 && S <= 20 * 4 * (64 / (lanes_d / 16));
  if (lanes_d == 128) {
    if (T == 1) { if (resident) TI_DA(1, 128, 20); else TI_DA(1, 128, 0); }
    else if (T == 2) { if (resident) TI_DA(2, 128, 20); else TI_DA(2, 128, 0); }
    else TI_DA(4, 128, 0);
  } else {
    if (T == 1) { if (resident) TI_DA(1, 64, 20); else TI_DA(1, 64, 0); }
    else if (T == 2) { if (resident) TI_DA(2, 64, 20); else TI_DA(2, 64, 0); }
    else TI_DA(4, 64, 0);
  }
#undef TI_DA
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "decode_attn launch: %s", hipGetErrorString(e));
  return TI_OK;
}

}  // namespace ti

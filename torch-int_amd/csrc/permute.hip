// int8 layout changes of the attention block, as single coalesced passes:
//   permute_0213:  [B, X, Y, D] -> [B, Y, X, D]   (rows of D bytes move intact: the
//                  head split / merge  view(B,T,H,d).transpose(1,2).contiguous())
//   transpose_last2: [B, R, C] -> [B, C, R]        (byte transpose: V -> V^T)
//   kv_append:     kbuf[bh, S + t, :] = knew[bh, t, :] and the same for V, one launch for both caches
#include "ti_common.h"

namespace ti {

// one thread per 16-byte chunk of the output; D % 16 == 0, 16-byte aligned pointers
__global__ __launch_bounds__(256) void permute_0213_v16_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst,
                                                               int X, int Y, int chunks, long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % chunks);
  long long row = i / chunks;            // output row index: (b, y, x)
  const int x = (int)(row % X);
  row /= X;
  const int y = (int)(row % Y);
  const long long b = row / Y;
  dst[i] = src[((b * X + x) * Y + y) * chunks + c];
}

__global__ __launch_bounds__(256) void permute_0213_bytes_kernel(const int8_t* __restrict__ src,
                                                                 int8_t* __restrict__ dst, int X, int Y, int D,
                                                                 long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % D);
  long long row = i / D;
  const int x = (int)(row % X);
  row /= X;
  const int y = (int)(row % Y);
  const long long b = row / Y;
  dst[i] = src[((b * X + x) * Y + y) * D + c];
}

// 64x64 byte tiles through LDS; any R, C
__global__ __launch_bounds__(256) void transpose_last2_kernel(const int8_t* __restrict__ src, int8_t* __restrict__ dst,
                                                              int R, int C) {
  __shared__ int8_t tile[64][64 + 4];
  const long long base = (long long)blockIdx.z * R * C;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int t = threadIdx.x;
  // load: thread t covers row t/4, bytes (t%4)*16 .. +15
  {
    const int r = r0 + (t >> 2), cb = c0 + (t & 3) * 16;
    if (r < R) {
      const int8_t* s = src + base + (long long)r * C + cb;
      if (cb + 16 <= C && ((reinterpret_cast<uintptr_t>(s) & 15) == 0)) {
        v4i v = *reinterpret_cast<const v4i*>(s);
        int8_t b[16];
        __builtin_memcpy(b, &v, 16);
#pragma unroll
        for (int j = 0; j < 16; ++j) tile[t >> 2][(t & 3) * 16 + j] = b[j];
      } else {
        for (int j = 0; j < 16; ++j)
          if (cb + j < C) tile[t >> 2][(t & 3) * 16 + j] = s[j];
      }
    }
  }
  __syncthreads();
  // store: thread t covers output row (column of the tile) t/4, bytes (t%4)*16 .. +15 along R
  {
    const int c = c0 + (t >> 2), rb = r0 + (t & 3) * 16;
    if (c < C) {
      int8_t b[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) b[j] = tile[(t & 3) * 16 + j][t >> 2];
      int8_t* d = dst + base + (long long)c * R + rb;
      if (rb + 16 <= R && ((reinterpret_cast<uintptr_t>(d) & 15) == 0)) {
        v4i v;
        __builtin_memcpy(&v, b, 16);
        *reinterpret_cast<v4i*>(d) = v;
      } else {
        for (int j = 0; j < 16; ++j)
          if (rb + j < R) d[j] = b[j];
      }
    }
  }
}

// rows of D bytes: row r = (bh, t) of the new tokens goes to row (bh * cap + S + t) of the cache buffer;
// blockIdx.y selects K (0) or V (1).  CH = bytes moved per thread (16 when D and the pointers allow, else 1).
template <int CH>
__global__ __launch_bounds__(256) void kv_append_kernel(const int8_t* __restrict__ knew, const int8_t* __restrict__ vnew,
                                                        int8_t* __restrict__ kbuf, int8_t* __restrict__ vbuf, int T,
                                                        int per_row, long long cap, long long S, long long total) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int c = (int)(i % per_row);
  const long long row = i / per_row;
  const long long bh = row / T, t = row % T;
  const int8_t* src = (blockIdx.y ? vnew : knew) + (row * per_row + c) * CH;
  int8_t* dst = (blockIdx.y ? vbuf : kbuf) + (((bh * cap + S + t) * per_row) + c) * CH;
  if (CH == 16)
    *reinterpret_cast<v4i*>(dst) = *reinterpret_cast<const v4i*>(src);
  else
    *dst = *src;
}

int launch_kv_append_s8(const int8_t* knew, const int8_t* vnew, int8_t* kbuf, int8_t* vbuf, long long BH, long long T,
                        long long D, long long cap, long long S, hipStream_t stream) {
  const long long bytes = BH * T * D;
  if (bytes == 0) return TI_OK;
  const uintptr_t all = reinterpret_cast<uintptr_t>(knew) | reinterpret_cast<uintptr_t>(vnew) |
                        reinterpret_cast<uintptr_t>(kbuf) | reinterpret_cast<uintptr_t>(vbuf);
  if (D % 16 == 0 && (all & 15) == 0) {
    const long long total = bytes / 16;
    hipLaunchKernelGGL(kv_append_kernel<16>, dim3((unsigned)((total + 255) / 256), 2), dim3(256), 0, stream, knew, vnew,
                       kbuf, vbuf, (int)T, (int)(D / 16), cap, S, total);
  } else {
    hipLaunchKernelGGL(kv_append_kernel<1>, dim3((unsigned)((bytes + 255) / 256), 2), dim3(256), 0, stream, knew, vnew,
                       kbuf, vbuf, (int)T, (int)D, cap, S, bytes);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "kv_append launch: %s", hipGetErrorString(e));
  return TI_OK;
}

int launch_permute_0213_s8(const int8_t* src, int8_t* dst, long long B, long long X, long long Y, long long D,
                           hipStream_t stream) {
  const long long bytes = B * X * Y * D;
  if (bytes == 0) return TI_OK;
  const bool v16 = (D % 16 == 0) && ((reinterpret_cast<uintptr_t>(src) & 15) == 0) &&
                   ((reinterpret_cast<uintptr_t>(dst) & 15) == 0);
  if (v16) {
    const long long total = bytes / 16;
    hipLaunchKernelGGL(permute_0213_v16_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       reinterpret_cast<const v4i*>(src), reinterpret_cast<v4i*>(dst), (int)X, (int)Y, (int)(D / 16),
                       total);
  } else {
    hipLaunchKernelGGL(permute_0213_bytes_kernel, dim3((unsigned)((bytes + 255) / 256)), dim3(256), 0, stream, src,
                       dst, (int)X, (int)Y, (int)D, bytes);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "permute launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// 64x64 tiles of a matrix with R % 4 == 0 and C % 16 == 0 (edge tiles are cut off at whole 16-byte chunks of a source
// row and whole dwords of an output row): a thread owns one 4x4 block of bytes.  The
// tile goes into the LDS as dwords (row pitch 17 dwords); thread (a, b) reads the dwords of rows 4a .. 4a+3 at
// dword column b, transposes the 4x4 bytes in registers with four + four v_perm_b32 and stores four dwords: bytes
// 4a .. 4a+3 of the output rows 4b .. 4b+3.  a runs fastest over the lanes, so a wave writes 64 contiguous bytes of
// each of four output rows per store instruction.  (The byte-by-byte kernel above makes 32 LDS accesses per 16
// bytes; this one makes 8.)
__global__ __launch_bounds__(256) void transpose_last2_tiles_kernel(const int8_t* __restrict__ src,
                                                                    int8_t* __restrict__ dst, int R, int C) {
  __shared__ unsigned tile[64][17];
  const long long base = (long long)blockIdx.z * R * C;
  const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
  const int t = threadIdx.x;
  {
    const int r = t >> 2, q = t & 3;
    if (r0 + r < R && c0 + q * 16 < C) {
      const v4i v = *reinterpret_cast<const v4i*>(src + base + (long long)(r0 + r) * C + c0 + q * 16);
#pragma unroll
      for (int j = 0; j < 4; ++j) tile[r][4 * q + j] = (unsigned)v[j];
    }
  }
  __syncthreads();
  const int a = t & 15, b = t >> 4;
  if (r0 + 4 * a >= R || c0 + 4 * b >= C) return;  // after the only barrier
  const unsigned w0 = tile[4 * a][b], w1 = tile[4 * a + 1][b], w2 = tile[4 * a + 2][b], w3 = tile[4 * a + 3][b];
  // v_perm_b32(hi, lo, sel): result byte i = byte sel[i] of the eight bytes {lo: 0..3, hi: 4..7}
  const unsigned t0 = __builtin_amdgcn_perm(w1, w0, 0x05010400u);  // w0.0 w1.0 w0.1 w1.1
  const unsigned t1 = __builtin_amdgcn_perm(w1, w0, 0x07030602u);  // w0.2 w1.2 w0.3 w1.3
  const unsigned t2 = __builtin_amdgcn_perm(w3, w2, 0x05010400u);
  const unsigned t3 = __builtin_amdgcn_perm(w3, w2, 0x07030602u);
  const unsigned o[4] = {__builtin_amdgcn_perm(t2, t0, 0x05040100u), __builtin_amdgcn_perm(t2, t0, 0x07060302u),
                         __builtin_amdgcn_perm(t3, t1, 0x05040100u), __builtin_amdgcn_perm(t3, t1, 0x07060302u)};
#pragma unroll
  for (int k = 0; k < 4; ++k)
    *reinterpret_cast<unsigned*>(dst + base + (long long)(c0 + 4 * b + k) * R + r0 + 4 * a) = o[k];
}

// The same with 128x128 tiles (R % 128 == 0, C % 128 == 0): whole 128-byte lines are read and written (eight lanes
// fetch one row of the tile, 32 lanes store 128 contiguous bytes of an output row), four 4x4 blocks per thread.
__global__ __launch_bounds__(256) void transpose_last2_tiles128_kernel(const int8_t* __restrict__ src,
                                                                       int8_t* __restrict__ dst, int R, int C) {
  __shared__ unsigned tile[128][33];
  const long long base = (long long)blockIdx.z * R * C;
  const int r0 = blockIdx.y * 128, c0 = blockIdx.x * 128;
  const int t = threadIdx.x;
  {
    const int q = t & 7;
    v4i v[4];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass)
      v[pass] = *reinterpret_cast<const v4i*>(src + base + (long long)(r0 + (t >> 3) + 32 * pass) * C + c0 + q * 16);
#pragma unroll
    for (int pass = 0; pass < 4; ++pass)
#pragma unroll
      for (int j = 0; j < 4; ++j) tile[(t >> 3) + 32 * pass][4 * q + j] = (unsigned)v[pass][j];
  }
  __syncthreads();
  const int a = t & 31;
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int b = (t >> 5) + 8 * pass;
    const unsigned w0 = tile[4 * a][b], w1 = tile[4 * a + 1][b], w2 = tile[4 * a + 2][b], w3 = tile[4 * a + 3][b];
    const unsigned t0 = __builtin_amdgcn_perm(w1, w0, 0x05010400u), t1 = __builtin_amdgcn_perm(w1, w0, 0x07030602u);
    const unsigned t2 = __builtin_amdgcn_perm(w3, w2, 0x05010400u), t3 = __builtin_amdgcn_perm(w3, w2, 0x07030602u);
    const unsigned o[4] = {__builtin_amdgcn_perm(t2, t0, 0x05040100u), __builtin_amdgcn_perm(t2, t0, 0x07060302u),
                           __builtin_amdgcn_perm(t3, t1, 0x05040100u), __builtin_amdgcn_perm(t3, t1, 0x07060302u)};
#pragma unroll
    for (int k = 0; k < 4; ++k)
      *reinterpret_cast<unsigned*>(dst + base + (long long)(c0 + 4 * b + k) * R + r0 + 4 * a) = o[k];
  }
}

int launch_transpose_last2_s8(const int8_t* src, int8_t* dst, long long B, long long R, long long C,
                              hipStream_t stream) {
  if (B * R * C == 0) return TI_OK;
  if (R % 128 == 0 && C % 128 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(dst) & 3) == 0) {
    dim3 grid128((unsigned)(C / 128), (unsigned)(R / 128), (unsigned)B);
    hipLaunchKernelGGL(transpose_last2_tiles128_kernel, grid128, dim3(256), 0, stream, src, dst, (int)R, (int)C);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "transpose launch: %s", hipGetErrorString(e));
    return TI_OK;
  }
  dim3 grid((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64), (unsigned)B);
  if (R % 4 == 0 && C % 16 == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0 &&
      (reinterpret_cast<uintptr_t>(dst) & 3) == 0)
    hipLaunchKernelGGL(transpose_last2_tiles_kernel, grid, dim3(256), 0, stream, src, dst, (int)R, (int)C);
  else
    hipLaunchKernelGGL(transpose_last2_kernel, grid, dim3(256), 0, stream, src, dst, (int)R, (int)C);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "transpose launch: %s", hipGetErrorString(e));
  return TI_OK;
}

}  // namespace ti

// INT8 x INT8 -> INT32 "NT" GEMM (C = A . B^T) for gfx950 with fused fp32
// epilogues.  One mainloop serves the W8A8 linears and the batched attention
// products; the epilogue kind is a template parameter.
//
// Mainloop (gemm_tile_kernel):
//   - a workgroup owns a BM x BN output tile and walks K in steps of 128 bytes;
//   - A (BM x 128) and B (BN x 128) panels are staged in LDS, two stages deep;
//     rows are 128 bytes = eight 16-byte chunks, and chunk c of row r is stored
//     at chunk position c ^ ((r >> 1) & 7) so that both the 16-byte row-wise
//     stores and the column-wise 16-byte fragment reads spread over all banks;
//   - each wavefront computes a (BM/WAVES_M) x (BN/WAVES_N) sub-tile out of
//     32x32 blocks with v_mfma_i32_32x32x32_i8 (K = 32 per instruction, 16
//     bytes of each operand per lane);
//   - SWAP selects which matrix feeds the "row" operand of the MFMA.  With
//     SWAP the weight rows do, their order inside each 32-row block is
//     permuted when the panel is written to LDS, and a lane ends up holding 16
//     consecutive output columns of one output row (16-byte s8 stores).
//     Without SWAP a lane holds one output column of 16 rows and the 32 lanes
//     of a half-wave store 128 contiguous bytes of 32-bit results.
#pragma once
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <type_traits>
#include "ti_common.h"

namespace ti {

static constexpr int BK = 128;        // bytes of K per mainloop step
static constexpr int CHUNKS = BK / 16;  // 16-byte chunks per LDS row

// position of a logical tile row inside the LDS panel
template <bool PERMUTE>
__device__ __forceinline__ int phys_row(int r) {
  if (!PERMUTE) return r;
  // inside each block of 32 rows: logical 16h + 4q + j  ->  MFMA row 8q + 4h + j
  return (r & ~31) | ((r & 12) << 1) | ((r & 16) >> 2) | (r & 3);
}

__device__ __forceinline__ int lds_off(int prow, int chunk) {
  return prow * BK + (((chunk ^ (prow >> 1)) & 7) << 4);
}

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int KIND_, bool SWAP_>
struct TileCfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KIND = KIND_;
  static constexpr bool SWAP = SWAP_;
  static constexpr int NT = WAVES_M * WAVES_N * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int A_SLOTS = BM * CHUNKS / NT, B_SLOTS = BN * CHUNKS / NT;
  static constexpr int STAGE_BYTES = (BM + BN) * BK;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be made of 32x32 blocks");
  static_assert((BM * CHUNKS) % NT == 0 && (BN * CHUNKS) % NT == 0, "panel must split evenly over threads");
};

// Maps the linear workgroup id to an output tile so that (i) the workgroups
// that share an XCD (ids congruent mod 8 are dispatched to the same XCD, each
// with a private L2) own a contiguous run of tiles and (ii) consecutive tiles
// walk down GROUP rows of tiles before moving to the next column, which keeps
// the A rows and B rows a run touches small enough to stay in that L2.
__device__ __forceinline__ void tile_of_workgroup(int pid, int tiles_m, int tiles_n, int& tm, int& tn, int GROUP = 8) {
  const int total = tiles_m * tiles_n;
  const int NXCD = 8;
  int per = (total + NXCD - 1) / NXCD;
  int tall = total % NXCD;
  if (tall == 0) tall = NXCD;
  int xcd = pid % NXCD, local = pid / NXCD;
  int id = (xcd < tall) ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
  int width = GROUP * tiles_n;
  int g = id / width;
  int first = g * GROUP;
  int gsz = tiles_m - first < GROUP ? tiles_m - first : GROUP;
  int in = id - g * width;
  tm = first + in % gsz;
  tn = in / gsz;
}

// 4x4 transpose across the four lanes of a quad: lane b (0..3) enters with x[k] = its own element k
// and leaves with x[k] = element b of lane k.  Two exchange rounds (partner lane ^ 2, then lane ^ 1)
// over the DPP quad permutes; every lane of the wave must take part.
__device__ __forceinline__ void quad_transpose(int (&x)[4], int lane) {
  const bool hi = lane & 2;
  int s0 = hi ? x[0] : x[2];
  int s1 = hi ? x[1] : x[3];
  int r0 = __builtin_amdgcn_mov_dpp(s0, 0x4E, 0xf, 0xf, true);  // quad_perm [2,3,0,1]
  int r1 = __builtin_amdgcn_mov_dpp(s1, 0x4E, 0xf, 0xf, true);
  if (hi) {
    x[0] = r0;
    x[1] = r1;
  } else {
    x[2] = r0;
    x[3] = r1;
  }
  const bool odd = lane & 1;
  s0 = odd ? x[0] : x[1];
  s1 = odd ? x[2] : x[3];
  r0 = __builtin_amdgcn_mov_dpp(s0, 0xB1, 0xf, 0xf, true);  // quad_perm [1,0,3,2]
  r1 = __builtin_amdgcn_mov_dpp(s1, 0xB1, 0xf, 0xf, true);
  if (odd) {
    x[0] = r0;
    x[2] = r1;
  } else {
    x[1] = r0;
    x[3] = r1;
  }
}

// four int8 values (already clamped to [-128, 127], held in ints) as one dword, first value in the low byte
__device__ __forceinline__ int pack_s8x4_ints(int a, int b, int c, int d) {
  const unsigned lo = __builtin_amdgcn_perm((unsigned)b, (unsigned)a, 0x0c0c0400u);  // a.byte0 | b.byte0 << 8
  const unsigned hi = __builtin_amdgcn_perm((unsigned)d, (unsigned)c, 0x0c0c0400u);
  return (int)__builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// Applies the epilogue to a wavefront's accumulators and stores them.
template <class Cfg>
__device__ __forceinline__ void store_tile(v16i (&acc)[Cfg::TM][Cfg::TN], const GemmParams& p, int batch, int m0,
                                           int n0, int wave_m, int wave_n, int lane) {
  using E = Epi<Cfg::KIND>;
  using Out = typename E::Out;
  using BiasT = typename E::Bias;
  constexpr int TM = Cfg::TM, TN = Cfg::TN;
  constexpr bool SWAP = Cfg::SWAP;
  const int M = p.M, N = p.N;
  const int frow = lane & 31;
  Out* __restrict__ C = reinterpret_cast<Out*>(p.C) + (long long)batch * p.strideC;
  const BiasT* __restrict__ bias = reinterpret_cast<const BiasT*>(p.bias);
  const float alpha = p.alpha, beta = p.beta;
  const int half = lane >> 5;
  if (SWAP) {
    // lane owns row m = .. + (lane & 31) and 16 consecutive columns per block
    constexpr int VEC = 16 / sizeof(Out);  // outputs per 16-byte store
    const bool vec_ok = (N % VEC) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
    const bool bias_al = (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
    if constexpr (sizeof(Out) == 1 && TN == 2 && !E::kAccumulate) {
      // Wave tiles two blocks wide whose 64 columns lie inside the matrix: a row's 64 output bytes sit in two
      // lanes (column halves) x two blocks.  v_permlane16_swap between the two blocks' packed dwords moves
      // block 1 of rows 0..15 into the lanes that held block 0 of rows 16..31 and the reverse, after which one
      // store instruction writes 16 rows x 64 contiguous bytes instead of 32 rows x 32.
      const int nw = n0 + wave_n * Cfg::WTN;
      if (vec_ok && (!E::kHasBias || bias_al) && nw + 64 <= N) {
        v4i braw[2] = {v4i{0, 0, 0, 0}, v4i{0, 0, 0, 0}};
        if (E::kHasBias) {
#pragma unroll
          for (int j = 0; j < 2; ++j) braw[j] = *reinterpret_cast<const v4i*>(bias + nw + j * 32 + half * 16);
        }
        const int col = nw + ((lane >> 4) & 1) * 32 + half * 16;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          int w[2][4];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            BiasT bv[16];
            __builtin_memcpy(bv, &braw[j], 16);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              int o[4];
#pragma unroll
              for (int k = 0; k < 4; ++k)
                o[k] = (int)E::apply(acc[i][j][4 * q + k], E::bias_term(bv[4 * q + k], beta), alpha);
              w[j][q] = pack_s8x4_ints(o[0], o[1], o[2], o[3]);
            }
          }
          v4i lo, hi;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            auto sw = __builtin_amdgcn_permlane16_swap((unsigned)w[0][q], (unsigned)w[1][q], false, false);
            lo[q] = (int)sw[0];  // rows 0..15 of the block row: blocks 0 | 1 by lane bit 4
            hi[q] = (int)sw[1];  // rows 16..31
          }
          const int mlo = m0 + wave_m * Cfg::WTM + i * 32 + (lane & 15);
          if (mlo < M) *reinterpret_cast<v4i*>(C + out_index(p, mlo, col)) = lo;
          if (mlo + 16 < M) *reinterpret_cast<v4i*>(C + out_index(p, mlo + 16, col)) = hi;
        }
        return;
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int nb = n0 + wave_n * Cfg::WTN + j * 32 + half * 16;
      float bt[16];
      if (E::kHasBias && vec_ok && bias_al && nb + 16 <= N) {
        // 16 consecutive bias values in one (int8) or four (32-bit) 16-byte loads
        BiasT bv[16];
        constexpr int BV = 16 / sizeof(BiasT);
#pragma unroll
        for (int q = 0; q < 16 / BV; ++q) {
          v4i w = *reinterpret_cast<const v4i*>(bias + nb + q * BV);
          __builtin_memcpy(&bv[q * BV], &w, 16);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) bt[v] = E::bias_term(bv[v], beta);
      } else {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          BiasT bv = BiasT(0);
          if (E::kHasBias && nb + v < N) bv = bias[nb + v];
          bt[v] = E::bias_term(bv, beta);
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = m0 + wave_m * Cfg::WTM + i * 32 + frow;
        if (m >= M) continue;
        Out* dst = C + out_index(p, m, nb);
        if (vec_ok && nb + 16 <= N) {
          if constexpr (sizeof(Out) == 1) {
            v4i w;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              unsigned b0 = (unsigned char)E::apply(acc[i][j][4 * q + 0], bt[4 * q + 0], alpha);
              unsigned b1 = (unsigned char)E::apply(acc[i][j][4 * q + 1], bt[4 * q + 1], alpha);
              unsigned b2 = (unsigned char)E::apply(acc[i][j][4 * q + 2], bt[4 * q + 2], alpha);
              unsigned b3 = (unsigned char)E::apply(acc[i][j][4 * q + 3], bt[4 * q + 3], alpha);
              w[q] = (int)(b0 | (b1 << 8) | (b2 << 16) | (b3 << 24));
            }
            *reinterpret_cast<v4i*>(dst) = w;
          } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              Out o0 = merge_old<E>(E::apply(acc[i][j][4 * q + 0], bt[4 * q + 0], alpha), dst + 4 * q + 0);
              Out o1 = merge_old<E>(E::apply(acc[i][j][4 * q + 1], bt[4 * q + 1], alpha), dst + 4 * q + 1);
              Out o2 = merge_old<E>(E::apply(acc[i][j][4 * q + 2], bt[4 * q + 2], alpha), dst + 4 * q + 2);
              Out o3 = merge_old<E>(E::apply(acc[i][j][4 * q + 3], bt[4 * q + 3], alpha), dst + 4 * q + 3);
              v4i w = {__builtin_bit_cast(int, o0), __builtin_bit_cast(int, o1),
                       __builtin_bit_cast(int, o2), __builtin_bit_cast(int, o3)};
              *reinterpret_cast<v4i*>(dst + 4 * q) = w;
            }
          }
        } else {
#pragma unroll
          for (int v = 0; v < 16; ++v)
            if (nb + v < N) dst[v] = merge_old<E>(E::apply(acc[i][j][v], bt[v], alpha), dst + v);
        }
      }
    }
  } else {
    // lane owns column n = .. + (lane & 31) and rows 8*(v/4) + 4*half + v%4 of each block
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wave_n * Cfg::WTN + j * 32 + frow;
      BiasT bv = BiasT(0);
      if (E::kHasBias && n < N) bv = bias[n];
      const float bt = E::bias_term(bv, beta);
      // 32-bit outputs of a block that lies inside the matrix: the lanes of a quad swap their four
      // rows x four columns, so that a lane ends with four consecutive columns of one row and a store
      // instruction writes eight whole 128-byte lines instead of two
      const int nq = n0 + wave_n * Cfg::WTN + j * 32;  // first column of the block
      if constexpr (sizeof(Out) == 4) {
       // (short K, e.g. Q.K^T with K = head size: the epilogue is most of the kernel and the plain stores,
       // which need no lane exchanges, are faster)
       if (p.K >= 1024 && (N & 3) == 0 && nq + 32 <= N && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            int x[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) x[k] = __builtin_bit_cast(int, E::apply(acc[i][j][4 * q + k], bt, alpha));
            quad_transpose(x, lane);
            const int m = m0 + wave_m * Cfg::WTM + i * 32 + 8 * q + 4 * half + (lane & 3);
            if (m < M) {
              Out* at = C + ((long long)m * N + nq + (frow & ~3));
              if constexpr (E::kAccumulate) {
                const v4i old = *reinterpret_cast<const v4i*>(at);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                  const int was = old[k], add = x[k];  // plain values: the casts below must not see vector elements
                  x[k] = __builtin_bit_cast(int, __builtin_bit_cast(Out, was) + __builtin_bit_cast(Out, add));
                }
              }
              v4i w = {x[0], x[1], x[2], x[3]};
              *reinterpret_cast<v4i*>(at) = w;
            }
          }
        }
        continue;
       }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wave_m * Cfg::WTM + i * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
          if (m < M && n < N) {
            Out fresh = E::apply(acc[i][j][v], bt, alpha);
            // plain row-major only: head-major output exists for 8-bit outputs, which take the branch above
            Out* at = C + ((long long)m * N + n);
            if constexpr (E::kAccumulate) fresh = *at + fresh;
            *at = fresh;
          }
        }
      }
    }
  }
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void gemm_tile_kernel(GemmParams p, int tiles_m, int tiles_n) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, NT = Cfg::NT, TM = Cfg::TM, TN = Cfg::TN;
  constexpr bool SWAP = Cfg::SWAP;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
  int tile_m, tile_n;
  tile_of_workgroup(blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int M = p.M, N = p.N, K = p.K;
  const int8_t* __restrict__ A = p.A + (long long)blockIdx.z * p.strideA;
  const int8_t* __restrict__ B = p.B + (long long)blockIdx.z * p.strideB;

  // ---- global -> LDS assignment: slot i of thread t moves chunk (t & 7) of row i*NT/8 + t/8
  const int ld_chunk = tid & 7;
  const int ld_row = tid >> 3;
  constexpr int ROWS_PER_SLOT = NT / CHUNKS;
  int a_goff[Cfg::A_SLOTS], b_goff[Cfg::B_SLOTS];
  int a_soff[Cfg::A_SLOTS], b_soff[Cfg::B_SLOTS];
#pragma unroll
  for (int i = 0; i < Cfg::A_SLOTS; ++i) {
    int r = i * ROWS_PER_SLOT + ld_row;
    int gr = m0 + r < M ? m0 + r : M - 1;  // rows past the edge re-read the last row; never stored
    a_goff[i] = gr * K + ld_chunk * 16;
    a_soff[i] = lds_off(phys_row<false>(r), ld_chunk);
  }
#pragma unroll
  for (int i = 0; i < Cfg::B_SLOTS; ++i) {
    int r = i * ROWS_PER_SLOT + ld_row;
    int gr = n0 + r < N ? n0 + r : N - 1;
    b_goff[i] = gr * K + ld_chunk * 16;
    b_soff[i] = BM * BK + lds_off(phys_row<SWAP>(r), ld_chunk);
  }

  v4i a_reg[Cfg::A_SLOTS], b_reg[Cfg::B_SLOTS];
  auto load_global = [&](int kt) {
    const int kbase = kt * BK;
    const bool ok = kbase + ld_chunk * 16 < K;  // K % 16 == 0: a chunk is all in or all out
#pragma unroll
    for (int i = 0; i < Cfg::A_SLOTS; ++i) {
      v4i z = {0, 0, 0, 0};
      a_reg[i] = ok ? *reinterpret_cast<const v4i*>(A + (size_t)(unsigned)a_goff[i] + kbase) : z;
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_SLOTS; ++i) {
      v4i z = {0, 0, 0, 0};
      b_reg[i] = ok ? *reinterpret_cast<const v4i*>(B + (size_t)(unsigned)b_goff[i] + kbase) : z;
    }
  };
  auto store_lds = [&](int stage) {
    char* s = smem + stage * Cfg::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < Cfg::A_SLOTS; ++i) *reinterpret_cast<v4i*>(s + a_soff[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < Cfg::B_SLOTS; ++i) *reinterpret_cast<v4i*>(s + b_soff[i]) = b_reg[i];
  };

  // ---- fragment addressing: lane reads row (lane & 31), chunk 2*ks + (lane >> 5)
  const int frow = lane & 31;
  const int fkey = ((lane >> 5) ^ (frow >> 1)) & 7;  // chunk position for ks = 0
  const int a_frag = (wave_m * Cfg::WTM + frow) * BK + (fkey << 4);
  const int b_frag = BM * BK + (wave_n * Cfg::WTN + frow) * BK + (fkey << 4);

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;

  auto compute = [&](int stage) {
    const char* s = smem + stage * Cfg::STAGE_BYTES;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      v4i fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[i] = *reinterpret_cast<const v4i*>(s + ((a_frag ^ (ks << 5)) + i * 32 * BK));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[j] = *reinterpret_cast<const v4i*>(s + ((b_frag ^ (ks << 5)) + j * 32 * BK));
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0)
                           : __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
  };

  const int KT = (K + BK - 1) / BK;
  if (KT > 0) {
    load_global(0);
    store_lds(0);
  }
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = kt + 1 < KT;
    if (more) load_global(kt + 1);
    compute(kt & 1);
    if (more) store_lds((kt + 1) & 1);
    __syncthreads();
  }

  store_tile<Cfg>(acc, p, blockIdx.z, m0, n0, wave_m, wave_n, lane);
}

// ---------------------------------------------------------------------------
// Pipelined, persistent mainloop for K % 64 == 0.
//
// Global -> LDS copies bypass registers (global_load_lds_dwordx4), K advances
// 64 bytes per step and STAGES LDS stages keep STAGES-1 steps of copies in
// flight.  A workgroup walks a list of output tiles (blockIdx.x, +gridDim.x,
// ...); the copy stream runs STAGES-1 steps ahead of the multiply stream and
// crosses tile boundaries, so the epilogue of one tile overlaps the first
// copies of the next.
//
// LDS stage = [A panel BM x 64][B panel BN x 64].  A row is four 16-byte
// chunks; chunk c of panel row r sits at chunk position c ^ ((r >> 2) & 3).
// One wavefront copy instruction fills 1 KiB of LDS = 16 consecutive panel
// rows, lane l landing at row l/4, position l%4; the swizzle (and, with SWAP,
// the row permutation of the B panel) is applied by choosing which global
// chunk each lane fetches.
//
// One K step of a wavefront: read the second half (k 32..63) of the step's
// fragments while the first half multiplies; then wait until this wave's own
// copies for the next step have landed (s_waitcnt vmcnt), pass one workgroup
// barrier (all copies visible; every wave done with the stage that is about
// to be refilled), issue the copies STAGES-1 steps ahead, read the first half
// of the next step's fragments and multiply the second half of this one.
#define TI_GLOBAL_AS __attribute__((address_space(1)))
#define TI_LDS_AS __attribute__((address_space(3)))

static constexpr int PBK = 64;

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_, int KIND_, bool SWAP_, int MIN_WAVES_ = 2>
struct PipeCfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KIND = KIND_;
  static constexpr int MIN_WAVES = MIN_WAVES_;  // waves per SIMD the register budget is sized for
  static constexpr int STAGES = STAGES_;
  static constexpr bool SWAP = SWAP_;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int STAGE_BYTES = (BM + BN) * PBK;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  static constexpr int COPIES = (BM + BN) / 16 / NWAVES;  // copy instructions per wave per step
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be made of 32x32 blocks");
  static_assert((BM + BN) % (16 * NWAVES) == 0 && BM % 16 == 0, "panels must split into 1 KiB copies per wave");
  static_assert(LDS_BYTES <= 160 * 1024 && STAGES >= 3, "LDS budget");
};

template <int N>
__device__ __forceinline__ void wait_copies_then_barrier() {
  // "memory": no LDS access may be moved across this point by the compiler
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// items = tiles_m * tiles_n * batch work items; item -> (batch, tile) with the tile index minor.
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, Cfg::MIN_WAVES) void gemm_pipe_kernel(GemmParams p, int tiles_m, int tiles_n, int items) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, COPIES = Cfg::COPIES;
  constexpr int S = Cfg::STAGES;
  constexpr bool SWAP = Cfg::SWAP;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
  const int M = p.M, N = p.N, K = p.K;
  const int KT = K / PBK;
  const int tiles = tiles_m * tiles_n;
  const int first = blockIdx.x, stride = gridDim.x;
  const int my_items = (items - first + stride - 1) / stride;  // >= 1 (grid <= items)
  const int G = my_items * KT;                                  // K steps this workgroup multiplies

  // ---- copy stream: copy j of this wave fills stage bytes [(wave*COPIES + j) * 1024, +1024)
  const TI_GLOBAL_AS int8_t* src[COPIES];
  // item -> (batch, tile of the batch).  With p.group_batches (few tiles per batch, batches a multiple of 8) all
  // tiles of a batch go to workgroups of one XCD (ids congruent mod 8), next to one another, so that the batch's
  // B operand (V^T of a head in P.V) is fetched into one L2 instead of into as many as the batch has tiles.
  auto decode_item = [&](int item, int& b, int& t) {
    if (p.group_batches) {
      const int l = item >> 3, q = l / tiles;
      b = q * 8 + (item & 7);
      t = l - q * tiles;
    } else {
      b = item / tiles;
      t = item - b * tiles;
    }
  };
  auto set_copy_item = [&](int item) {
    int b, t;
    decode_item(item, b, t);
    int tile_m, tile_n;
    tile_of_workgroup(t, tiles_m, tiles_n, tile_m, tile_n, p.band);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int8_t* A = a_of_batch(p, b);
    const int8_t* B = b_of_batch(p, b);
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      const int slab = wave * COPIES + j;        // 16-row slab inside [A panel | B panel]
      const int prow = slab * 16 + (lane >> 2);  // panel row this lane fills (A rows first)
      const int pos = lane & 3;
      if (slab * 16 < BM) {
        const int chunk = pos ^ ((prow >> 2) & 3);
        const int gr = m0 + prow < M ? m0 + prow : M - 1;  // edge rows re-read the last row; never stored
        src[j] = (const TI_GLOBAL_AS int8_t*)(A + (size_t)gr * p.lda + chunk * 16);
      } else {
        const int br = prow - BM;
        const int chunk = pos ^ ((br >> 2) & 3);
        int lr = br;
        if (SWAP) lr = (br & ~31) | ((br & 4) << 2) | ((br & 24) >> 1) | (br & 3);  // MFMA row 8q+4h+j -> 16h+4q+j
        const int gr = n0 + lr < N ? n0 + lr : N - 1;
        src[j] = (const TI_GLOBAL_AS int8_t*)(B + (size_t)gr * p.ldb + chunk * 16);
      }
    }
  };
  // Copy cursor: work item, K step inside it, global step.  When it runs past the last
  // item it keeps re-copying the final K step into the stage that is free anyway, so
  // that exactly S-1 steps of copies are in flight at every step and the wait counts
  // below never change.
  int c_item = first, c_kt = 0, c_g = 0, c_live = 1;
  auto issue_copies = [&]() {
    TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + (c_g % S) * Cfg::STAGE_BYTES + wave * COPIES * 1024;
#pragma unroll
    for (int j = 0; j < COPIES; ++j)
      __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[j] + c_kt * PBK), (TI_LDS_AS void*)(dst + j * 1024),
                                       16, 0, 0);
    c_kt += c_live;
    ++c_g;
  };
  auto advance_copy_item = [&]() {  // call when c_live && c_kt == KT
    if (c_g < G) {
      c_kt = 0;
      c_item += stride;
      set_copy_item(c_item);
    } else {
      c_live = 0;
      c_kt = KT - 1;
    }
  };

  // ---- fragment addressing: lane reads panel row (lane & 31), chunk 2*ks + (lane >> 5)
  const int frow = lane & 31;
  const int fpos = ((lane >> 5) ^ (frow >> 2)) & 3;  // chunk position for ks = 0
  const int a_frag = (wave_m * Cfg::WTM + frow) * PBK + (fpos << 4);
  const int b_frag = BM * PBK + (wave_n * Cfg::WTN + frow) * PBK + (fpos << 4);

  v16i acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
  };
  auto read_frags = [&](int g, int ks, v4i (&fa)[TM], v4i (&fb)[TN]) {
    const char* s = smem + (g % S) * Cfg::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[i] = *reinterpret_cast<const v4i*>(s + ((a_frag ^ (ks << 5)) + i * 32 * PBK));
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *reinterpret_cast<const v4i*>(s + ((b_frag ^ (ks << 5)) + j * 32 * PBK));
  };
  auto mma = [&](v4i (&fa)[TM], v4i (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0)
                         : __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
  };
  // scheduling hint: one LDS read after each of the first TM+TN MFMAs of a group
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < TM + TN; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
  };

  // ---- prologue: S-1 steps of copies, wait for the first
  set_copy_item(c_item);
#pragma unroll
  for (int s = 0; s < S - 1; ++s) {
    issue_copies();
    if (c_live && c_kt == KT) advance_copy_item();
  }
  wait_copies_then_barrier<(S - 2) * COPIES>();

  v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
  read_frags(0, 0, fa0, fb0);
  zero_acc();

  int item = first, kt = 0, g = 0;  // multiply cursor
  // One K step.  LAST = last K step of a work item: the next item's first fragments are
  // read after the epilogue instead, so they do not occupy registers during it.
  auto step = [&](auto last) {
    constexpr bool LAST = decltype(last)::value;
    read_frags(g, 1, fa1, fb1);
    mma(fa0, fb0);
    interleave();
    wait_copies_then_barrier<(S - 3) * COPIES>();  // step g+1 landed; g+2 .. g+S-2 may be in flight
    issue_copies();                                // step g+S-1 into the stage step g-1 used
    if (!LAST) read_frags(g + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    if (!LAST) interleave();
  };
  auto finish_item = [&]() {
    int b, t;
    decode_item(item, b, t);
    int tile_m, tile_n;
    tile_of_workgroup(t, tiles_m, tiles_n, tile_m, tile_n, p.band);
    // opaque copy of the lane id: keeps the epilogue's address arithmetic inside the loop
    // (hoisted, it would occupy registers during the whole mainloop)
    int lane_here = lane;
    asm volatile("" : "+v"(lane_here));
    store_tile<Cfg>(acc, p, b, tile_m * BM, tile_n * BN, wave_m, wave_n, lane_here);
    item += stride;
    kt = 0;
    zero_acc();
  };

  while (g < G) {
    // steps until the multiply or the copy cursor reaches the end of its work item
    int n = KT - kt;
    if (c_live && KT - c_kt < n) n = KT - c_kt;
    const bool item_done = kt + n == KT;
    const int plain = item_done ? n - 1 : n;
    for (int i = 0; i < plain; ++i) {
      step(std::false_type{});
      ++g;
    }
    if (item_done) {
      step(std::true_type{});
      ++g;
    }
    kt += n;
    if (c_live && c_kt == KT) advance_copy_item();
    if (item_done) {
      finish_item();
      if (g < G) read_frags(g, 0, fa0, fb0);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the trailing filler copies must land before the LDS is released
}

// ---------------------------------------------------------------------------
// The same persistent pipeline with K steps of 128 bytes and two LDS stages.
// A panel row of one step is one whole 128-byte cache line, so every line of
// the operands crosses the L2 -> L1 path once (with 64-byte steps each line is
// requested again one step later, after 64 KiB of other lines have passed
// through the L1), and there is one workgroup barrier per 128 bytes of K.
//
// LDS stage = [A panel BM x 128][B panel BN x 128]; chunk c of panel row r at
// chunk position c ^ ((r >> 1) & 7).  One copy instruction fills 1 KiB = 8
// panel rows, lane l landing at row l/8, position l%8.
//
// One K step = four 32-byte slices.  Fragments of slice s+1 are read while
// slice s multiplies.  After the reads of the last slice: wait for them and for
// this wave's copies of the next step, pass the barrier (next stage complete,
// this stage no longer read by anyone), issue the copies two steps ahead into
// the stage just released, read the first slice of the next step and multiply
// the last slice of this one.
static constexpr int QBK = 128;

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int KIND_, bool SWAP_>
struct Pipe2Cfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KIND = KIND_;
  static constexpr bool SWAP = SWAP_;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 32, TN = WTN / 32;
  static constexpr int STAGE_BYTES = (BM + BN) * QBK;
  static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
  static constexpr int COPIES = (BM + BN) / 8 / NWAVES;  // copy instructions per wave per step
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be made of 32x32 blocks");
  static_assert((BM + BN) % (8 * NWAVES) == 0 && (BM / 8) % COPIES == 0, "a wave copies 1 KiB slabs of one panel");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, 2) void gemm_pipe2_kernel(GemmParams p, int tiles_m, int tiles_n, int items) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, COPIES = Cfg::COPIES;
  constexpr bool SWAP = Cfg::SWAP;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
  const int M = p.M, N = p.N, K = p.K;
  const int KT = K / QBK;
  const int tiles = tiles_m * tiles_n;
  const int first = blockIdx.x, stride = gridDim.x;
  const int my_items = (items - first + stride - 1) / stride;  // >= 1 (grid <= items)
  const int G = my_items * KT;                                  // K steps this workgroup multiplies

  // ---- copy stream: copy j of this wave fills stage bytes [(wave*COPIES + j) * 1024, +1024)
  const bool copies_a = wave * COPIES * 8 < BM;  // this wave fills A panel rows (else B panel rows)
  const TI_GLOBAL_AS int8_t* src[COPIES];
  // item -> (batch, tile of the batch); p.group_batches: all tiles of a batch on one XCD (see gemm_pipe_kernel)
  auto decode_item = [&](int item, int& b, int& t) {
    if (p.group_batches) {
      const int l = item >> 3, q = l / tiles;
      b = q * 8 + (item & 7);
      t = l - q * tiles;
    } else {
      b = item / tiles;
      t = item - b * tiles;
    }
  };
  auto set_copy_item = [&](int item) {
    int b, t;
    decode_item(item, b, t);
    int tile_m, tile_n;
    tile_of_workgroup(t, tiles_m, tiles_n, tile_m, tile_n, p.band);
    const int first_row = copies_a ? tile_m * BM : tile_n * BN;  // of the panel in its operand
    const int last_row = (copies_a ? M : N) - 1;                 // edge rows re-read the last row; never stored
    const size_t ld = copies_a ? p.lda : p.ldb;
    const int8_t* origin = copies_a ? a_of_batch(p, b) : b_of_batch(p, b);
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      const int prow = (wave * COPIES + j) * 8 + (lane >> 3) - (copies_a ? 0 : BM);  // row inside the panel
      const int chunk = (lane & 7) ^ ((prow >> 1) & 7);
      int lr = prow;
      if (SWAP && !copies_a) lr = (prow & ~31) | ((prow & 4) << 2) | ((prow & 24) >> 1) | (prow & 3);  // MFMA row 8q+4h+j -> 16h+4q+j
      const int gr = first_row + lr < last_row ? first_row + lr : last_row;
      src[j] = (const TI_GLOBAL_AS int8_t*)(origin + (size_t)gr * ld + chunk * 16);
    }
  };
  // Copy cursor (work item, K step inside it, global step).  Past the last item it keeps
  // re-copying the final K step into the stage that is free anyway, so that one step of
  // copies is in flight at every barrier and the wait counts never change.
  int c_item = first, c_kt = 0, c_g = 0, c_live = 1;
  auto issue_copies = [&]() {
    TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + (c_g & 1) * Cfg::STAGE_BYTES + wave * COPIES * 1024;
#pragma unroll
    for (int j = 0; j < COPIES; ++j)
      __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[j] + c_kt * QBK), (TI_LDS_AS void*)(dst + j * 1024),
                                       16, 0, 0);
    c_kt += c_live;
    ++c_g;
  };
  auto advance_copy_item = [&]() {  // call when c_live && c_kt == KT
    if (c_g < G) {
      c_kt = 0;
      c_item += stride;
      set_copy_item(c_item);
    } else {
      c_live = 0;
      c_kt = KT - 1;
    }
  };

  // ---- fragment addressing: lane reads panel row (lane & 31), chunk 2*slice + (lane >> 5)
  const int frow = lane & 31;
  const int fpos = ((lane >> 5) ^ (frow >> 1)) & 7;  // chunk position for slice 0
  const int a_frag = (wave_m * Cfg::WTM + frow) * QBK + (fpos << 4);
  const int b_frag = BM * QBK + (wave_n * Cfg::WTN + frow) * QBK + (fpos << 4);

  v16i acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
  };
  auto read_frags = [&](int g, int slice, v4i (&fa)[TM], v4i (&fb)[TN]) {
    const char* s = smem + (g & 1) * Cfg::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < TM; ++i)
      fa[i] = *reinterpret_cast<const v4i*>(s + ((a_frag ^ (slice << 5)) + i * 32 * QBK));
#pragma unroll
    for (int j = 0; j < TN; ++j)
      fb[j] = *reinterpret_cast<const v4i*>(s + ((b_frag ^ (slice << 5)) + j * 32 * QBK));
  };
  auto mma = [&](v4i (&fa)[TM], v4i (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = SWAP ? __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0)
                         : __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
  };
  // scheduling hint: one LDS read after each of the first TM+TN MFMAs of a group
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < TM + TN; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // 1 MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // 1 DS read
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
  };

  // ---- prologue: two steps of copies, wait for the first
  set_copy_item(c_item);
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    issue_copies();
    if (c_live && c_kt == KT) advance_copy_item();
  }
  wait_copies_then_barrier<COPIES>();

  v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
  read_frags(0, 0, fa0, fb0);
  zero_acc();

  int item = first, kt = 0, g = 0;  // multiply cursor
  // One K step.  LAST = last K step of a work item: the next item's first fragments are
  // read after the epilogue instead, so they do not occupy registers during it.
  auto step = [&](auto last) {
    constexpr bool LAST = decltype(last)::value;
    read_frags(g, 1, fa1, fb1);
    mma(fa0, fb0);
    interleave();
    read_frags(g, 2, fa0, fb0);
    mma(fa1, fb1);
    interleave();
    read_frags(g, 3, fa1, fb1);
    mma(fa0, fb0);
    interleave();
    // the lgkmcnt wait is what allows this stage to be overwritten after the barrier
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    issue_copies();  // step g+2 into the stage this step used
    if (!LAST) read_frags(g + 1, 0, fa0, fb0);
    mma(fa1, fb1);
    if (!LAST) interleave();
  };
  auto finish_item = [&]() {
    int b, t;
    decode_item(item, b, t);
    int tile_m, tile_n;
    tile_of_workgroup(t, tiles_m, tiles_n, tile_m, tile_n, p.band);
    // opaque copy of the lane id: keeps the epilogue's address arithmetic inside the loop
    int lane_here = lane;
    asm volatile("" : "+v"(lane_here));
    store_tile<Cfg>(acc, p, b, tile_m * BM, tile_n * BN, wave_m, wave_n, lane_here);
    item += stride;
    kt = 0;
    zero_acc();
  };

  while (g < G) {
    // steps until the multiply or the copy cursor reaches the end of its work item
    int n = KT - kt;
    if (c_live && KT - c_kt < n) n = KT - c_kt;
    const bool item_done = kt + n == KT;
    const int plain = item_done ? n - 1 : n;
    for (int i = 0; i < plain; ++i) {
      step(std::false_type{});
      ++g;
    }
    if (item_done) {
      step(std::true_type{});
      ++g;
    }
    kt += n;
    if (c_live && c_kt == KT) advance_copy_item();
    if (item_done) {
      finish_item();
      if (g < G) read_frags(g, 0, fa0, fb0);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the trailing filler copies must land before the LDS is released
}

// ---------------------------------------------------------------------------
// Variant of the pipelined persistent kernel built from 16x16 blocks
// (v_mfma_i32_16x16x64_i8: one instruction covers the whole 64-byte K step).
// Its output tile can be any multiple of 16 per wave, which gives tile counts
// that divide the chip evenly where 256x256 does not: OPT-13B widths are
// multiples of 160, and 2048x5120 outputs make exactly 256 tiles of 256x160.
//
// Same LDS stage layout, swizzle, copy stream and barrier scheme as
// gemm_pipe_kernel.  Differences: a wave copies (BM+BN)/NWAVES panel rows per
// step, the last copy instruction with only part of its lanes enabled when
// that is not a multiple of 16; fragments of step g+1 are read while step g
// multiplies; the weight rows always feed the MFMA row operand, so a lane ends
// with four consecutive output columns of one row per block (4-byte s8 or
// 16-byte 32-bit stores).
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int STAGES_, int KIND_>
struct Pipe16Cfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KIND = KIND_, STAGES = STAGES_;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 16, TN = WTN / 16;
  static constexpr int STAGE_BYTES = (BM + BN) * PBK;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  static constexpr int RPW = (BM + BN) / NWAVES;  // panel rows a wave copies per step
  static constexpr int TAIL_ROWS = RPW % 16;
  static constexpr int COPIES = RPW / 16 + (TAIL_ROWS ? 1 : 0);
  // Registers: 4 per accumulator block, 4 per fragment.  When two full sets of fragments would not fit
  // next to the accumulators, the weight fragments are kept in one set and reloaded block by block,
  // each right after the MFMAs that consumed it.
  static constexpr bool SINGLE_B = 4 * TM * TN + 8 * (TM + TN) >= 224;
  static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be made of 16x16 blocks");
  static_assert((BM + BN) % NWAVES == 0 && RPW % 4 == 0, "a wave must copy whole groups of four rows");
  static_assert(LDS_BYTES <= 160 * 1024 && STAGES >= 3, "LDS budget");
};

// 4x4 transpose of dwords across the four 16-lane rows of a wave: lane (r, g) = r + 16 g enters with x[k] and
// leaves with x[k] = what lane (r, k) held in x[g].  Two v_permlane32_swap and two v_permlane16_swap; every lane
// of the wave must take part.
__device__ __forceinline__ void row_transpose4(int (&x)[4]) {
  auto a = __builtin_amdgcn_permlane32_swap((unsigned)x[0], (unsigned)x[2], false, false);  // rows 2,3 of x0 <-> rows 0,1 of x2
  auto b = __builtin_amdgcn_permlane32_swap((unsigned)x[1], (unsigned)x[3], false, false);
  auto c = __builtin_amdgcn_permlane16_swap(a[0], b[0], false, false);  // odd rows of the first <-> even rows of the second
  auto d = __builtin_amdgcn_permlane16_swap(a[1], b[1], false, false);
  x[0] = (int)c[0];
  x[1] = (int)c[1];
  x[2] = (int)d[0];
  x[3] = (int)d[1];
}

// Epilogue of the 16x16-block kernels: the lane holds row (lane & 15) and four consecutive columns
// 4 * (lane >> 4) .. +3 of every block.
template <class Cfg>
__device__ __forceinline__ void store_tile16(v4i (&acc)[Cfg::TM][Cfg::TN], const GemmParams& p, int b, int tile_m,
                                             int tile_n, int wave_m, int wave_n, int lane_here) {
  using E = Epi<Cfg::KIND>;
  using Out = typename E::Out;
  using BiasT = typename E::Bias;
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN;
  const int M = p.M, N = p.N;
  const int er = lane_here & 15, eg = lane_here >> 4;
  Out* __restrict__ C = reinterpret_cast<Out*>(p.C) + (long long)b * p.strideC;
  const BiasT* __restrict__ bias = reinterpret_cast<const BiasT*>(p.bias);
  const bool vec_ok = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
  const bool bias_al = (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
  if constexpr (sizeof(Out) == 1 && TN >= 4) {
    // 8-bit outputs of a wave tile that lies inside the matrix: the four lanes that share an output row swap
    // their 4-byte pieces of four column blocks, so that a lane ends with the 16 consecutive bytes of one block
    // and a store instruction writes 64 contiguous bytes of each of 16 rows instead of 16: a quarter of the
    // write requests.  (A condition on the tile, not the lane: all lanes of the wave take the swaps.)
    const int nw = tile_n * BN + wave_n * Cfg::WTN;  // first column of the wave tile
    if ((N & 15) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0 && nw + Cfg::WTN <= N && (p.out_d & 15) == 0) {
      // groups of four column blocks (the last group may be shorter and keeps its 4-byte stores)
#pragma unroll
      for (int j0 = 0; j0 < TN; j0 += 4) {
        constexpr int kFull = 4;
        const int nblk = TN - j0 < kFull ? TN - j0 : kFull;  // compile-time after unrolling
        float bt[4][4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          if (jj >= nblk) continue;
          const int nb = nw + (j0 + jj) * 16 + 4 * eg;
          BiasT bv[4] = {BiasT(0), BiasT(0), BiasT(0), BiasT(0)};
          if (E::kHasBias) {
            if ((reinterpret_cast<uintptr_t>(bias) & 3) == 0) {
              const int w = *reinterpret_cast<const int*>(bias + nb);
              __builtin_memcpy(bv, &w, 4);
            } else {
#pragma unroll
              for (int v = 0; v < 4; ++v) bv[v] = bias[nb + v];
            }
          }
#pragma unroll
          for (int v = 0; v < 4; ++v) bt[jj][v] = E::bias_term(bv[v], p.beta);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          const int m = tile_m * BM + wave_m * Cfg::WTM + i * 16 + er;
          int x[4] = {0, 0, 0, 0};
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            if (jj >= nblk) continue;
            x[jj] = pack_s8x4_ints(E::apply_int(acc[i][j0 + jj][0], bt[jj][0], p.alpha),
                                   E::apply_int(acc[i][j0 + jj][1], bt[jj][1], p.alpha),
                                   E::apply_int(acc[i][j0 + jj][2], bt[jj][2], p.alpha),
                                   E::apply_int(acc[i][j0 + jj][3], bt[jj][3], p.alpha));
          }
          if (nblk == 4) {
            row_transpose4(x);  // lane (er, eg) now holds block j0 + eg of its row, columns 0..15
            if (m < M) *reinterpret_cast<v4i*>(C + out_index(p, m, nw + (j0 + eg) * 16)) = v4i{x[0], x[1], x[2], x[3]};
          } else {
#pragma unroll
            for (int jj = 0; jj < 4; ++jj)
              if (jj < nblk && m < M) *reinterpret_cast<int*>(C + out_index(p, m, nw + (j0 + jj) * 16 + 4 * eg)) = x[jj];
          }
        }
      }
      return;
    }
  }
  // accumulate-into-output kind: fetch what the tile holds now, the loads in flight together before the
  // first use -- the whole wave tile when its TM*TN*4 registers fit, else one column block at a time
  constexpr bool HOLD_ALL = E::kAccumulate && TM * TN <= 12;
  constexpr int HJ = E::kAccumulate ? (HOLD_ALL ? TN : 1) : 1;
  typename std::conditional<E::kAccumulate, v4f, char>::type held[E::kAccumulate ? TM : 1][HJ];
  auto fetch_held = [&](int j, int slot) {
    if constexpr (E::kAccumulate) {
      const int nb = tile_n * BN + wave_n * Cfg::WTN + j * 16 + 4 * eg;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = tile_m * BM + wave_m * Cfg::WTM + i * 16 + er;
        const float* src = reinterpret_cast<const float*>(C) + out_index(p, m < M ? m : M - 1, nb < N ? nb : 0);
        v4f h = {0.f, 0.f, 0.f, 0.f};
        if (vec_ok && nb + 4 <= N) {
          h = *reinterpret_cast<const v4f*>(src);
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (nb + v < N) h[v] = src[v];
        }
        held[i][slot] = h;
      }
    }
  };
  if constexpr (HOLD_ALL) {
#pragma unroll
    for (int j = 0; j < TN; ++j) fetch_held(j, j);
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int nb = tile_n * BN + wave_n * Cfg::WTN + j * 16 + 4 * eg;
    if constexpr (E::kAccumulate && !HOLD_ALL) fetch_held(j, 0);
    float bt[4];
    if (E::kHasBias && vec_ok && bias_al && nb + 4 <= N) {
      BiasT bv[4];
      if (sizeof(BiasT) == 1) {
        const int w = *reinterpret_cast<const int*>(bias + nb);
        __builtin_memcpy(bv, &w, 4);
      } else {
        const v4i w = *reinterpret_cast<const v4i*>(bias + nb);
        __builtin_memcpy(bv, &w, 16);
      }
#pragma unroll
      for (int v = 0; v < 4; ++v) bt[v] = E::bias_term(bv[v], p.beta);
    } else {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        BiasT bv = BiasT(0);
        if (E::kHasBias && nb + v < N) bv = bias[nb + v];
        bt[v] = E::bias_term(bv, p.beta);
      }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = tile_m * BM + wave_m * Cfg::WTM + i * 16 + er;
      if (m >= M) continue;
      Out o[4];
#pragma unroll
      for (int v = 0; v < 4; ++v) o[v] = E::apply(acc[i][j][v], bt[v], p.alpha);
      Out* dst = C + out_index(p, m, nb < N ? nb : 0);
      if constexpr (E::kAccumulate) {
#pragma unroll
        for (int v = 0; v < 4; ++v) o[v] = held[i][HOLD_ALL ? j : 0][v] + o[v];
      }
      if (vec_ok && nb + 4 <= N) {
        if (sizeof(Out) == 4) {
          using W = typename std::conditional<sizeof(Out) == 4, Out, int>::type;
          v4i w4 = {__builtin_bit_cast(int, (W)o[0]), __builtin_bit_cast(int, (W)o[1]),
                    __builtin_bit_cast(int, (W)o[2]), __builtin_bit_cast(int, (W)o[3])};
          *reinterpret_cast<v4i*>(dst) = w4;
        } else {
          *reinterpret_cast<unsigned*>(dst) = (unsigned)(unsigned char)o[0] | ((unsigned)(unsigned char)o[1] << 8) |
                                              ((unsigned)(unsigned char)o[2] << 16) |
                                              ((unsigned)(unsigned char)o[3] << 24);
        }
      } else {
#pragma unroll
        for (int v = 0; v < 4; ++v)
          if (nb + v < N) dst[v] = o[v];
      }
    }
  }
}

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, 2) void gemm_pipe16_kernel(GemmParams p, int tiles_m, int tiles_n, int items) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, COPIES = Cfg::COPIES, S = Cfg::STAGES;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
  const int M = p.M, N = p.N, K = p.K;
  const int KT = K / PBK;
  const int tiles = tiles_m * tiles_n;
  const int first = blockIdx.x, stride = gridDim.x;
  const int my_items = (items - first + stride - 1) / stride;
  const int G = my_items * KT;

  // ---- copy stream: copy j of this wave fills panel rows wave*RPW + 16j .. +15 of [A panel | B panel]
  const TI_GLOBAL_AS int8_t* src[COPIES];
  auto set_copy_item = [&](int item) {
    const int b = item / tiles;
    int tile_m, tile_n;
    tile_of_workgroup(item - b * tiles, tiles_m, tiles_n, tile_m, tile_n, p.band);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int8_t* A = a_of_batch(p, b);
    const int8_t* B = b_of_batch(p, b);
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      int prow = wave * Cfg::RPW + j * 16 + (lane >> 2);
      prow = prow < BM + BN ? prow : BM + BN - 1;  // lanes beyond a partial last copy are disabled anyway
      const int pos = lane & 3;
      if (prow < BM) {
        const int chunk = pos ^ ((prow >> 2) & 3);
        const int gr = m0 + prow < M ? m0 + prow : M - 1;  // edge rows re-read the last row; never stored
        src[j] = (const TI_GLOBAL_AS int8_t*)(A + (size_t)gr * p.lda + chunk * 16);
      } else {
        const int br = prow - BM;
        const int chunk = pos ^ ((br >> 2) & 3);
        const int gr = n0 + br < N ? n0 + br : N - 1;
        src[j] = (const TI_GLOBAL_AS int8_t*)(B + (size_t)gr * p.ldb + chunk * 16);
      }
    }
  };
  int c_item = first, c_kt = 0, c_g = 0, c_live = 1;
  auto issue_copies = [&]() {
    TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + (c_g % S) * Cfg::STAGE_BYTES + wave * Cfg::RPW * PBK;
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      if (Cfg::TAIL_ROWS == 0 || j + 1 < COPIES || lane < Cfg::TAIL_ROWS * 4)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[j] + c_kt * PBK),
                                         (TI_LDS_AS void*)(dst + j * 1024), 16, 0, 0);
    }
    c_kt += c_live;
    ++c_g;
  };
  auto advance_copy_item = [&]() {  // call when c_live && c_kt == KT
    if (c_g < G) {
      c_kt = 0;
      c_item += stride;
      set_copy_item(c_item);
    } else {
      c_live = 0;
      c_kt = KT - 1;
    }
  };

  // ---- fragment addressing: lane reads panel row (lane & 15), chunk (lane >> 4)
  const int r = lane & 15, g4 = lane >> 4;
  const int fpos = (g4 ^ (r >> 2)) & 3;
  const int a_frag = (wave_m * Cfg::WTM + r) * PBK + (fpos << 4);
  const int b_frag = BM * PBK + (wave_n * Cfg::WTN + r) * PBK + (fpos << 4);

  v4i acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = v4i{0, 0, 0, 0};
  };
  auto read_frags = [&](int gs, v4i (&fa)[TM], v4i (&fb)[TN]) {
    const char* st = smem + (gs % S) * Cfg::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const v4i*>(st + a_frag + i * 16 * PBK);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const v4i*>(st + b_frag + j * 16 * PBK);
  };
  auto mma = [&](v4i (&fa)[TM], v4i (&fb)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
  };
  auto interleave = [&]() {  // one LDS read after each of the first TM+TN MFMAs
#pragma unroll
    for (int i = 0; i < TM + TN; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
  };

  set_copy_item(c_item);
#pragma unroll
  for (int s = 0; s < S - 1; ++s) {
    issue_copies();
    if (c_live && c_kt == KT) advance_copy_item();
  }
  wait_copies_then_barrier<(S - 2) * COPIES>();

  v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
  read_frags(0, fa0, fb0);
  zero_acc();

  int item = first, kt = 0, gs = 0;  // multiply cursor
  // One K step: multiply the fragments in (fc, fd) while those of the next step load into (fn, fm).
  auto step = [&](v4i (&fc)[TM], v4i (&fd)[TN], v4i (&fn)[TM], v4i (&fm)[TN], auto last) {
    constexpr bool LAST = decltype(last)::value;
    wait_copies_then_barrier<(S - 3) * COPIES>();  // step gs+1 landed; every wave is done with step gs-1
    issue_copies();                                // step gs+S-1 into the stage step gs-1 used
    if constexpr (Cfg::SINGLE_B) {
      // the weight fragments live in fb0 only (fd / fm are ignored)
      const char* st = smem + ((gs + 1) % S) * Cfg::STAGE_BYTES;
      if (!LAST) {
#pragma unroll
        for (int i = 0; i < TM; ++i) fn[i] = *reinterpret_cast<const v4i*>(st + a_frag + i * 16 * PBK);
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb0[j], fc[i], acc[i][j], 0, 0, 0);
        if (!LAST) fb0[j] = *reinterpret_cast<const v4i*>(st + b_frag + j * 16 * PBK);
      }
    } else {
      if (!LAST) read_frags(gs + 1, fn, fm);
      mma(fc, fd);
      if (!LAST) interleave();
    }
    ++gs;
  };
  auto finish_item = [&]() {
    const int b = item / tiles;
    int tile_m, tile_n;
    tile_of_workgroup(item - b * tiles, tiles_m, tiles_n, tile_m, tile_n, p.band);
    int lane_here = lane;  // opaque copy: keeps the epilogue's address arithmetic out of the mainloop
    asm volatile("" : "+v"(lane_here));
    store_tile16<Cfg>(acc, p, b, tile_m, tile_n, wave_m, wave_n, lane_here);
    item += stride;
    kt = 0;
    zero_acc();
  };

  while (gs < G) {
    // steps until the multiply or the copy cursor reaches the end of its work item
    int n = KT - kt;
    if (c_live && KT - c_kt < n) n = KT - c_kt;
    const bool item_done = kt + n == KT;
    int plain = item_done ? n - 1 : n;  // steps that also load the next step's fragments
    for (; plain >= 2; plain -= 2) {
      step(fa0, fb0, fa1, fb1, std::false_type{});
      step(fa1, fb1, fa0, fb0, std::false_type{});
    }
    if (plain == 1) {
      step(fa0, fb0, fa1, fb1, std::false_type{});
#pragma unroll
      for (int i = 0; i < TM; ++i) fa0[i] = fa1[i];
      if (!Cfg::SINGLE_B) {
#pragma unroll
        for (int j = 0; j < TN; ++j) fb0[j] = fb1[j];
      }
    }
    if (item_done) step(fa0, fb0, fa1, fb1, std::true_type{});
    kt += n;
    if (c_live && c_kt == KT) advance_copy_item();
    if (item_done) {
      finish_item();
      if (gs < G) read_frags(gs, fa0, fb0);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the trailing filler copies must land before the LDS is released
}

// The 16x16-block kernel with K steps of 128 bytes and two LDS stages (see gemm_pipe2_kernel for the
// stage layout and the step structure; a step here is two 64-byte slices, one MFMA deep each).
//
// FUSED (split-K in one launch): the work items are (output tile, K slice) pairs, and ALL slices of a tile run on
// workgroups of the SAME XCD (workgroup ids congruent mod 8), so that the int32 partial tiles meet in that XCD's
// L2 and no device-scope release / acquire (which writes back and invalidates a whole L2) is needed.  Every wave
// parks its accumulators in the workspace (16 bytes per lane and MFMA block, in register order), waits until the
// L2 has acknowledged the stores, and counts itself on an arrival counter of (tile, wave index) with an atomic
// that executes in the L2.  The wave that arrives last among the `splits` waves with its index adds the others'
// accumulators to its own, applies the epilogue to its part of the tile and puts the counter back to zero.
// Nobody waits for anybody, so there is nothing that can hang; integer sums make the result independent of
// the order of arrival.
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int KIND_, bool GROUPED_ = false, int MAX_STAGES_ = 3,
          bool FUSED_ = false>
struct Pipe16QCfg {
  static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, KIND = KIND_;
  static constexpr bool FUSED = FUSED_;
  static_assert(!(FUSED_ && GROUPED_), "the fused split takes one problem");
  // GROUPED: the "batches" are the problems of a GemmGroup (same activations and shape; weight, bias,
  // output and scales per problem), so that q/k/v projections run as one persistent launch
  static constexpr bool GROUPED = GROUPED_;
  static constexpr int NWAVES = WAVES_M * WAVES_N;
  static constexpr int NT = NWAVES * 64;
  static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
  static constexpr int TM = WTM / 16, TN = WTN / 16;
  static constexpr int STAGE_BYTES = (BM + BN) * QBK;
  // three stages when the LDS holds them (256x160): copies then run two to three K steps ahead of their use,
  // which covers the latency of operands that come from HBM instead of the last-level cache
  // (128x80 tiles, whose short rounds are mostly that latency when the weights are not cached, take more)
  static constexpr int FIT_STAGES = (160 * 1024) / STAGE_BYTES;
  static constexpr int STAGES = MAX_STAGES_ < 2 ? 2 : FIT_STAGES < 2 ? 2 : MAX_STAGES_ < FIT_STAGES ? MAX_STAGES_ : FIT_STAGES;
  static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
  static constexpr int RPW = (BM + BN) / NWAVES;  // panel rows a wave copies per step
  static constexpr int TAIL_ROWS = RPW % 8;
  static constexpr int COPIES = RPW / 8 + (TAIL_ROWS ? 1 : 0);
  static constexpr bool SINGLE_B = 4 * TM * TN + 8 * (TM + TN) >= 224;  // as in Pipe16Cfg
  static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be made of 16x16 blocks");
  static_assert((BM + BN) % NWAVES == 0 && RPW % 2 == 0, "a wave must copy whole pairs of rows");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
};

template <class Cfg>
__global__ __launch_bounds__(Cfg::NT, 2) void gemm_pipe16q_kernel(GemmParams p, int tiles_m, int tiles_n, int items,
                                                                  GemmGroup grp) {
  constexpr int BM = Cfg::BM, BN = Cfg::BN, TM = Cfg::TM, TN = Cfg::TN, COPIES = Cfg::COPIES;
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wave_m = wave / Cfg::WAVES_N, wave_n = wave % Cfg::WAVES_N;
  const int M = p.M, N = p.N, K = p.K;
  const int KT = K / QBK;
  const int tiles = tiles_m * tiles_n;
  // Work items of this workgroup: first, first + stride, ... below `items`.  FUSED: the items of this workgroup's
  // XCD (id mod 8; the grid is a multiple of 8) are numbered l = (tile of the XCD) * splits + slice, where the
  // XCD's tiles are the tile ids congruent to the XCD mod 8.
  const int xcd = blockIdx.x & 7;
  const int first = Cfg::FUSED ? (int)(blockIdx.x >> 3) : (int)blockIdx.x;
  const int stride = Cfg::FUSED ? (int)(gridDim.x >> 3) : (int)gridDim.x;
  if constexpr (Cfg::FUSED) items = tiles > xcd ? ((tiles - xcd + 7) >> 3) * p.splits : 0;
  const int my_items = items > first ? (items - first + stride - 1) / stride : 0;
  if (my_items == 0) return;  // the same for every wave of the workgroup, before the first barrier
  const int G = my_items * KT;
  // item -> (batch or K slice b, tile id)
  auto decode_item = [&](int item, int& b, int& tile_id) {
    if constexpr (Cfg::FUSED) {
      const int t = item / p.splits;
      b = item - t * p.splits;
      tile_id = t * 8 + xcd;
    } else if (p.group_batches) {  // all tiles of a batch on one XCD, next to one another (see gemm_pipe_kernel)
      const int l = item >> 3, q = l / tiles;
      b = q * 8 + (item & 7);
      tile_id = l - q * tiles;
    } else {
      b = item / tiles;
      tile_id = item - b * tiles;
    }
  };
  // FUSED: all workgroups of a tile must run on one XCC (the hardware deals workgroup ids out round robin, from a
  // start that depends on the queue).  Checked, not assumed: thread 0 marks this workgroup's XCC id in the tile's
  // word with a device-scope atomic when it takes the tile up and looks at the marks of the others when it is done.
  unsigned xcc_bit = 0, xcc_others = 0;
  auto mark_xcc = [&](int item) {
    if constexpr (Cfg::FUSED) {
      if (threadIdx.x == 0) {
        int b, tile_id;
        decode_item(item, b, tile_id);
        xcc_bit = 1u << (__builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf);  // HW_REG_XCC_ID, bits 3:0
        xcc_others = __hip_atomic_fetch_or(p.xcc_seen + tile_id, xcc_bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  };
  mark_xcc(first);

  // ---- copy stream: copy j of this wave fills panel rows wave*RPW + 8j .. +7 of [A panel | B panel]
  const TI_GLOBAL_AS int8_t* src[COPIES];
  auto set_copy_item = [&](int item) {
    int b, tile_id;
    decode_item(item, b, tile_id);
    int tile_m, tile_n;
    tile_of_workgroup(tile_id, tiles_m, tiles_n, tile_m, tile_n, p.band);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int8_t* A = Cfg::GROUPED ? p.A : a_of_batch(p, b);
    const int8_t* B = Cfg::GROUPED ? grp.B[b] : b_of_batch(p, b);
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      int prow = wave * Cfg::RPW + j * 8 + (lane >> 3);
      prow = prow < BM + BN ? prow : BM + BN - 1;  // lanes beyond a partial last copy are disabled anyway
      const int pos = lane & 7;
      if (prow < BM) {
        const int chunk = pos ^ ((prow >> 1) & 7);
        const int gr = m0 + prow < M ? m0 + prow : M - 1;  // edge rows re-read the last row; never stored
        src[j] = (const TI_GLOBAL_AS int8_t*)(A + (size_t)gr * p.lda + chunk * 16);
      } else {
        const int br = prow - BM;
        const int chunk = pos ^ ((br >> 1) & 7);
        const int gr = n0 + br < N ? n0 + br : N - 1;
        src[j] = (const TI_GLOBAL_AS int8_t*)(B + (size_t)gr * p.ldb + chunk * 16);
      }
    }
  };
  constexpr int STAGES = Cfg::STAGES;
  auto next_slot = [](int slot) { return slot + 1 == STAGES ? 0 : slot + 1; };
  int c_item = first, c_kt = 0, c_g = 0, c_live = 1, c_slot = 0;
  auto issue_copies = [&]() {
    TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + c_slot * Cfg::STAGE_BYTES + wave * Cfg::RPW * QBK;
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      if (Cfg::TAIL_ROWS == 0 || j + 1 < COPIES || lane < Cfg::TAIL_ROWS * 8)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[j] + c_kt * QBK),
                                         (TI_LDS_AS void*)(dst + j * 1024), 16, 0, 0);
    }
    c_kt += c_live;
    ++c_g;
    c_slot = next_slot(c_slot);
  };
  auto advance_copy_item = [&]() {  // call when c_live && c_kt == KT
    if (c_g < G) {
      c_kt = 0;
      c_item += stride;
      set_copy_item(c_item);
    } else {
      c_live = 0;
      c_kt = KT - 1;
    }
  };

  // ---- fragment addressing: lane reads panel row (lane & 15), chunk 4*slice + (lane >> 4)
  const int r = lane & 15, g4 = lane >> 4;
  const int fpos = (g4 ^ (r >> 1)) & 7;  // chunk position for slice 0
  const int a_frag = (wave_m * Cfg::WTM + r) * QBK + (fpos << 4);
  const int b_frag = BM * QBK + (wave_n * Cfg::WTN + r) * QBK + (fpos << 4);

  v4i acc[TM][TN];
  auto zero_acc = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = v4i{0, 0, 0, 0};
  };
  auto read_a = [&](int slot, int slice, v4i (&fa)[TM]) {
    const char* st = smem + slot * Cfg::STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const v4i*>(st + ((a_frag ^ (slice << 6)) + i * 16 * QBK));
  };
  auto read_b1 = [&](int slot, int slice, int j) {
    const char* st = smem + slot * Cfg::STAGE_BYTES;
    return *reinterpret_cast<const v4i*>(st + ((b_frag ^ (slice << 6)) + j * 16 * QBK));
  };
  auto read_frags = [&](int slot, int slice, v4i (&fa)[TM], v4i (&fb)[TN]) {
    read_a(slot, slice, fa);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[j] = read_b1(slot, slice, j);
  };
  auto interleave = [&]() {  // one LDS read after each of the first TM+TN MFMAs
#pragma unroll
    for (int i = 0; i < TM + TN; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - (TM + TN), 0);
  };
  // Multiplies the fragments (fc, fd) while those of (stage gs_next, slice_next) load into (fn, fm); with
  // SINGLE_B the weight fragments live in fd only and are replaced block by block.
  auto mma_and_fetch = [&](v4i (&fc)[TM], v4i (&fd)[TN], v4i (&fn)[TM], v4i (&fm)[TN], int gs_next, int slice_next,
                           auto fetch) {
    constexpr bool FETCH = decltype(fetch)::value;
    if constexpr (Cfg::SINGLE_B) {
      if (FETCH) read_a(gs_next, slice_next, fn);
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fd[j], fc[i], acc[i][j], 0, 0, 0);
        if (FETCH) fd[j] = read_b1(gs_next, slice_next, j);
      }
    } else {
      if (FETCH) read_frags(gs_next, slice_next, fn, fm);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fd[j], fc[i], acc[i][j], 0, 0, 0);
      if (FETCH) interleave();
    }
  };

  set_copy_item(c_item);
#pragma unroll
  for (int s = 0; s < STAGES; ++s) {
    issue_copies();
    if (c_live && c_kt == KT) advance_copy_item();
  }
  wait_copies_then_barrier<(STAGES - 1) * COPIES>();  // step 0 has landed

  v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];  // fb1 is unused with SINGLE_B
  read_frags(0, 0, fa0, fb0);
  zero_acc();

  int item = first, kt = 0, gs = 0, slot = 0;  // multiply cursor; slot = gs % STAGES
  auto step = [&](auto last) {
    constexpr bool LAST = decltype(last)::value;
    mma_and_fetch(fa0, fb0, fa1, Cfg::SINGLE_B ? fb0 : fb1, slot, 1, std::true_type{});
    // Step gs+1 has landed once at most the copies of the steps after it are outstanding (loads complete in
    // order; stores of an epilogue in between only make the count conservative).  The lgkmcnt wait is what
    // allows this stage to be overwritten after the barrier.  (Allowing for the epilogue's stores in the first
    // waits of the next tile, through a uniform branch around the wait, was measured slower: 184 against 178 us
    // at 8192x5120x5120.)
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((STAGES - 2) * COPIES) : "memory");
    issue_copies();  // step gs+STAGES into the stage this step used
    slot = next_slot(slot);
    mma_and_fetch(fa1, Cfg::SINGLE_B ? fb0 : fb1, fa0, fb0, slot, 0, std::integral_constant<bool, !LAST>{});
    ++gs;
  };
  auto finish_item = [&]() {
    int b, tile_id;
    decode_item(item, b, tile_id);
    int tile_m, tile_n;
    tile_of_workgroup(tile_id, tiles_m, tiles_n, tile_m, tile_n, p.band);
    int lane_here = lane;  // opaque copy: keeps the epilogue's address arithmetic out of the mainloop
    asm volatile("" : "+v"(lane_here));
    if constexpr (Cfg::FUSED) {
      constexpr long long PER_WAVE = (long long)TM * TN * 64;  // v4i elements a wave parks per (tile, slice)
      const int splits = p.splits;
      v4i* parts = reinterpret_cast<v4i*>(p.parts);
      v4i* mine = parts + (((long long)tile_id * splits + b) * Cfg::NWAVES + wave) * PER_WAVE + lane_here;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) mine[(i * TN + j) * 64] = acc[i][j];
      // acknowledged by the L2 (stores and loads share the counter: this also waits for the copies in flight)
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      if (threadIdx.x == 0 && (xcc_others & ~xcc_bit) != 0)  // a workgroup of this tile ran on another XCC
        __hip_atomic_store(p.xcc_error, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      int* counter = p.arrivals + tile_id * Cfg::NWAVES + wave;
      int earlier = 0;
      if (lane_here == 0)
        earlier = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      earlier = __builtin_amdgcn_readfirstlane(earlier);
      if (earlier == splits - 1) {  // uniform over the wave
        for (int t = 0; t < splits; ++t) {
          if (t == b) continue;
          const v4i* theirs = parts + (((long long)tile_id * splits + t) * Cfg::NWAVES + wave) * PER_WAVE + lane_here;
          // two rows of blocks at a time: 2 TN loads in flight, then the adds (one statement per block would make
          // the compiler wait for every load before it issues the next)
          constexpr int RB = TM % 2 == 0 && TN <= 5 ? 2 : 1;
#pragma unroll
          for (int i0 = 0; i0 < TM; i0 += RB) {
            v4i got[RB][TN];
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j) got[i][j] = theirs[((i0 + i) * TN + j) * 64];
#pragma unroll
            for (int i = 0; i < RB; ++i)
#pragma unroll
              for (int j = 0; j < TN; ++j) acc[i0 + i][j] += got[i][j];
          }
        }
        if (lane_here == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        // every workgroup of the tile made its mark before its wave 0 counted itself: the last wave 0 clears the word
        if (threadIdx.x == 0) __hip_atomic_store(p.xcc_seen + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        store_tile16<Cfg>(acc, p, 0, tile_m, tile_n, wave_m, wave_n, lane_here);
      }
      if (my_items > 1 && item + stride < items) mark_xcc(item + stride);
    } else if constexpr (Cfg::GROUPED) {
      GemmParams q = p;  // problem b of the group as a one-batch problem
      q.bias = grp.bias[b];
      q.C = grp.C[b];
      q.alpha = grp.alpha[b];
      q.beta = grp.beta[b];
      store_tile16<Cfg>(acc, q, 0, tile_m, tile_n, wave_m, wave_n, lane_here);
    } else {
      store_tile16<Cfg>(acc, p, b, tile_m, tile_n, wave_m, wave_n, lane_here);
    }
    item += stride;
    kt = 0;
    zero_acc();
  };

  while (gs < G) {
    // steps until the multiply or the copy cursor reaches the end of its work item
    int n = KT - kt;
    if (c_live && KT - c_kt < n) n = KT - c_kt;
    const bool item_done = kt + n == KT;
    const int plain = item_done ? n - 1 : n;
    for (int i = 0; i < plain; ++i) step(std::false_type{});
    if (item_done) step(std::true_type{});
    kt += n;
    if (c_live && c_kt == KT) advance_copy_item();
    if (item_done) {
      finish_item();
      if (gs < G) read_frags(slot, 0, fa0, fb0);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);  // the trailing filler copies must land before the LDS is released
}

// Epilogue of the M <= 16 kernels: the lane holds row m and columns nb .. nb+3.
template <int KIND>
__device__ __forceinline__ void store_skinny_tile(v4i acc, const GemmParams& p, int batch, int m, int nb) {
  using E = Epi<KIND>;
  using Out = typename E::Out;
  using BiasT = typename E::Bias;
  const int N = p.N;
  Out* C = reinterpret_cast<Out*>(p.C) + (long long)batch * p.strideC;
  const BiasT* bias = reinterpret_cast<const BiasT*>(p.bias);
  Out o[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    BiasT bv = BiasT(0);
    if (E::kHasBias && nb + v < N) bv = bias[nb + v];
    o[v] = E::apply(acc[v], E::bias_term(bv, p.beta), p.alpha);
  }
  Out* dst = C + out_index(p, m, nb < N ? nb : 0);
  if constexpr (E::kAccumulate) {
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (nb + v < N) o[v] = merge_old<E>(o[v], dst + v);
  }
  const bool whole = (N % 4 == 0) && nb + 4 <= N && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
  if (whole && sizeof(Out) == 4) {
    using W = typename std::conditional<sizeof(Out) == 4, Out, int>::type;
    v4i w4 = {__builtin_bit_cast(int, (W)o[0]), __builtin_bit_cast(int, (W)o[1]), __builtin_bit_cast(int, (W)o[2]),
              __builtin_bit_cast(int, (W)o[3])};
    *reinterpret_cast<v4i*>(dst) = w4;
  } else if (whole) {
    *reinterpret_cast<unsigned*>(dst) = (unsigned)(unsigned char)o[0] | ((unsigned)(unsigned char)o[1] << 8) |
                                        ((unsigned)(unsigned char)o[2] << 16) | ((unsigned)(unsigned char)o[3] << 24);
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (nb + v < N) dst[v] = o[v];
  }
}

// The same epilogue with its memory operands already in registers (fetched while the strip was still being
// multiplied, so that their latency is not on the path between two blocks): bias values bv[0..3] of columns
// nb .. nb+3 (zero where there is no bias or the column is outside the matrix) and, for the accumulate kind, the
// current output values old[0..3].  Lanes with live == false (rows past M) compute and store nothing, but the
// arithmetic sits outside that branch on purpose: the registers of bv and old are then consumed on every path,
// and the compiler needs no wait in front of the next prefetch into them.
template <int KIND>
__device__ __forceinline__ void store_skinny_tile_pre(v4i acc, const GemmParams& p, int batch, int m, int nb,
                                                      const typename Epi<KIND>::Bias (&bv)[4],
                                                      const typename Epi<KIND>::Out (&old)[4], bool live) {
  using E = Epi<KIND>;
  using Out = typename E::Out;
  const int N = p.N;
  Out* C = reinterpret_cast<Out*>(p.C) + (long long)batch * p.strideC;
  Out o[4];
#pragma unroll
  for (int v = 0; v < 4; ++v) {
    o[v] = E::apply(acc[v], E::bias_term(bv[v], p.beta), p.alpha);
    if constexpr (E::kAccumulate) o[v] = old[v] + o[v];
  }
  if (!live) return;
  Out* dst = C + out_index(p, m, nb < N ? nb : 0);
  const bool whole = (N % 4 == 0) && nb + 4 <= N && (reinterpret_cast<uintptr_t>(C) & 15) == 0;
  if (whole && sizeof(Out) == 4) {
    using W = typename std::conditional<sizeof(Out) == 4, Out, int>::type;
    v4i w4 = {__builtin_bit_cast(int, (W)o[0]), __builtin_bit_cast(int, (W)o[1]), __builtin_bit_cast(int, (W)o[2]),
              __builtin_bit_cast(int, (W)o[3])};
    *reinterpret_cast<v4i*>(dst) = w4;
  } else if (whole) {
    *reinterpret_cast<unsigned*>(dst) = (unsigned)(unsigned char)o[0] | ((unsigned)(unsigned char)o[1] << 8) |
                                        ((unsigned)(unsigned char)o[2] << 16) | ((unsigned)(unsigned char)o[3] << 24);
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v)
      if (nb + v < N) dst[v] = o[v];
  }
}

// ---------------------------------------------------------------------------
// Skinny GEMM for M <= 16 (decode): HBM-bound, every weight byte is used once.
//
// A workgroup of NW waves owns 16 weight rows (output columns); the waves
// split K evenly and add their partial 16x16 tiles through LDS at the end.
// Weight fragments go straight from global memory into MFMA operand registers
// (no LDS): for the j-th v_mfma_i32_16x16x64_i8 of a 256-byte K block, lane
// (r = lane & 15, g = lane >> 4) loads 16-byte chunk 4j + g of row r, so one
// load instruction reads 64 contiguous bytes of each of 16 rows.
// All loads of NBLK blocks are issued before the first MFMA so that each wave
// keeps NBLK KiB of weights in flight.
template <int NBLK, int KIND>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(GemmParams p) {
  extern __shared__ int red[];  // [NW - 1][256]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nw = blockDim.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int M = p.M, N = p.N, K = p.K;
  const int n0 = blockIdx.x * 16;
  const int8_t* A = p.A + (long long)blockIdx.z * p.strideA;
  const int8_t* B = p.B + (long long)blockIdx.z * p.strideB;
  const int nrow = n0 + r < N ? n0 + r : N - 1;
  const int mrow = r < M ? r : M - 1;
  const v4i* wp = reinterpret_cast<const v4i*>(B + (size_t)nrow * K) + g;
  const v4i* xp = reinterpret_cast<const v4i*>(A + (size_t)mrow * K) + g;
  // this wave's range of 16-byte chunks, a whole number of 256-byte blocks (16 chunks) long
  const int chunks = K >> 4;
  const int per_wave = (((chunks + nw - 1) / nw) + 15) & ~15;
  const int c_begin = wave * per_wave;
  const int c_end = c_begin + per_wave < chunks ? c_begin + per_wave : chunks;

  v4i acc = {0, 0, 0, 0};
  int c = c_begin;
  for (; c + 16 * NBLK <= c_end; c += 16 * NBLK) {
    v4i w[NBLK][4], x[NBLK][4];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
      for (int j = 0; j < 4; ++j) w[b][j] = wp[c + b * 16 + j * 4];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
      for (int j = 0; j < 4; ++j) x[b][j] = xp[c + b * 16 + j * 4];
#pragma unroll
    for (int b = 0; b < NBLK; ++b)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(w[b][j], x[b][j], acc, 0, 0, 0);
  }
  for (; c < c_end; c += 16) {  // remaining blocks; chunks past the end count as zeros
    const v4i z = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool ok = c + j * 4 + g < c_end;
      v4i w = ok ? wp[c + j * 4] : z;
      v4i x = ok ? xp[c + j * 4] : z;
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(w, x, acc, 0, 0, 0);
    }
  }

  // ---- add the K slices (integer adds: any order gives the same bits)
  if (wave > 0) {
#pragma unroll
    for (int v = 0; v < 4; ++v) red[(wave - 1) * 256 + v * 64 + lane] = acc[v];
  }
  __syncthreads();
  if (wave > 0) return;
  for (int w = 0; w < nw - 1; ++w)
#pragma unroll
    for (int v = 0; v < 4; ++v) acc[v] += red[w * 256 + v * 64 + lane];

  if (r >= M) return;
  store_skinny_tile<KIND>(acc, p, blockIdx.z, r, n0 + 4 * g);
}

// ---------------------------------------------------------------------------
// Streaming GEMM for M <= 16 with many output columns (decode projections):
// the weight matrix is read once, in 1 KiB contiguous runs.
//
// A workgroup of four waves owns 16 weight rows at a time (a "strip") and
// walks K in blocks of 1024 bytes; it is persistent and takes several strips.
// One global->LDS copy instruction moves the whole 1 KiB block of one row
// (64 lanes x 16 bytes, contiguous in HBM); lane l fetches chunk l ^ row, so
// that the later 16-byte fragment reads of 16 different rows at the same
// logical chunk hit 16 different bank groups.  The 16 activation rows of the
// block (rows >= M repeat row M-1; L2-resident) are staged the same way.
// S stages of 32 KiB keep S-1 blocks of copies in flight and the copy stream
// runs across strip boundaries.  Wave w multiplies the w-th 256-byte quarter
// of a block with four v_mfma_i32_16x16x64_i8; at the end of a strip the four
// partial tiles are added through LDS and wave 0 applies the epilogue.
//
// Loads and stores share one in-order counter per wave, so any wait of the
// storing wave on a younger load also waits for the acknowledgement of the
// strip's output stores, and the workgroup waits with it at the next barrier.
// Hence: wave 0 issues no copies (waves 1 to 3 do; the barrier after their
// wait tells wave 0 that the block is in the LDS); the epilogue's memory
// operands (bias, old outputs of the accumulating kind) are fetched when a
// strip starts and consumed when it ends; and the two roles run separate
// instances of the loop, so that the compiler places no wait of its own
// between a strip's stores and the next prefetch.  The barrier at the end of a
// strip waits for LDS traffic only (__syncthreads would drain the copies).
// Together: 20.8 -> 19.6 us for 1x20480x5120 and 24.4 -> 22.4 us with 16 rows.
// Requires K % 1024 == 0.
static constexpr int SBK = 1024;
// cache policy of the weight-row copies: non-temporal (`nt`).  Every weight byte is read once per launch, and a
// decode step streams far more weights than the 256 MB last-level cache holds; without the hint each line is
// allocated there on its way through (1x36864x9216 57.7 -> 54.2 us, 4x9216x36864 66.5 -> 60.5 us, cold weights).
static constexpr int STREAM_WEIGHT_AUX = 2;
static constexpr int S_RED = 3 * 256 * 4;  // partial tiles of waves 1..3

// MX = activation rows staged per block (1, 4 or 16 >= M); S = LDS stages.
// GROUPED: the "batches" are the problems of a GemmGroup (same activations and shape; weight, bias,
// output and scales per problem) instead of slices of one strided tensor.
// PARTS = 2 or 4 (one batch, plain row-major output): the launch multiplies the VIEW of the problem in which every
// row of the activations and of the weights is cut into PARTS rows of K / PARTS bytes -- p holds the view: M, N
// and PARTS times the real ones, K, lda, ldb a PARTS-th -- and the epilogue adds the PARTS entries of the product
// of the views that belong to one output, out[m][n] = sum_f C'[n PARTS + f][m PARTS + f].  A weight matrix with few,
// long rows (fc2 of a decode step) then has PARTS times the strips, of rows a PARTS-th as far apart.
template <int KIND, int MX, int S, bool GROUPED = false, int PARTS = 1>
__global__ __launch_bounds__(256) void gemm_stream_kernel(GemmParams p, int strips_per_batch, int strips,
                                                          GemmGroup grp) {
  static_assert(PARTS == 1 || ((PARTS == 2 || PARTS == 4) && !GROUPED), "views of two or four parts, one problem");
  constexpr int ROWS = 16 + MX;              // row copies per block
  constexpr int COPIES = (ROWS + 2) / 3;     // per copying wave (1..3); indices past ROWS repeat the last row copy
  constexpr int STAGE = ROWS * SBK;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  int* red = reinterpret_cast<int*>(smem + S * STAGE);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int M = p.M, N = p.N, K = p.K;
  const int KB = K / SBK;
  const int first = blockIdx.x, stride = gridDim.x;
  // Runs of 8 consecutive strips (one 128-byte line of every 8-bit output row) stay on one XCD, so that its L2
  // merges the eight 16-byte pieces of a line (16x20480x5120 with 8-bit outputs: 23.4 -> 22.4 us): workgroup w
  // runs on XCD w % 8.  Grids that are not a multiple of 8 take strips blockIdx.x, +gridDim.x, ...
  const bool xmap = (gridDim.x & 7) == 0;
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, n_local = gridDim.x >> 3;
  auto nth_strip = [&](int i) -> int {
    if (!xmap) return first + i * stride;
    const int t = local + i * n_local;
    return ((((t >> 3) << 3) + xcd) << 3) + (t & 7);
  };
  int my_strips = 0;
  while (nth_strip(my_strips) < strips) ++my_strips;
  if (my_strips == 0) return;  // before the first barrier, and the same for every wave of the workgroup
  const int G = my_strips * KB;

  // copy q of a block: q < 16 weight row q, else activation row q - 16; wave w >= 1 does q = w-1, w+2, ...
  const int cw = wave > 0 ? wave - 1 : 0;
  const TI_GLOBAL_AS int8_t* src[COPIES];
  auto set_copy_strip = [&](int strip) {
    const int b = strip / strips_per_batch;
    const int n0 = (strip - b * strips_per_batch) * 16;
    const int8_t* A = GROUPED ? p.A : p.A + (long long)b * p.strideA;
    const int8_t* B = GROUPED ? grp.B[b] : p.B + (long long)b * p.strideB;
#pragma unroll
    for (int i = 0; i < COPIES; ++i) {
      int q = cw + 3 * i;
      q = q < ROWS ? q : ROWS - 1;
      if (q < 16) {
        const int nrow = n0 + q < N ? n0 + q : N - 1;
        src[i] = (const TI_GLOBAL_AS int8_t*)(B + (size_t)nrow * p.ldb + ((lane ^ q) << 4));
      } else {
        const int xr = q - 16;
        const int mrow = xr < M ? xr : M - 1;
        src[i] = (const TI_GLOBAL_AS int8_t*)(A + (size_t)mrow * p.lda + ((lane ^ xr) << 4));
      }
    }
  };
  // Copy cursor; past the last strip it keeps re-copying the final block into the free
  // stage so that the number of copies in flight (and the wait count) never changes.
  int c_i = 0, c_kb = 0, c_g = 0, c_live = 1;
  auto issue = [&]() {
    TI_LDS_AS char* dst = (TI_LDS_AS char*)smem + (c_g % S) * STAGE;
    const size_t off = (size_t)c_kb * SBK;
#pragma unroll
    for (int i = 0; i < COPIES; ++i) {
      int q = cw + 3 * i;
      q = q < ROWS ? q : ROWS - 1;
      // the activation rows are re-read by every workgroup and keep the default policy
      if (q < 16)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[i] + off), (TI_LDS_AS void*)(dst + q * SBK),
                                         16, 0, STREAM_WEIGHT_AUX);
      else
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(src[i] + off), (TI_LDS_AS void*)(dst + q * SBK),
                                         16, 0, 0);
    }
    c_kb += c_live;
    ++c_g;
    if (c_live && c_kb == KB) {
      if (c_g < G) {
        c_kb = 0;
        set_copy_strip(nth_strip(++c_i));
      } else {
        c_live = 0;
        c_kb = KB - 1;
      }
    }
  };
  // fragment j of this wave's quarter: logical chunk wave*16 + 4j + g, stored at chunk ^ row
  const int xr = r < MX ? r : MX - 1;
  int woff[4], xoff[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int c = wave * 16 + 4 * j + g;
    woff[j] = r * SBK + ((c ^ r) << 4);
    xoff[j] = (16 + xr) * SBK + ((c ^ xr) << 4);
  }

  if (wave > 0) {
    set_copy_strip(nth_strip(0));
#pragma unroll
    for (int i = 0; i < S - 1; ++i) issue();
  }

  // The epilogue's memory operands of the strip being multiplied (wave 0 only): fetched when the strip starts.
  using EpiT = Epi<KIND>;
  typename EpiT::Bias bias_pre[4];
  typename EpiT::Out old_pre[4];
  auto fetch_epilogue_operands = [&](int strip_) {
    if constexpr (PARTS > 1) {
      // lane (r, g) of the view's tile ends up with the real outputs (m = r / PARTS, n = n_first .. + 4 / PARTS - 1)
      const int n_real = N / PARTS, m_real = M / PARTS;
      const int n_first = strip_ * (16 / PARTS) + g * (4 / PARTS);
      const int m = r / PARTS < m_real ? r / PARTS : m_real - 1;
      const typename EpiT::Bias* bias = reinterpret_cast<const typename EpiT::Bias*>(p.bias);
      const typename EpiT::Out* C = reinterpret_cast<const typename EpiT::Out*>(p.C);
#pragma unroll
      for (int v = 0; v < 4 / PARTS; ++v) {
        const int n = n_first + v < n_real ? n_first + v : n_real - 1;
        if constexpr (EpiT::kHasBias) bias_pre[v] = bias[n];
        else bias_pre[v] = typename EpiT::Bias(0);
        if constexpr (EpiT::kAccumulate) old_pre[v] = C[(size_t)m * n_real + n];
      }
      return;
    }
    const int b = strip_ / strips_per_batch;
    const int nb = (strip_ - b * strips_per_batch) * 16 + 4 * g;
    const typename EpiT::Bias* bias = reinterpret_cast<const typename EpiT::Bias*>(GROUPED ? grp.bias[b] : p.bias);
    // Unconditional loads from clamped addresses (columns past N are never stored): a register that is first
    // cleared and then loaded under a condition would make the compiler wait for every outstanding vector-memory
    // operation, the previous strip's output stores included, before the clear.
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if constexpr (EpiT::kHasBias) bias_pre[v] = bias[nb + v < N ? nb + v : N - 1];
      else bias_pre[v] = typename EpiT::Bias(0);
    }
    if constexpr (EpiT::kAccumulate) {
      const typename EpiT::Out* C = reinterpret_cast<const typename EpiT::Out*>(GROUPED ? grp.C[b] : p.C) +
                                    (GROUPED ? 0 : (long long)b * p.strideC);
      const typename EpiT::Out* at = C + out_index(p, r < M ? r : M - 1, nb < N ? nb : 0);
#pragma unroll
      for (int v = 0; v < 4; ++v) old_pre[v] = at[nb + v < N ? v : 0];
    }
  };
  // The wave that applies the epilogue (0) and the copying waves (1..3) run separate instances of the loop:
  // with one instance and "if (wave == 0)" around the prefetch and around its use, the compiler cannot tell
  // that the two conditions agree and puts a wait for every outstanding vector-memory operation (the previous
  // strip's output stores included) in front of the prefetch.  Both instances execute the same barriers.
  auto run = [&](auto role) {
    constexpr bool kEpilogueWave = decltype(role)::value;
    v4i acc = {0, 0, 0, 0};
    int gs = 0;  // blocks multiplied so far
    for (int si = 0; si < my_strips; ++si) {
      const int strip = nth_strip(si);
      if constexpr (kEpilogueWave) fetch_epilogue_operands(strip);
      for (int kb = 0; kb < KB; ++kb, ++gs) {
        // block gs has landed (S-2 younger blocks may be in flight); all waves are done with block gs-1
        if constexpr (!kEpilogueWave) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((S - 2) * COPIES) : "memory");
        asm volatile("s_barrier" ::: "memory");
        if constexpr (!kEpilogueWave) issue();  // block gs+S-1 into the stage block gs-1 used
        const char* st = smem + (gs % S) * STAGE;
        v4i wf[4], xf[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          wf[j] = *reinterpret_cast<const v4i*>(st + woff[j]);
          xf[j] = *reinterpret_cast<const v4i*>(st + xoff[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[j], xf[j], acc, 0, 0, 0);
      }
      // ---- strip finished: add the four quarters (integer adds: any order gives the same bits)
      if constexpr (!kEpilogueWave) {
#pragma unroll
        for (int v = 0; v < 4; ++v) red[(wave - 1) * 256 + v * 64 + lane] = acc[v];
      }
      // the partial tiles are in the LDS; the copies in flight stay in flight (__syncthreads would drain them)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      if constexpr (kEpilogueWave) {
#pragma unroll
        for (int w = 0; w < 3; ++w)
#pragma unroll
          for (int v = 0; v < 4; ++v) acc[v] += red[w * 256 + v * 64 + lane];
        if constexpr (PARTS > 1) {
          // entry (n' = 4g + v, m' = r) of the view's tile belongs to output (n' / PARTS, m' / PARTS) when
          // n' % PARTS == m' % PARTS: each lane picks its own, the PARTS lanes of an output add up
          using E = Epi<KIND>;
          using Out = typename E::Out;
          const int n_real = N / PARTS, m_real = M / PARTS;
          const int f = r & (PARTS - 1);
          int d[4 / PARTS];
          if constexpr (PARTS == 4) {
            d[0] = f == 0 ? acc[0] : f == 1 ? acc[1] : f == 2 ? acc[2] : acc[3];
          } else {
            d[0] = f == 0 ? acc[0] : acc[1];
            d[1] = f == 0 ? acc[2] : acc[3];
          }
#pragma unroll
          for (int v = 0; v < 4 / PARTS; ++v) {
            d[v] += __shfl_xor(d[v], 1, 64);
            if constexpr (PARTS == 4) d[v] += __shfl_xor(d[v], 2, 64);
          }
          const int m = r / PARTS;
          const int n_first = strip * (16 / PARTS) + g * (4 / PARTS);
          Out* C = reinterpret_cast<Out*>(p.C);
#pragma unroll
          for (int v = 0; v < 4 / PARTS; ++v) {
            Out o = E::apply(d[v], E::bias_term(bias_pre[v], p.beta), p.alpha);
            if constexpr (E::kAccumulate) o = old_pre[v] + o;
            if (f == 0 && m < m_real && n_first + v < n_real) C[(size_t)m * n_real + n_first + v] = o;
          }
          acc = v4i{0, 0, 0, 0};
          continue;
        }
        const int b = strip / strips_per_batch;
        if (GROUPED) {
          GemmParams q = p;  // problem b of the group as a one-batch problem
          q.bias = grp.bias[b];
          q.C = grp.C[b];
          q.alpha = grp.alpha[b];
          q.beta = grp.beta[b];
          store_skinny_tile_pre<KIND>(acc, q, 0, r, (strip - b * strips_per_batch) * 16 + 4 * g, bias_pre, old_pre,
                                      r < M);
        } else {
          store_skinny_tile_pre<KIND>(acc, p, b, r, (strip - b * strips_per_batch) * 16 + 4 * g, bias_pre, old_pre,
                                      r < M);
        }
      }
      // the next write to red[] is at least one workgroup barrier (top of the next block) away
      acc = v4i{0, 0, 0, 0};
    }
  };
  if (wave == 0) run(std::true_type{});
  else run(std::false_type{});
  __builtin_amdgcn_s_waitcnt(0x0F70);  // trailing filler copies must land before the LDS is released
}

// ---------------------------------------------------------------------------
// One row of activations (a decode step at batch 1) against W[N][K], K % 1024 == 0: dot products on the vector
// ALUs (v_dot4_i32_i8) instead of the matrix cores, whose 16x16 tiles would be fifteen sixteenths padding here
// and, worse, force the weights to be read as strips of 16 rows.  A wave owns one weight row at a time and reads it
// flat: every load instruction fetches 1 KiB of consecutive bytes (64 lanes x 16), non-temporal, eight in flight
// per wave -- the access shape with which a read-only pass reaches 6.5-6.9 TB/s on this chip, where strips of 16
// rows reach 5.9-6.7 and less when the rows lie a multiple of 4 KiB apart.  The activation row lives in the LDS;
// lane l multiplies its 16 weight bytes of a block with bytes 16 l .. 16 l + 15 of the same block of x.  At the end
// of a row the 64 lanes add up (integer sums: the bits are those of every other kernel) and lane 0 applies the
// epilogue.  A workgroup is four waves on four consecutive rows; blockIdx.y = problem of a GemmGroup.
// 1x20480x5120 19.5 -> 18.2 us, 1x5120x5120 8.2 -> 6.4, 1x9216x9216 17.7 -> 16.0, 1x36864x9216 52.6 -> 50.3.
static constexpr int GEMV_LOADS = 8;
template <int KIND, bool GROUPED>
__global__ __launch_bounds__(256) void gemm_gemv_kernel(GemmParams p, GemmGroup grp) {
  using E = Epi<KIND>;
  using Out = typename E::Out;
  using BiasT = typename E::Bias;
  extern __shared__ __attribute__((aligned(16))) char xs[];  // [K]
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int N = p.N, K = p.K, KB = K >> 10;
  const int prob = GROUPED ? blockIdx.y : 0;
  const int n = blockIdx.x * 4 + wave;
  const int nc = n < N ? n : N - 1;  // a wave past the last row repeats it and stores nothing
  const int8_t* B = GROUPED ? grp.B[prob] : p.B;
  const char* row = reinterpret_cast<const char*>(B) + (size_t)nc * p.ldb + lane * 16;
  // the first weight loads fly while the activation row is staged
  v4i w[GEMV_LOADS];
#pragma unroll
  for (int u = 0; u < GEMV_LOADS; ++u)
    w[u] = u < KB ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(row + (size_t)u * 1024)) : v4i{0, 0, 0, 0};
  // the epilogue's memory operands as well (lane 0 uses them)
  const BiasT* bias = reinterpret_cast<const BiasT*>(GROUPED ? grp.bias[prob] : p.bias);
  Out* C = reinterpret_cast<Out*>(GROUPED ? grp.C[prob] : p.C);
  Out* dst = C + out_index(p, 0, nc);
  BiasT bv = BiasT(0);
  if constexpr (E::kHasBias) bv = bias[nc];
  Out old = Out(0);
  if constexpr (E::kAccumulate) old = *dst;
  for (int i = threadIdx.x * 16; i < K; i += 256 * 16)
    *reinterpret_cast<v4i*>(xs + i) = *reinterpret_cast<const v4i*>(reinterpret_cast<const char*>(p.A) + i);
  __syncthreads();
  int acc = 0;
  for (int b0 = 0; b0 < KB; b0 += GEMV_LOADS) {
    v4i cur[GEMV_LOADS];
#pragma unroll
    for (int u = 0; u < GEMV_LOADS; ++u) cur[u] = w[u];
    if (b0 + GEMV_LOADS < KB) {
#pragma unroll
      for (int u = 0; u < GEMV_LOADS; ++u)
        w[u] = b0 + GEMV_LOADS + u < KB
                   ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(row + (size_t)(b0 + GEMV_LOADS + u) * 1024))
                   : v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < GEMV_LOADS; ++u) {
      if (b0 + u < KB) {
        const v4i xv = *reinterpret_cast<const v4i*>(xs + (b0 + u) * 1024 + lane * 16);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_sdot4(cur[u][j], xv[j], acc, false);
      }
    }
  }
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0 && n < N) {
    const float alpha = GROUPED ? grp.alpha[prob] : p.alpha;
    const float beta = GROUPED ? grp.beta[prob] : p.beta;
    Out o = E::apply(acc, E::bias_term(bv, beta), alpha);
    if constexpr (E::kAccumulate) o = old + o;
    *dst = o;
  }
}

// waves per workgroup for the skinny kernel: enough waves to cover HBM latency, at
// least one 256-byte block of K per wave
static int skinny_waves(const GemmParams& p) {
  const long long strips = (long long)((p.N + 15) / 16) * p.batch;
  long long nw = (4096 + strips - 1) / strips;
  const long long kmax = p.K / 256 > 0 ? p.K / 256 : 1;
  if (nw > kmax) nw = kmax;
  if (nw > 16) nw = 16;
  if (nw < 1) nw = 1;
  return (int)nw;
}

// Any-shape fallback (K not a multiple of 16 or operands not 16-byte aligned):
// one thread per output element, scalar loop over K.
template <int KIND>
__global__ __launch_bounds__(256) void gemm_scalar_kernel(GemmParams p) {
  using E = Epi<KIND>;
  using Out = typename E::Out;
  using BiasT = typename E::Bias;
  const long long total = (long long)p.M * p.N;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int m = (int)(idx / p.N), n = (int)(idx % p.N);
  const int8_t* a = p.A + (long long)blockIdx.z * p.strideA + (long long)m * p.K;
  const int8_t* b = p.B + (long long)blockIdx.z * p.strideB + (long long)n * p.K;
  int acc = 0;
  for (int k = 0; k < p.K; ++k) acc += (int)a[k] * (int)b[k];
  BiasT bv = BiasT(0);
  if (E::kHasBias) bv = reinterpret_cast<const BiasT*>(p.bias)[n];
  Out* C = reinterpret_cast<Out*>(p.C) + (long long)blockIdx.z * p.strideC;
  Out* at = C + out_index(p, m, n);
  *at = merge_old<E>(E::apply(acc, E::bias_term(bv, p.beta), p.alpha), at);
}

// ------------------------------------------------------------------ host side

// Raises a kernel's dynamic-LDS limit once per device.  `done` is the caller's per-instantiation bit mask of
// devices already handled; threads that race on a first call both set the attribute, which is harmless.
template <class Kern>
static int allow_lds(Kern kern, int bytes, std::atomic<unsigned long long>& done) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) dev = 0;
  const unsigned long long bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_relaxed) & bit) return TI_OK;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                     bytes);
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  done.fetch_or(bit, std::memory_order_relaxed);
  return TI_OK;
}

template <class Cfg>
static int launch_tile(const GemmParams& p, hipStream_t stream) {
  static std::atomic<unsigned long long> lds_ok{0};
  auto kern = gemm_tile_kernel<Cfg>;
  if (int rc = allow_lds(kern, Cfg::LDS_BYTES, lds_ok)) return rc;
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
  dim3 grid(tiles_m * tiles_n, 1, p.batch);
  hipLaunchKernelGGL(kern, grid, dim3(Cfg::NT), Cfg::LDS_BYTES, stream, p, tiles_m, tiles_n);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// Compute units of the current device (256 when no device answers), cached per device index.
static int num_cus() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || count <= 0) count = 256;
    n = count;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

template <class Cfg, class Kern, class... Extra>
static int launch_persistent(Kern kern, const GemmParams& p_in, hipStream_t stream, Extra... extra) {
  GemmParams p = p_in;
  // An XCD's 32 resident workgroups cover band x (32 / band) tiles per round and fetch band * BM + (32 / band) * BN
  // panel rows for them: 8 x 4 is the minimum for square tiles, 4 x 8 for tiles that are much taller than wide
  // (256x160: 2304 rows against 2688; measured 1 % faster, 5 % with 32-bit outputs at N = 20480).
  p.band = 3 * Cfg::BN <= 2 * Cfg::BM ? 4 : 8;
  static std::atomic<unsigned long long> lds_ok{0};
  if (int rc = allow_lds(kern, Cfg::LDS_BYTES, lds_ok)) return rc;
  const int tiles_m = (p.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (p.N + Cfg::BN - 1) / Cfg::BN;
  const long long items = (long long)tiles_m * tiles_n * p.batch;
  if (items > 0x7fffffffLL) return fail(TI_ERR_INVALID_ARG, "too many output tiles (%lld)", items);
  // one resident workgroup per LDS-sized slot; a multiple of 8 keeps the XCD mapping of tile ids
  const long long slots = (long long)num_cus() * ((160 * 1024) / Cfg::LDS_BYTES);
  const int grid = (int)(items < slots ? items : slots);
  // gemm_pipe_kernel and gemm_pipe16q_kernel (the others ignore it): the tiles of a batch on one XCD when a batch has four to eight
  // of them and there are more tiles than resident workgroups (P.V of 160 heads x 512 x 512: 19.5 -> 17.7 us; with one
  // or two tiles per batch, or all tiles resident at once, the plain order is 4-7 % faster)
  p.group_batches = p.batch % 8 == 0 && tiles_m * tiles_n >= 4 && tiles_m * tiles_n <= 8 && items >= slots && grid % 8 == 0;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, p, tiles_m, tiles_n, (int)items, extra...);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// ---------------------------------------------------------------------------
// Split-K: when a problem has too few output tiles to fill the chip, K is cut
// into `splits` slices that run as the batches of one launch of the pipelined
// kernel (raw int32 output into a workspace [splits][M][N]); this kernel then
// adds the slices and applies the epilogue.  Integer partial sums make the
// result independent of the split.
template <class Cfg>
static int launch_pipe(const GemmParams& p, hipStream_t stream) {
  return launch_persistent<Cfg>(gemm_pipe_kernel<Cfg>, p, stream);
}
template <class Cfg>
static int launch_pipe2(const GemmParams& p, hipStream_t stream) {
  return launch_persistent<Cfg>(gemm_pipe2_kernel<Cfg>, p, stream);
}
template <class Cfg>
static int launch_pipe16q(const GemmParams& p, hipStream_t stream, const GemmGroup& grp = GemmGroup{}) {
  return launch_persistent<Cfg>(gemm_pipe16q_kernel<Cfg>, p, stream, grp);
}
template <class Cfg>
static int launch_pipe16(const GemmParams& p, hipStream_t stream) {
  return launch_persistent<Cfg>(gemm_pipe16_kernel<Cfg>, p, stream);
}

template <int KIND>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(GemmParams p, const int* __restrict__ ws, int splits) {
  using E = Epi<KIND>;
  using Out = typename E::Out;
  using BiasT = typename E::Bias;
  const long long total = (long long)p.M * p.N;
  const long long i0 = ((long long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i0 >= total) return;
  const BiasT* bias = reinterpret_cast<const BiasT*>(p.bias);
  // blockIdx.y = problem of a batched product: its slices follow one another in the workspace
  ws += (long long)blockIdx.y * splits * total;
  Out* C = reinterpret_cast<Out*>(p.C) + (long long)blockIdx.y * p.strideC;
  if ((p.N & 3) == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {  // four consecutive columns of one row
    v4i acc = *reinterpret_cast<const v4i*>(ws + i0);
    for (int s = 1; s < splits; ++s) acc += *reinterpret_cast<const v4i*>(ws + (long long)s * total + i0);
    const int n = (int)(i0 % p.N);
    Out* dst = C + out_index(p, (int)(i0 / p.N), n);
    Out o[4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      BiasT bv = BiasT(0);
      if (E::kHasBias) bv = bias[n + v];
      o[v] = merge_old<E>(E::apply(acc[v], E::bias_term(bv, p.beta), p.alpha), dst + v);
    }
    if (sizeof(Out) == 4) {
      using W = typename std::conditional<sizeof(Out) == 4, Out, int>::type;
      v4i w4 = {__builtin_bit_cast(int, (W)o[0]), __builtin_bit_cast(int, (W)o[1]), __builtin_bit_cast(int, (W)o[2]),
                __builtin_bit_cast(int, (W)o[3])};
      *reinterpret_cast<v4i*>(dst) = w4;
    } else {
      *reinterpret_cast<unsigned*>(dst) = (unsigned)(unsigned char)o[0] | ((unsigned)(unsigned char)o[1] << 8) |
                                          ((unsigned)(unsigned char)o[2] << 16) | ((unsigned)(unsigned char)o[3] << 24);
    }
  } else {
    for (int v = 0; v < 4 && i0 + v < total; ++v) {
      int acc = 0;
      for (int s = 0; s < splits; ++s) acc += ws[(long long)s * total + i0 + v];
      BiasT bv = BiasT(0);
      if (E::kHasBias) bv = bias[(i0 + v) % p.N];
      Out* at = C + out_index(p, (int)((i0 + v) / p.N), (int)((i0 + v) % p.N));
      *at = merge_old<E>(E::apply(acc, E::bias_term(bv, p.beta), p.alpha), at);
    }
  }
}

// Number of K slices for an (M,N,K) linear on this chip (1 = do not split) and the tile of the
// raw-int32 GEMM that computes the slices.  A small cost model fitted to measurements at OPT-13B/66B
// widths with cache-cold weights, per 64-byte K step: a 256x256 workgroup takes about 0.85 us with a CU
// to itself, 256x160 0.55 us, 256x288 0.92 us, 128x160 0.375 us, 128x288 0.6 us; a 128x128 workgroup 0.35 us alone and 0.70 us
// when two share a CU; 8 us per round for pipeline fill and epilogue (4 us for 128x160, which has half the panel
// rows to fetch and half the tile to store, 5 us for 128x288; at 512 rows or fewer they replace 256-row tiles that would need twice
// the slices for the same number of workgroups: 512x5120x5120 31 -> 25.5 us, 128x20480x5120 38 -> 34 us,
// 128x5120x20480 37 -> 32 us, 512x9216x9216 64 -> 57 us, 128x36864x9216 101 -> 83 us, while 512x5120x20480 stays with
// 256x160: 64 against 70 us); the int32 partial tiles are written
// once and read once (they mostly stay in the last-level cache), plus the second launch.  The
// unsplit candidates are in the race too, so that a shape whose 256x160 or 256x288 tiles already fill
// the chip is left to the ordinary dispatch.
//
// 128x80 tiles (four waves, one per SIMD; 0.27 us per 64-byte step with weights from HBM, 0.47 us when two share
// a CU, 2.5 us per round) are the one candidate that also stands for itself unsplit: at 512 rows and N = 5120 they
// are 256 tiles over the whole of K in ONE launch, with no partial tiles and no second launch (cache-cold
// 512x5120x5120: 29.2 -> 24.4 us, 384x5120x5120: 27.3 -> 24.3 us, 1024x5120x5120: 42.7 -> 40.1 us; split,
// 128x5120x5120: 19.6 -> 16.4 us), although a workgroup of this shape multiplies at half the rate of a 256x160 one
// (its four waves read 7 fragments from the LDS per 10 MFMAs); with K = 20480 the larger tiles win
// (512x5120x20480: 79 against 64 us).  More than three LDS stages did not help it (four to six: +1 to +3 %).
enum SplitTile { SPLIT_128 = 0, SPLIT_256 = 1, SPLIT_256x160 = 2, SPLIT_256x288 = 3, SPLIT_128x160 = 4, SPLIT_128x288 = 5,
                 SPLIT_128x80 = 6, SPLIT_128x192 = 7, SPLIT_256x192 = 8 };
// `batch` > 1: a batched product (A and B per batch); every tile count, byte count and the streaming floor scale with
// it, the one-launch form is not available, and the tile shapes are those that exist for every epilogue of the
// raw-int32 kernels.
static int choose_splits(long long M, long long N, long long K, int* tile_kind = nullptr, double* time_us = nullptr,
                         long long batch = 1) {
  if (tile_kind) *tile_kind = SPLIT_128;
  if (time_us) *time_us = -1.0;  // no estimate
  if (M <= 16 || M > 1024 || K % PBK != 0 || K < 1024) return 1;
  const double cus = num_cus();
  const long long steps = K / PBK;
  int best = 1, best_kind = SPLIT_128;
  double best_t = 1e30;
  // the 128-row forms of the tall tiles first, then by size: a later candidate must be clearly faster to replace
  // an earlier one
  // (128x192 tiles: widths that 192 divides but neither 160 nor 288 nor 80 does - 12288 and 49152, the GPT-3-sized
  // layers of upstream's scripts/bench_linear_kernels.sh - had only the 128x128 and 256x256 tiles of the 64-byte-step
  // and 32x32-block kernels to split over; 512 x 12288 outputs are exactly 256 tiles of 128x192 and run unsplit)
  // (256x192 tiles, unsplit only: 256 x 49152 or 1024 x 12288 outputs are exactly 256 of them.  Their two LDS stages
  // leave weights that come from HBM one step of cover, and the split forms lost to the 128x192 tiles: 512 x 12288 x
  // 49152 in two slices 319 against 309 us, 512 x 49152 x 12288 331 against 290 us for 256x128 tiles)
  const int order[9] = {SPLIT_128x80, SPLIT_128x160, SPLIT_128x192, SPLIT_128x288, SPLIT_128, SPLIT_256, SPLIT_256x160,
                        SPLIT_256x192, SPLIT_256x288};
  for (int oi = 0; oi < 9; ++oi) {
    const int kind = order[oi];
    const bool wide192 = kind == SPLIT_128x192;
    const bool tall192 = kind == SPLIT_256x192;
    const bool half = kind == SPLIT_128x160 || kind == SPLIT_128x288;  // 128-row forms of the two tall tiles
    const bool small = kind == SPLIT_128x80;
    const int bm = kind == SPLIT_128 || half || small || wide192 ? 128 : 256;
    const int bn = small ? 80 : wide192 || tall192 ? 192 : kind == SPLIT_128 ? 128 : kind == SPLIT_256 ? 256
                   : kind == SPLIT_256x288 || kind == SPLIT_128x288 ? 288 : 160;
    if (kind >= SPLIT_256x160 && N % bn != 0) continue;
    if ((wide192 || tall192) && (N % 160 == 0 || N % 288 == 0)) continue;  // those widths keep their tuned tiles
    const double tiles = (double)((M + bm - 1) / bm) * (double)((N + bn - 1) / bn) * (double)batch;
    for (int s = 1; s <= 16; ++s) {
      if (steps % s != 0 || steps / s < 4) continue;
      if (kind >= SPLIT_256x160 && (K / s) % QBK != 0) continue;  // these tiles step 128 bytes at a time
      if (half && s == 1) continue;                                // exist as raw-int32 kernels only
      if (tall192 && s > 1) continue;
      if (batch > 1 && s == 1 && (small || wide192 || tall192)) continue;  // unsplit batched products keep their dispatch
      // an unsplit candidate stands for what the ordinary dispatch would launch, which takes the 256-row tiles only
      // when they fill most of the chip (and 128x128 tiles otherwise)
      if (s == 1 && kind != SPLIT_128 && !small && tiles < 0.75 * cus) continue;
      if (s == 1 && (wide192 || tall192) && tiles > cus) continue;  // more than a round: left to the ordinary dispatch
      const double wgs = tiles * s;
      double rounds, step_us, fixed_us = 8.0;
      if (kind == SPLIT_128) {
        rounds = (double)(long long)((wgs + 2 * cus - 1) / (2 * cus));
        step_us = wgs <= cus ? 0.35 : 0.70;
      } else if (small) {  // two fit a CU and then share it
        rounds = wgs <= cus ? 1.0 : (double)(long long)((wgs + 2 * cus - 1) / (2 * cus));
        step_us = wgs <= cus ? 0.27 : 0.47;
        fixed_us = 2.5;
      } else {
        rounds = (double)(long long)((wgs + cus - 1) / cus);
        step_us = kind == SPLIT_256 ? 0.85 : kind == SPLIT_256x160 ? 0.55 : kind == SPLIT_256x288 ? 0.92
                  : kind == SPLIT_128x160 ? 0.375 : wide192 ? 0.41 : tall192 ? 0.66 : 0.6;
        if (half) fixed_us = kind == SPLIT_128x160 ? 4.0 : 5.0;  // fewer panel rows to fetch first, half the tile to store
        if (wide192) fixed_us = 4.5;
      }
      double t = rounds * ((double)(steps / s) * step_us + fixed_us);
      // The weights come from HBM: a workgroup keeps about `ahead` K steps of its weight rows in flight, and what
      // all resident workgroups have in flight over a 2 us round trip bounds the streaming rate (5 TB/s at most).
      const double ahead = kind == SPLIT_128 ? 4.0 : kind == SPLIT_256x160 || half || small || wide192 ? 2.5 : 1.5;
      const double step_bytes = (double)bn * (kind == SPLIT_128 ? 64.0 : 128.0);
      const double resident = wgs < cus * (kind == SPLIT_128 ? 2 : 1) ? wgs : cus * (kind == SPLIT_128 ? 2 : 1);
      double rate = resident * ahead * step_bytes / 2.0;  // bytes per us
      // 5 TB/s at most; 3.5 TB/s for the 64-byte steps of the 128x128 tiles, which ask for every line twice
      // (128x9216x36864: 110 us against 83 us with 128x288 tiles)
      // (128x80 tiles ask for 80 scattered lines per step: 3.8 TB/s, 2.4 TB/s when two workgroups share a CU:
      // 128x20480x5120 30 us, 256x20480x5120 48 us)
      const double cap = kind == SPLIT_128 ? 3.5e6 : small ? (wgs <= cus ? 3.8e6 : 2.4e6) : 5.0e6;
      if (rate > cap) rate = cap;
      const double t_stream = (double)batch * (double)N * (double)K / rate + (small ? 4.0 : 8.0);
      if (t < t_stream) t = t_stream;
      // the slices' partial tiles: written once and read once (they mostly stay in the last-level cache) plus the
      // second launch; in the one-launch form they stay in the XCD's L2 and the reading is the last workgroup's tail
      const bool one_launch = batch == 1 && kind >= SPLIT_256x160 && M % bm == 0 && s <= (kind == SPLIT_256x288 ? 2 : 4);
      if (s > 1 && one_launch) t += (double)(2 * s - 1) * M * N * 4.0 / 8.0e6 + 1.0;
      else if (s > 1) t += (double)batch * (double)(2 * s + 1) * M * N * 4.0 / 5.5e6 + 3.0;  // at 5.5 TB/s, in us
      if (t < best_t * 0.97) {  // prefer fewer slices and the smaller tile unless the gain is clear
        best_t = t;
        best = s;
        best_kind = kind;
      }
    }
  }
  if (tile_kind) *tile_kind = best_kind;
  if (time_us && best_t < 1e29) *time_us = best_t;
  return best;
}

// kernel family of the calling thread's last launch (defined in gemm_s8.hip)
extern thread_local const char* g_last_kernel;

// The raw-int32 GEMM over the K slices of a split-K linear (defined once, in gemm_s8.hip).
int launch_splitk_raw(int tile, const GemmParams& q, hipStream_t stream);

// Split-K inside one launch (defined once, in gemm_s8.hip): fills q.arrivals / q.xcc_of_id / q.xcc_error for a
// launch with `counters` arrival counters on `stream` and returns 1, or returns 0 when that form cannot be used
// here (switched off, the placement of workgroups on XCDs is not the expected one, the stream is being captured
// before the first use, too many streams or counters) - the caller then takes the two-launch form - or minus a
// TI_ERR_* code when an earlier fused launch reported a misplaced workgroup.
int fused_split_prepare(hipStream_t stream, long long counters, GemmParams& q);

// One launch of the FUSED form of the 16x16-block kernel: q.K is the slice length, q.splits the slice count.
template <class Cfg>
static int launch_fused(const GemmParams& q_in, hipStream_t stream) {
  GemmParams q = q_in;
  q.band = 3 * Cfg::BN <= 2 * Cfg::BM ? 4 : 8;
  static std::atomic<unsigned long long> lds_ok{0};
  if (int rc = allow_lds(gemm_pipe16q_kernel<Cfg>, Cfg::LDS_BYTES, lds_ok)) return rc;
  const int tiles_m = q.M / Cfg::BM, tiles_n = q.N / Cfg::BN;  // whole tiles only (the caller checked)
  const long long tiles = (long long)tiles_m * tiles_n;
  // every XCD gets the same number of workgroups: enough for its tiles x slices, at most what is resident
  const long long slots = (long long)num_cus() * ((160 * 1024) / Cfg::LDS_BYTES) / 8 * 8;
  long long grid = ((tiles + 7) / 8) * q.splits * 8;
  if (grid > slots) grid = slots;
  hipLaunchKernelGGL(gemm_pipe16q_kernel<Cfg>, dim3((unsigned)grid), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, q, tiles_m,
                     tiles_n, 0, GemmGroup{});
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// Tiles of 256 rows for a linear or batched product with M, N > 128: 256x256 (32x32 blocks), or 256x160 /
// 256x288 / 256x128 (16x16 blocks) when the width divides and they fill the CUs more evenly (2048x5120: 160 tiles
// of 256x256 but 256 of 256x160; 2048x9216: 288 tiles of 256x256 = two rounds, but exactly 256 of 256x288;
// 2048x4096: 128 of 256x256 but 256 of 256x128).  Each candidate is priced as its rate relative to the 256x256
// kernel at full occupancy, measured (128-byte steps: 0.94 for 256x160 with its three LDS stages, 0.95 for 256x288,
// 0.93 for 256x128; 64-byte steps, K not a multiple of 128: 0.78 and 0.9), times the share of CU rounds its tiles
// fill (useful outputs over the outputs the rounds of a tiling have room for: partial tiles and partial rounds both
// count as waste; batched products count tiles only, they are bound by HBM, where padding costs no bytes).  The
// 128x128 kernel (64-byte steps, two stages) runs at half that rate per CU, a little more with two workgroups on
// every CU, and takes over where few tiles of 256 rows would leave most CUs idle.
enum WideTile { WIDE_NONE = 0, WIDE_256x160, WIDE_256x288, WIDE_256x128, WIDE_256x256, WIDE_256x192 };
struct WidePick {
  int tile;       // WideTile; WIDE_NONE = leave it to the 128x128 / small-tile kernels
  double eff;     // efficiency of the choice relative to the 256x256 kernel on a full chip (0 for WIDE_NONE)
};
static WidePick pick_wide(long long M, long long N, long long K, long long batch) {
  const long long cus = num_cus();
  const long long t256 = ((M + 255) / 256) * ((N + 255) / 256) * batch;
  const long long t128 = ((M + 127) / 128) * ((N + 127) / 128) * batch;
  auto fill = [&](long long tiles, int bn) {
    const double room = (double)(((tiles + cus - 1) / cus) * cus);
    return batch == 1 ? (double)M * N / (room * 256.0 * bn) : (double)tiles / room;
  };
  const long long rows256 = (M + 255) / 256;
  const bool wide_step = K % QBK == 0;
  const double f160 = wide_step ? 0.94 : 0.78;
  const double f288 = wide_step ? 0.95 : 0.9;
  const double F192 = 0.90;
  const double e256 = fill(t256, 256);
  const double e160 = N % 160 == 0 ? f160 * fill(rows256 * (N / 160) * batch, 160) : 0.0;
  const double e288 = N % 288 == 0 ? f288 * fill(rows256 * (N / 288) * batch, 288) : 0.0;
  // The 256x128 tiles and the comparison with the 128x128 kernel are for linears with a K of some length
  // (the rates above were measured at K >= 4096; at K = 768 the 128x128 kernel's short prologue wins); batched
  // products keep their tuned 256x256 / 128x128 choice, they are bound by HBM, not by the matrix pipe.
  // (a batched product with an inner dimension that long is a stack of linears, not an attention product, and is
  // priced like them: 8 x 1024 x 1024 x 12288 makes 256 tiles of 256x128 where it made 128 of 256x256)
  const bool priced = K >= 2048 && t128 >= 128;
  const double e128w = priced && wide_step && N % 128 == 0 ? 0.93 * fill(rows256 * (N / 128) * batch, 128) : 0.0;
  const double e128 = t128 >= 2 * cus ? 0.6 : t128 >= cus ? 0.47 : 0.47 * (double)t128 / (double)cus;
  // 256x192 (two LDS stages) for the widths that 192 divides but 160 and 288 do not (12288, 49152: 512 x 49152
  // outputs are 512 tiles, two full rounds, where 256x256 tiles make 384, a round and a half)
  const double e192 = priced && wide_step && N % 192 == 0 && N % 160 != 0 && N % 288 != 0
                          ? F192 * fill(rows256 * (N / 192) * batch, 192) : 0.0;
  const double best_other = e256 > e160 ? (e256 > e288 ? (e256 > e128w ? e256 : e128w) : (e288 > e128w ? e288 : e128w))
                                  : (e160 > e288 ? (e160 > e128w ? e160 : e128w) : (e288 > e128w ? e288 : e128w));
  const double best = best_other > e192 ? best_other : e192;
  if (!(t256 >= 160 || (priced && best > e128))) return WidePick{WIDE_NONE, 0.0};
  if (e192 > best_other * 1.03) return WidePick{WIDE_256x192, e192};
  if (e160 > e256 && e160 >= e288 && e160 >= e128w) return WidePick{WIDE_256x160, e160};
  if (e288 > e256 && e288 >= e128w) return WidePick{WIDE_256x288, e288};
  if (e128w > e256) return WidePick{WIDE_256x128, e128w};
  return WidePick{WIDE_256x256, e256};
}

// K slices for a batched product (1 = none): only where the problems together have too few 128x128 tiles to fill
// the chip twice and the inner dimension is long; attention-shaped products (K = head size, or many heads) keep
// their own dispatch.
static int batched_splits(long long batch, long long M, long long N, long long K, int* tile_kind = nullptr) {
  if (tile_kind) *tile_kind = SPLIT_128;
  if (batch <= 1 || M <= 16 || M > 1024 || N <= 16 || K < 2048 || K % PBK != 0) return 1;
  const long long t128 = ((M + 127) / 128) * ((N + 127) / 128) * batch;
  if (t128 >= 2 * (long long)num_cus()) return 1;
  return choose_splits(M, N, K, tile_kind, nullptr, batch);
}

// Rows to cut off the end of a linear with many rows and run as a second, small problem (0 = none).
// A tiled GEMM pays for whole tiles and whole rounds of 256 CUs: 2112 rows (a 4 x 528-token prefill; prefill lengths
// are padded to 16, not to 256) are nine row tiles where 2048 rows are eight, 288 tiles of 256x160 instead of 256 - a
// second round for 64 rows.  When the rows beyond the last multiple of 256 are few, the first M - r rows run on the
// tiling that suits them and the r rows left over as a problem of their own through the split-K forms, if the cost
// model prices the pair clearly below the whole.  Times in us: a tiling of efficiency e takes M N K / e at the 256x256
// kernel's rate (0.85 us per 64-byte step and 256 tiles) plus 8 us of fill and epilogue; the small problem is priced
// by choose_splits (its workspace must have been given), rows <= 16 as weight streaming at 4.5 TB/s.
static int row_split_rows(long long M, long long N, long long K, long long* rest_ws_bytes = nullptr) {
  if (rest_ws_bytes) *rest_ws_bytes = 0;
  static const bool enabled = [] {  // TORCH_INT_ROW_SPLIT=0 keeps every linear in one piece
    const char* v = getenv("TORCH_INT_ROW_SPLIT");
    return !(v && v[0] == '0');
  }();
  if (!enabled) return 0;
  const long long r = M % 256;
  if (M <= 1024 || r == 0 || r > 128 || N <= 128 || K % QBK != 0 || K < 1024) return 0;
  const WidePick whole = pick_wide(M, N, K, 1), main = pick_wide(M - r, N, K, 1);
  if (whole.tile == WIDE_NONE || main.tile == WIDE_NONE) return 0;
  auto tiled_us = [&](long long rows, double eff) {
    return (double)rows * (double)N * (double)(K / 64) * 0.85 / (65536.0 * (double)num_cus() * eff) + 8.0;
  };
  double rest_us = 0.0;
  long long need = 0;
  if (r <= 16) {
    rest_us = (double)N * (double)K / 4.5e6 + 4.0;
  } else {
    int tile = 0;
    const int splits = choose_splits(r, N, K, &tile, &rest_us);
    if (rest_us < 0.0) return 0;
    need = splits > 1 ? (long long)splits * r * N * 4 : 0;
  }
  if (tiled_us(M - r, main.eff) + rest_us + 3.0 >= 0.95 * tiled_us(M, whole.eff)) return 0;
  if (rest_ws_bytes) *rest_ws_bytes = need;
  return (int)r;
}

template <int KIND, bool GROUPED>
static int launch_gemv(const GemmParams& p, const GemmGroup& grp, int problems, hipStream_t stream) {
  static std::atomic<unsigned long long> lds_ok{0};
  if (int rc = allow_lds(gemm_gemv_kernel<KIND, GROUPED>, 48 * 1024, lds_ok)) return rc;
  hipLaunchKernelGGL((gemm_gemv_kernel<KIND, GROUPED>), dim3((unsigned)((p.N + 3) / 4), (unsigned)problems), dim3(256),
                     (size_t)p.K, stream, p, grp);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
  return TI_OK;
}
// the shapes the kernel takes: one row, one batch, whole KiB blocks, a row of x that the LDS holds thrice over
static inline bool gemv_takes(const GemmParams& p) {
  return p.M == 1 && p.batch == 1 && p.K % 1024 == 0 && p.K <= 48 * 1024 && p.lda == p.K;
}

// Stages and resident workgroups of the streaming kernel.  One row: three stages of 17 KiB with two workgroups per
// CU read cold weights 3-6 % faster than two stages with three or four (1x20480x5120 20.1 -> 19.0 us, 1x36864x9216
// 54.2 -> 52.3 us) -- unless the strips then fall into rounds that leave CUs idle (576 strips on 512 workgroups:
// 62.5 against 58.3 us), where two stages with three workgroups (768) stay.  Five to sixteen rows: two stages of
// 32 KiB with two workgroups per CU, except where one workgroup per CU with three stages quantises much better
// (16x9216x36864, 576 strips: 86.9 -> 75.0 us).  Two to four rows keep two stages and three workgroups.
static inline bool stream_deep_pipeline(int M, long long strips, int cus) {
  auto waste = [&](long long slots) {  // work of the fullest workgroup slot over the mean
    if (strips <= slots) return 1.0;
    return (double)((strips + slots - 1) / slots * slots) / (double)strips;
  };
  if (M == 1) return waste(2LL * cus) <= 1.15 * waste(3LL * cus);
  if (M > 4) return waste(2LL * cus) >= 1.3 * waste(1LL * cus);
  return false;
}

template <int KIND>
int launch_kind(const GemmParams& p, void* workspace, long long workspace_bytes, hipStream_t stream) {
  using Out = typename Epi<KIND>::Out;
  const bool aligned = (p.K % 16 == 0) && ((reinterpret_cast<uintptr_t>(p.A) & 15) == 0) &&
                       ((reinterpret_cast<uintptr_t>(p.B) & 15) == 0) &&
                       (p.strideA % 16 == 0) && (p.strideB % 16 == 0);  // the stores check C themselves
  if (!aligned) {
    g_last_kernel = "scalar";
    const long long total = (long long)p.M * p.N;
    dim3 grid((unsigned)((total + 255) / 256), 1, p.batch);
    hipLaunchKernelGGL(gemm_scalar_kernel<KIND>, grid, dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
    return TI_OK;
  }
  if (p.M <= 16 && p.K % SBK == 0 && (long long)((p.N + 15) / 16) * p.batch >= 256) {
    g_last_kernel = "stream";
    const int spb = (p.N + 15) / 16;
    const long long strips = (long long)spb * p.batch;
    if (strips > 0x7fffffffLL) return fail(TI_ERR_INVALID_ARG, "too many output strips (%lld)", strips);
    const int cus = num_cus();
    auto launch = [&](auto kern, int stages, int rows, int per_cu) -> int {
      const int lds = stages * rows * SBK + S_RED;
      static std::atomic<unsigned long long> lds_ok{0};  // one mask per kernel instantiation (the lambda is generic)
      if (int rc = allow_lds(kern, lds, lds_ok)) return rc;
      const long long slots = (long long)cus * per_cu;
      hipLaunchKernelGGL(kern, dim3((unsigned)(strips < slots ? strips : slots)), dim3(256), lds, stream, p, spb,
                         (int)strips, GemmGroup{});
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
      return TI_OK;
    };
    // Few, long weight rows (fc2 of a decode step: 1x5120x20480, 1x9216x36864): the view of the problem in which
    // every row is cut into four (two rows of activations: two) parts has that many times the strips, and its rows
    // lie a part instead of a whole row apart, which spreads the 16 rows of a strip over the memory channels
    // (a multiple of 4 KiB between them does not): 1x5120x20480 22.4 -> 19.6 us, 1x9216x36864 58.5 -> 52.2 us,
    // 2x5120x20480 23.9 -> 20.1 us.
    const int parts = p.batch == 1 && p.out_d == 0 && p.m_base == 0 && p.lda == p.K && p.ldb == p.K && p.N % 16 == 0 &&
                              p.K >= 8192 && spb <= 4 * cus
                          ? (p.M == 1 && p.K % 4096 == 0 && p.K % 16384 != 0       ? 4
                             : p.M == 2 && p.K % 2048 == 0 && p.K % 8192 != 0 ? 2
                                                                              : 1)
                          : 1;  // not when the parts are again a multiple of 4 KiB apart (1x4096x16384: 13.5 -> 15.1 us)
    // one row of activations: the flat-reading dot-product kernel, except against the few very long rows where the
    // view with rows cut into parts is ahead (1x9216x36864: 52.2 against 54.6 us; 1x5120x20480: 19.6 against 18.5)
    if (gemv_takes(p) && !(parts > 1 && p.K > 24 * 1024)) {
      g_last_kernel = "gemv";
      return launch_gemv<KIND, false>(p, GemmGroup{}, 1, stream);
    }
    if (parts > 1) {
      g_last_kernel = "stream_parts";
      GemmParams q = p;
      q.M = p.M * parts;
      q.N = p.N * parts;
      q.K = q.lda = q.ldb = p.K / parts;
      const int view_strips = q.N / 16;
      auto launch_view = [&](auto kern) -> int {
        const int lds = 2 * 20 * SBK + S_RED;
        static std::atomic<unsigned long long> lds_ok{0};
        if (int rc = allow_lds(kern, lds, lds_ok)) return rc;
        const long long slots = 3LL * cus;
        hipLaunchKernelGGL(kern, dim3((unsigned)(view_strips < slots ? view_strips : slots)), dim3(256), lds, stream, q,
                           view_strips, view_strips, GemmGroup{});
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
        return TI_OK;
      };
      return parts == 4 ? launch_view(gemm_stream_kernel<KIND, 4, 2, false, 4>)
                        : launch_view(gemm_stream_kernel<KIND, 4, 2, false, 2>);
    }
    const bool deep = stream_deep_pipeline(p.M, strips, cus);
    if (p.M == 1) return deep ? launch(gemm_stream_kernel<KIND, 1, 3>, 3, 17, 2) : launch(gemm_stream_kernel<KIND, 1, 2>, 2, 17, 3);
    if (p.M <= 4) return launch(gemm_stream_kernel<KIND, 4, 2>, 2, 20, 3);
    return deep ? launch(gemm_stream_kernel<KIND, 16, 3>, 3, 32, 1) : launch(gemm_stream_kernel<KIND, 16, 2>, 2, 32, 2);
  }
  if (p.M <= 16) {
    g_last_kernel = "skinny";
    const int nw = skinny_waves(p);
    dim3 grid((p.N + 15) / 16, 1, p.batch);
    const size_t lds = (size_t)(nw - 1) * 256 * sizeof(int);
    // blocks of K per wave decide how many loads are worth batching
    const int blocks_per_wave = p.K / 256 / nw;
    if (blocks_per_wave >= 4)
      hipLaunchKernelGGL((gemm_skinny_kernel<4, KIND>), grid, dim3(64 * nw), lds, stream, p);
    else if (blocks_per_wave >= 2)
      hipLaunchKernelGGL((gemm_skinny_kernel<2, KIND>), grid, dim3(64 * nw), lds, stream, p);
    else
      hipLaunchKernelGGL((gemm_skinny_kernel<1, KIND>), grid, dim3(64 * nw), lds, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "gemm launch: %s", hipGetErrorString(e));
    return TI_OK;
  }
  if (p.batch > 1 && p.batch <= 65535 && p.lda == p.K && p.ldb == p.K && p.out_d == 0 && workspace != nullptr &&
      (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
    // A batched product with few output tiles and a long inner dimension (upstream's benchmark/bench_bmm.py multiplies
    // [batch, seq, 12288] operands): K slices as for the linears, the slices of all problems being the batches of one
    // raw-int32 launch, then one reduction launch.
    int tile = SPLIT_128;
    const int splits = batched_splits(p.batch, p.M, p.N, p.K, &tile);
    const long long need = (long long)splits * p.batch * p.M * p.N * 4;
    if (splits > 1 && workspace_bytes >= need) {
      g_last_kernel = tile == SPLIT_128      ? "splitk_128x128"
                      : tile == SPLIT_256    ? "splitk_256x256"
                      : tile == SPLIT_256x160 ? "splitk_256x160"
                      : tile == SPLIT_128x160 ? "splitk_128x160"
                      : tile == SPLIT_128x288 ? "splitk_128x288"
                      : tile == SPLIT_128x80  ? "splitk_128x80"
                      : tile == SPLIT_128x192 ? "splitk_128x192"
                                              : "splitk_256x288";
      GemmParams q = p;
      q.K = p.K / splits;
      q.kslices = splits;
      q.strideAk = q.K;
      q.strideBk = q.K;
      q.batch = p.batch * splits;
      q.strideC = (long long)p.M * p.N;
      q.C = workspace;
      q.bias = nullptr;
      if (int rc = launch_splitk_raw(tile, q, stream)) return rc;
      const long long quads = ((long long)p.M * p.N + 3) / 4;
      hipLaunchKernelGGL(splitk_reduce_kernel<KIND>, dim3((unsigned)((quads + 255) / 256), (unsigned)p.batch), dim3(256), 0,
                         stream, p, static_cast<const int*>(workspace), splits);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "split-K reduce launch: %s", hipGetErrorString(e));
      return TI_OK;
    }
  }
  if (p.batch == 1 && p.lda == p.K && p.ldb == p.K && p.M > 1024) {
    // many rows, a few of them beyond the last multiple of 256: two problems (see row_split_rows)
    long long need = 0;
    const int r = row_split_rows(p.M, p.N, p.K, &need);
    if (r > 0 && (need == 0 || (workspace != nullptr && workspace_bytes >= need))) {
      GemmParams head = p;
      head.M = p.M - r;
      if (int rc = launch_kind<KIND>(head, workspace, workspace_bytes, stream)) return rc;
      static thread_local char label[96];
      const int used = snprintf(label, sizeof(label), "%s+", g_last_kernel);
      GemmParams rest = p;
      rest.M = r;
      rest.A = p.A + (long long)head.M * p.lda;
      if (p.out_d == 0) rest.C = static_cast<Out*>(p.C) + (long long)head.M * p.N;
      else rest.m_base = p.m_base + head.M;
      if (int rc = launch_kind<KIND>(rest, workspace, workspace_bytes, stream)) return rc;
      if (used > 0 && used < (int)sizeof(label)) snprintf(label + used, sizeof(label) - used, "%s", g_last_kernel);
      g_last_kernel = label;
      return TI_OK;
    }
  }
  if (p.batch == 1 && p.lda == p.K && p.ldb == p.K) {
    int tile = SPLIT_128;
    const int splits = choose_splits(p.M, p.N, p.K, &tile);
    const long long need = (long long)splits * p.M * p.N * 4;
    if (splits == 1 && tile == SPLIT_128x80) {
      g_last_kernel = "pipe16_128x80";
      return launch_pipe16q<Pipe16QCfg<128, 80, 4, 1, KIND>>(p, stream);
    }
    if (splits == 1 && tile == SPLIT_128x192) {
      g_last_kernel = "pipe16_128x192";
      return launch_pipe16q<Pipe16QCfg<128, 192, 4, 2, KIND>>(p, stream);
    }
    if (splits == 1 && tile == SPLIT_256x192) {
      g_last_kernel = "pipe16_256x192";
      return launch_pipe16q<Pipe16QCfg<256, 192, 4, 2, KIND>>(p, stream);
    }
    if (splits > 1 && workspace != nullptr && workspace_bytes >= need &&
        (reinterpret_cast<uintptr_t>(workspace) & 15) == 0) {
      g_last_kernel = tile == SPLIT_128      ? "splitk_128x128"
                      : tile == SPLIT_256    ? "splitk_256x256"
                      : tile == SPLIT_256x160 ? "splitk_256x160"
                      : tile == SPLIT_128x160 ? "splitk_128x160"
                      : tile == SPLIT_128x288 ? "splitk_128x288"
                      : tile == SPLIT_128x80  ? "splitk_128x80"
                      : tile == SPLIT_128x192 ? "splitk_128x192"
                                              : "splitk_256x288";
      // not for the accumulating epilogue: its reads of the old outputs, done by one workgroup per tile instead of
      // by the whole chip in the reduction kernel, cost more than the launch saved (512x9216x36864: 288 against
      // 178 us, 256x5120x5120: 29 against 22 us)
      if constexpr (KIND != EPI_S32_RAW && KIND != EPI_F32_BIAS_ACC) {
        // one launch when the tile is one of the 16x16-block kernel's and covers M in whole tiles
        const int bm = tile == SPLIT_256x160 || tile == SPLIT_256x288 ? 256 : 128;
        const int bn = tile == SPLIT_128x80 ? 80 : tile == SPLIT_128x192 ? 192
                       : tile == SPLIT_256x160 || tile == SPLIT_128x160 ? 160 : 288;
        const bool tall = tile == SPLIT_128x80 || tile == SPLIT_128x160 || tile == SPLIT_128x288 ||
                          tile == SPLIT_256x160 || tile == SPLIT_256x288 || tile == SPLIT_128x192;
        // up to four slices: the wave that arrives last reads the others' accumulators one slice after the other,
        // and beyond four that tail costs more than the reduction launch it saves (measured: 2 slices -3 to -12 %,
        // 4 slices -3 to -8 %, 7 and 8 slices +3 to +6 %)
        // (256x288 tiles, which spill registers, with two slices only: 512x9216x36864 in four slices 181 against 179 us)
        // (a workspace on a 256-byte boundary only: the 1 KiB regions the waves park and read back must not share a
        // 128-byte line with a neighbour's, or a line fetched for one region could be reused, stale, for the next)
        if (tall && splits <= (tile == SPLIT_256x288 ? 2 : 4) && p.M % bm == 0 && p.N % bn == 0 &&
            (reinterpret_cast<uintptr_t>(workspace) & 255) == 0) {
          const long long tiles = (long long)(p.M / bm) * (p.N / bn);
          GemmParams f = p;
          f.K = p.K / splits;
          f.strideA = f.K;
          f.strideB = f.K;
          f.strideC = 0;
          f.splits = splits;
          f.parts = workspace;
          const int usable = fused_split_prepare(stream, tiles * 8, f);
          if (usable < 0) return -usable;
          if (usable) {
            switch (tile) {
              case SPLIT_128x80:
                g_last_kernel = "fusedk_128x80";
                return launch_fused<Pipe16QCfg<128, 80, 4, 1, KIND, false, 3, true>>(f, stream);
              case SPLIT_128x160:
                g_last_kernel = "fusedk_128x160";
                return launch_fused<Pipe16QCfg<128, 160, 4, 2, KIND, false, 3, true>>(f, stream);
              case SPLIT_128x192:
                g_last_kernel = "fusedk_128x192";
                return launch_fused<Pipe16QCfg<128, 192, 4, 2, KIND, false, 3, true>>(f, stream);
              case SPLIT_128x288:
                g_last_kernel = "fusedk_128x288";
                return launch_fused<Pipe16QCfg<128, 288, 4, 2, KIND, false, 3, true>>(f, stream);
              case SPLIT_256x160:
                g_last_kernel = "fusedk_256x160";
                return launch_fused<Pipe16QCfg<256, 160, 4, 2, KIND, false, 3, true>>(f, stream);
              default:
                g_last_kernel = "fusedk_256x288";
                return launch_fused<Pipe16QCfg<256, 288, 4, 2, KIND, false, 3, true>>(f, stream);
            }
          }
        }
      }
      GemmParams q = p;  // the K slices are the batches of one raw-int32 GEMM into the workspace
      q.K = p.K / splits;
      q.batch = splits;
      q.strideA = q.K;
      q.strideB = q.K;
      q.strideC = (long long)p.M * p.N;
      q.C = workspace;
      q.bias = nullptr;
      q.out_T = q.out_d = 0;  // the partial products are plain [splits][M][N]; only the reduction permutes
      const int rc = launch_splitk_raw(tile, q, stream);
      if (rc) return rc;
      const long long quads = ((long long)p.M * p.N + 3) / 4;
      hipLaunchKernelGGL(splitk_reduce_kernel<KIND>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream, p,
                         static_cast<const int*>(workspace), splits);
      hipError_t e = hipGetLastError();
      if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "split-K reduce launch: %s", hipGetErrorString(e));
      return TI_OK;
    }
  }
  // 8-bit outputs take the orientation whose lanes own 16 consecutive columns.
  constexpr bool SWAP = sizeof(Out) == 1;
  const long long t256 = (long long)((p.M + 255) / 256) * ((p.N + 255) / 256) * p.batch;
  const long long t128 = (long long)((p.M + 127) / 128) * ((p.N + 127) / 128) * p.batch;
  if (p.K % PBK == 0 && p.K >= PBK) {
    // a 256-wide tile on a narrow or short output would mostly multiply padding
    const bool wide = p.N > 128 && p.M > 128;
    if (wide) {
      // Measured with pick_wide's rule against the one before it, which looked at the count of 256x256 tiles only and
      // sent everything under 160 of them to the 128x128 kernel: 1600x5120x20480 290 -> 161 us, 1600x5120x5120
      // 76 -> 47, 2048x4096x4096 48 -> 35, 2048x4096x16384 170 -> 118, 2048x2560x2560 25 -> 20, 2048x12288x12288
      // 285 -> 253.
      const bool wide_step = p.K % QBK == 0;
      switch (pick_wide(p.M, p.N, p.K, p.batch).tile) {
        case WIDE_256x160:
          g_last_kernel = "pipe16_256x160";
          if (wide_step) return launch_pipe16q<Pipe16QCfg<256, 160, 4, 2, KIND>>(p, stream);
          return launch_pipe16<Pipe16Cfg<256, 160, 4, 2, 5, KIND>>(p, stream);
        case WIDE_256x288:
          g_last_kernel = "pipe16_256x288";
          if (wide_step) return launch_pipe16q<Pipe16QCfg<256, 288, 4, 2, KIND>>(p, stream);
          return launch_pipe16<Pipe16Cfg<256, 288, 4, 2, 4, KIND>>(p, stream);
        case WIDE_256x128:
          g_last_kernel = "pipe16_256x128";
          return launch_pipe16q<Pipe16QCfg<256, 128, 4, 2, KIND>>(p, stream);
        case WIDE_256x192:
          g_last_kernel = "pipe16_256x192";
          return launch_pipe16q<Pipe16QCfg<256, 192, 4, 2, KIND>>(p, stream);
        case WIDE_256x256:
          g_last_kernel = "pipe_256x256";
          if (wide_step) return launch_pipe2<Pipe2Cfg<256, 256, 2, 4, KIND, SWAP>>(p, stream);  // whole cache lines per row
          return launch_pipe<PipeCfg<256, 256, 2, 4, 4, KIND, SWAP>>(p, stream);
        default:
          break;
      }
    }
    // 128-wide outputs with many rows (P.V of a long prefill): 256x128 tiles, three stages of 128-byte steps
    if (p.N == 128 && p.K % QBK == 0 && p.M >= 512 && (long long)((p.M + 255) / 256) * p.batch >= 2 * num_cus()) {
      g_last_kernel = "pipe16_256x128";
      return launch_pipe16q<Pipe16QCfg<256, 128, 4, 2, KIND>>(p, stream);
    }
    if (t128 >= 128) {
      g_last_kernel = "pipe_128x128";
      return launch_pipe<PipeCfg<128, 128, 2, 2, 4, KIND, SWAP>>(p, stream);
    }
  }
  if (t256 >= 160) {
    g_last_kernel = "tile_256x256";
    return launch_tile<TileCfg<256, 256, 2, 4, KIND, SWAP>>(p, stream);
  }
  if (t128 >= 128) {
    g_last_kernel = "tile_128x128";
    return launch_tile<TileCfg<128, 128, 2, 2, KIND, SWAP>>(p, stream);
  }
  g_last_kernel = "tile_64x64";
  return launch_tile<TileCfg<64, 64, 2, 2, KIND, SWAP>>(p, stream);
}

}  // namespace ti

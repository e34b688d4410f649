// Prefill attention for any number of keys and head sizes 64 / 128, without the fp32 score tensor in memory:
// probs = round(127 softmax(max(alpha q.k^T + mask, lowest))) and, on request, context = s8(alpha_pv probs . V).
// The bits are those of bmm_s8t_s8n_f32t -> attn_softmax_q -> bmm_s8t_s8n_s8t: the row maximum is taken over all
// keys before any exponential, and the row sum adds the exponentials in the reference order (chunk c of four
// consecutive keys belongs to partial sum c % 64, a partial sum takes its chunks in ascending order, the 64
// partial sums meet in a xor butterfly 32 .. 1).  Because the sum needs the maximum and the probabilities need the
// sum, the keys are swept three times, each sweep recomputing the int8 products (cheap on the matrix pipe):
//   sweep 1  x = max(alpha acc + mask, lowest), running row maximum, and per key tile whether anything in it can
//            have a non-zero probability (exp underflows to exactly 0 below -87);
//   sweep 2  e = exp(x - m) over the live tiles, partial sums -> 127 / sum;
//   sweep 3  e again (only in blocks of keys where some probability can round to more than 0), p = rint(e * 127 / sum),
//            and either the store of p or p . V on the spot.
// Tiles that are dead for the whole workgroup (keys above the diagonal of a causal mask) are skipped in sweeps
// 2 and 3: they add exact zeros.
//
// One workgroup of four waves per (batch * head, block of 64 query rows); a wave owns 16 query rows.  Keys go
// through the LDS in tiles of 256 (16 blocks of v_mfma_i32_16x16x64_i8 per wave): one tile is exactly one round
// of the 64 partial sums, so lane (r, g) of a wave keeps 16 partial sums (block j of a tile = chunk 4 j + g) and
// adds tile after tile to them.  Two workgroups share a CU; while one waits for its tile the other computes.
#include "ti_common.h"
#include "softmax_math.h"

namespace ti {

#define TI_GLOBAL_AS __attribute__((address_space(1)))
#define TI_LDS_AS __attribute__((address_space(3)))

constexpr int AL_ROWS = 64;      // query rows per workgroup
constexpr int AL_TILE = 256;     // keys per tile
constexpr int AL_MAX_TILES = 16; // live-tile bit mask: S <= 4096
constexpr int AL_VPITCH = AL_TILE + 16;

// 16-byte chunk c of row `row` of a panel whose rows hold D bytes sits at this chunk position
template <int D>
__device__ __forceinline__ int al_swz(int row, int c) {
  return D == 128 ? (c ^ ((row >> 1) & 7)) : (c ^ ((row >> 2) & 3));
}

// Classes of the additive mask, one per (batch, block of 64 query rows, tile of 256 keys), made once per mask by
// mask_classes_kernel and shared by every head and layer that uses the mask: MIXED = read the mask values; ZERO =
// every value is +-0 (adding it changes nothing: the mask is not read); UNIFORM = every value is the same number,
// -1e30 or below (x = alpha acc + v is then v itself for any |alpha acc| < 1e12, since half an ulp of v is above
// 3e22: the first sweep takes its maximum from one mask value and neither loads the keys nor multiplies).  Under a
// causal mask only the tiles on the diagonal are MIXED.
constexpr int MC_MIXED = 0, MC_ZERO = 1, MC_UNIFORM = 2;

__global__ __launch_bounds__(256) void mask_classes_kernel(const float* __restrict__ mask, unsigned char* __restrict__ cls,
                                                           int T, int S, int row_blocks, int ntiles) {
  const int tile = blockIdx.x % ntiles;
  const int rb = (blockIdx.x / ntiles) % row_blocks;
  const long long b = blockIdx.x / (ntiles * row_blocks);
  const int t0 = rb * AL_ROWS, k0 = tile * AL_TILE;
  const int rows = T - t0 < AL_ROWS ? T - t0 : AL_ROWS;
  const int quads = (S - k0 < AL_TILE ? S - k0 : AL_TILE) >> 2;  // S is a multiple of 16
  const float* base = mask + (b * T + t0) * (long long)S + k0;
  const int first = __float_as_int(base[0]);
  bool zero = true, same = true;
  for (int i = threadIdx.x; i < rows * quads; i += 256) {
    const int row = i / quads, qd = i - row * quads;
    const v4f v = *reinterpret_cast<const v4f*>(base + (long long)row * S + 4 * qd);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      zero = zero && v[e] == 0.0f;
      same = same && __float_as_int(v[e]) == first;
    }
  }
  const int all_zero = __syncthreads_and(zero), all_same = __syncthreads_and(same);
  if (threadIdx.x == 0)
    cls[blockIdx.x] = all_zero ? MC_ZERO : (all_same && __int_as_float(first) <= -1e30f) ? MC_UNIFORM : MC_MIXED;
}

// PART: the head size in memory (dr) is smaller than the LDS row size D; the forms for dr == D carry none of its tests.
template <int D, bool PV, bool MASKED, bool PART>
__global__ __launch_bounds__(256, 2) void attn_long_kernel(const int8_t* __restrict__ q, const int8_t* __restrict__ k,
                                                           const float* __restrict__ mask, int8_t* __restrict__ probs,
                                                           int T, int S, long long stride_q, long long stride_k,
                                                           int heads, int row_blocks, float alpha,
                                                           const int8_t* __restrict__ vt, int8_t* __restrict__ ctx,
                                                           float alpha_pv, const unsigned char* __restrict__ cls, int dr_arg) {
  const int dr = PART ? dr_arg : D;
  // dr = the head size in memory, a multiple of 16 up to D (the LDS row size, 64 or 128): rows of q, k and the
  // context are dr bytes long, V^T has dr rows; the chunks of an LDS row beyond dr hold zeros, which add nothing to
  // the integer products, and the context blocks beyond dr are computed on whatever the LDS holds and not stored.
  constexpr int CH = D / 16;       // 16-byte chunks per row
  constexpr int KS = D / 64;       // MFMAs (64 bytes of head dimension each) per block
  constexpr int RPI = 1024 / D;    // panel rows one copy instruction fills
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* qs_base = smem;                          // [64][D]
  char* ks_base = smem + AL_ROWS * D;            // [256][D]
  char* vs_base = ks_base + AL_TILE * D;         // [D][AL_VPITCH]            (PV only)
  int* flags = reinterpret_cast<int*>(vs_base + (PV ? D * AL_VPITCH : 0));  // [4] live-tile masks of the waves
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_bh = gridDim.x / row_blocks;
  const long long bh = blockIdx.x % n_bh;
  const int t0 = (row_blocks - 1 - (int)(blockIdx.x / n_bh)) * AL_ROWS;  // heaviest blocks of a causal mask first
  const int ntiles = (S + AL_TILE - 1) / AL_TILE;
  const int r = lane & 15, g = lane >> 4;
  // mask classes of this workgroup's row block (nullptr: every tile MIXED)
  const unsigned char* cls_row = MASKED && cls != nullptr ? cls + ((bh / heads) * row_blocks + t0 / AL_ROWS) * ntiles : nullptr;
  auto tile_class = [&](int tile) { return cls_row != nullptr ? (int)cls_row[tile] : MC_MIXED; };

  const int8_t* qb = q + bh * stride_q;
  const int8_t* kb = k + bh * stride_k;
  // ---- Q tile, once
  for (int i = wave; i < AL_ROWS / RPI; i += 4) {
    const int row = i * RPI + lane / CH, pos = lane % CH;
    const int t = t0 + row < T ? t0 + row : T - 1;  // rows past the end repeat the last one; never stored
    const int chunk = al_swz<D>(row, pos);
    if (!PART || chunk * 16 < dr)
      __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(qb + (long long)t * dr + (chunk << 4)),
                                       (TI_LDS_AS void*)((TI_LDS_AS char*)qs_base + i * 1024), 16, 0, 0);
    else
      *reinterpret_cast<v4i*>(qs_base + i * 1024 + lane * 16) = v4i{0, 0, 0, 0};
  }
  auto load_k_tile = [&](int tile) {
    const int k0 = tile * AL_TILE;
    const int nkeys = S - k0 < AL_TILE ? S - k0 : AL_TILE;  // a multiple of 16
    for (int i = wave; i < nkeys / RPI; i += 4) {
      const int row = i * RPI + lane / CH, pos = lane % CH;
      const int chunk = al_swz<D>(row, pos);
      if (!PART || chunk * 16 < dr)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(kb + (long long)(k0 + row) * dr + (chunk << 4)),
                                         (TI_LDS_AS void*)((TI_LDS_AS char*)ks_base + i * 1024), 16, 0, 0);
      else
        *reinterpret_cast<v4i*>(ks_base + i * 1024 + lane * 16) = v4i{0, 0, 0, 0};
    }
  };
  auto load_v_tile = [&](int tile) {
    if constexpr (PV) {
      const int k0 = tile * AL_TILE;
      const int nkeys = S - k0 < AL_TILE ? S - k0 : AL_TILE;
      const int8_t* vb = vt + bh * (long long)dr * S + k0;
      for (int i = wave; i < (D * AL_VPITCH) / 1024; i += 4) {
        const int o = i * 1024 + lane * 16;
        const int row = o / AL_VPITCH;
        int col = o - row * AL_VPITCH;
        col = col < nkeys ? col : 0;  // pad bytes and columns past the last key get a copy of chunk 0: multiplied by p = 0
        if (!PART || row < dr)  // rows of V^T beyond the head size stay as they are: their context blocks are not stored
          __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(vb + (long long)row * S + col),
                                           (TI_LDS_AS void*)((TI_LDS_AS char*)vs_base + i * 1024), 16, 0, 0);
      }
    }
  };

  const int t = t0 + wave * 16 + r;
  const int tc = t < T ? t : T - 1;
  const float* mrow = MASKED ? mask + (((bh / heads) * T + tc) * (long long)S) : nullptr;
  const float lowest = -3.402823466e+38f;
  const char* qs = qs_base + (wave * 16 + r) * D;
  const char* ks = ks_base + r * D;

  // x of one tile: acc[j][v] <- bits of max(alpha * (q . k) + mask, lowest) for block j, keys 16 j + 4 g + v
  v4i acc[16];
  v4i qf[KS];
  auto tile_scores = [&](int tile, auto nb_, bool use_mask) __attribute__((always_inline)) {
    const int nb = nb_;
    const int k0 = tile * AL_TILE;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      acc[j] = v4i{0, 0, 0, 0};
      if (j < nb) {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          const v4i kf = *reinterpret_cast<const v4i*>(ks + j * 16 * D + (al_swz<D>(r, 4 * s + g) << 4));
          acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf, qf[s], acc[j], 0, 0, 0);
        }
      }
    }
    // mask values four blocks at a time, the next four in flight while these are used
    v4f mk[2][4];
    auto fetch_mask = [&](int j0, v4f (&dst)[4]) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        dst[u] = v4f{0.f, 0.f, 0.f, 0.f};
        if (MASKED && use_mask && j0 + u < nb) dst[u] = *reinterpret_cast<const v4f*>(mrow + k0 + 16 * (j0 + u) + 4 * g);
      }
    };
    fetch_mask(0, mk[0]);
#pragma unroll
    for (int j0 = 0; j0 < 16; j0 += 4) {
      const int cur = (j0 >> 2) & 1;
      if (j0 + 4 < 16) fetch_mask(j0 + 4, mk[cur ^ 1]);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int j = j0 + u;
        if (j < nb) {
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            float x = Epi<EPI_F32_SCALE>::apply(acc[j][v], 0.0f, alpha);
            if (MASKED && use_mask) x = x + mk[cur][u][v];
            x = __builtin_fmaxf(x, lowest);  // NaN included
            acc[j][v] = __float_as_int(x);
          }
        }
      }
    }
  };
  auto blocks_of = [&](int tile) {
    const int left = S - tile * AL_TILE;
    return (left < AL_TILE ? left : AL_TILE) >> 4;
  };
  // The per-tile bodies below are generic lambdas run as body(nb) for the tile's number of key blocks, with the 16
  // of a full tile as a compile-time constant: every "block j exists" test then folds away and the fragment reads,
  // matrix instructions and mask loads of different blocks overlap instead of waiting for one another block by
  // block.  (Inlined by force: called from two places each, the lambdas would otherwise stay functions and push
  // the register arrays they capture by reference into scratch memory.)
  // the tile's copies have landed (and, PART, the zeros this wave wrote beside them); then the workgroup meets
#define TI_AL_TILE_READY()                                                                         \
  do {                                                                                             \
    if constexpr (PART) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");   \
    else asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");                             \
  } while (0)
#define TI_FOR_BLOCKS_OF(tile, body)                            \
  do {                                                          \
    const int nb_rt = blocks_of(tile);                          \
    if (nb_rt == 16) body(std::integral_constant<int, 16>{});   \
    else body(nb_rt);                                           \
  } while (0)

  // ---- sweep 1: row maximum and the largest x of every tile
  float m = lowest;
  float tmax[AL_MAX_TILES];
#pragma unroll
  for (int i = 0; i < AL_MAX_TILES; ++i) tmax[i] = lowest;
  bool have_q = false;  // the query fragments are read after the first wait that covers the copy of the Q tile
  auto read_q = [&]() {
    if (!have_q) {
#pragma unroll
      for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const v4i*>(qs + (al_swz<D>(wave * 16 + r, 4 * s + g) << 4));
      have_q = true;
    }
  };
#pragma unroll 1
  for (int tile = 0; tile < ntiles; ++tile) {
    const int mc = tile_class(tile);
    if (MASKED && mc == MC_UNIFORM) {  // every x of the tile is this one mask value (uniform over the workgroup)
      const float v = __builtin_fmaxf(mrow[tile * AL_TILE], lowest);
      m = __builtin_fmaxf(m, v);
#pragma unroll
      for (int i = 0; i < AL_MAX_TILES; ++i)
        if (i == tile) tmax[i] = v;
      continue;
    }
    __syncthreads();  // every wave is done with the previous tile
    load_k_tile(tile);
    TI_AL_TILE_READY();
    read_q();
    float top = lowest;
    auto body0 = [&](auto nb_) __attribute__((always_inline)) {
      const int nb = nb_;
      tile_scores(tile, nb_, mc != MC_ZERO);
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (j < nb)
          top = __builtin_fmaxf(top, __builtin_fmaxf(__builtin_fmaxf(__int_as_float(acc[j][0]), __int_as_float(acc[j][1])),
                                                     __builtin_fmaxf(__int_as_float(acc[j][2]), __int_as_float(acc[j][3]))));
    };
    TI_FOR_BLOCKS_OF(tile, body0);
    m = __builtin_fmaxf(m, top);
#pragma unroll
    for (int i = 0; i < AL_MAX_TILES; ++i)
      if (i == tile) tmax[i] = top;
  }
  {
    float o = __shfl_xor(m, 16, 64);
    m = m > o ? m : o;
    o = __shfl_xor(m, 32, 64);
    m = m > o ? m : o;
  }
  // tiles with something above exp's cut-off in this wave, then in the workgroup
  unsigned live_w = 0;
#pragma unroll
  for (int i = 0; i < AL_MAX_TILES; ++i)
    if (i < ntiles && __builtin_amdgcn_ballot_w64(tmax[i] - m > -87.0f) != 0) live_w |= 1u << i;
  if (lane == 0) flags[wave] = (int)live_w;
  __syncthreads();
  const unsigned live_g = (unsigned)(flags[0] | flags[1] | flags[2] | flags[3]);

  // ---- sweep 2: the row sum, in the reference order
  float part[16];
#pragma unroll
  for (int jj = 0; jj < 16; ++jj) part[jj] = 0.0f;
#pragma unroll 1
  for (int tile = 0; tile < ntiles; ++tile) {
    if (!(live_g >> tile & 1)) continue;  // uniform over the workgroup
    __syncthreads();
    load_k_tile(tile);
    TI_AL_TILE_READY();
    read_q();
    if (!(live_w >> tile & 1)) continue;  // uniform over the wave: every e is 0, p + 0 = p
    const bool use_mask = tile_class(tile) != MC_ZERO;
    auto body1 = [&](auto nb_) __attribute__((always_inline)) {
      const int nb = nb_;
      tile_scores(tile, nb_, use_mask);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        if (j < nb) {
          const float top = __builtin_fmaxf(__builtin_fmaxf(__int_as_float(acc[j][0]), __int_as_float(acc[j][1])),
                                            __builtin_fmaxf(__int_as_float(acc[j][2]), __int_as_float(acc[j][3])));
          if (__builtin_amdgcn_ballot_w64(top - m > -87.0f) != 0) {
            float p = part[j];
#pragma unroll
            for (int v = 0; v < 4; ++v) p = p + exp_nonpos(__int_as_float(acc[j][v]) - m);
            part[j] = p;
          }
        }
      }
    };
    TI_FOR_BLOCKS_OF(tile, body1);
  }
#pragma unroll
  for (int w = 8; w >= 1; w >>= 1)
#pragma unroll
    for (int jj = 0; jj < w; ++jj) part[jj] = part[jj] + part[jj + w];
  float sum = part[0];
  sum = sum + __shfl_xor(sum, 32, 64);
  sum = sum + __shfl_xor(sum, 16, 64);
  const float scale = 127.0f / sum;
  // Sweep 3 needs an exponential only where the probability can be non-zero: p = rint(e * scale) is 0 whenever
  // e * scale < 0.5.  With x - m <= ln(0.45 / scale) - 0.02 the exponential is below 0.442 / scale (its error is
  // parts per million, the logarithm's as well), the product below 0.45, the rounded value 0: skipping such values
  // changes no bit.  The row maximum itself contributes e = 1, so sum >= 1, scale <= 127 and the bound is at most
  // -5.6: in a peaked row nearly every block of sixteen keys falls under it for all sixteen rows of the wave.
  const float skip_below = __builtin_fmaxf(__logf(0.45f / scale) - 0.02f, -87.0f);

  // ---- sweep 3: probabilities, stored or multiplied with V
  v4i o[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) o[c] = v4i{0, 0, 0, 0};
  const char* vrow = vs_base + r * AL_VPITCH + 4 * g;  // V^T row (= head-dimension index) r of block c is 16 c + r
  int8_t* prow = probs != nullptr ? probs + (bh * T + tc) * (long long)S : nullptr;
#pragma unroll 1
  for (int tile = 0; tile < ntiles; ++tile) {
    const bool tile_live = live_g >> tile & 1;
    if (tile_live) {
      __syncthreads();
      load_k_tile(tile);
      load_v_tile(tile);
      TI_AL_TILE_READY();
      read_q();
    }
    const bool wave_live = live_w >> tile & 1;
    if (PV && !wave_live) continue;
    const bool use_mask = tile_class(tile) != MC_ZERO;
    auto body2 = [&](auto nb_) __attribute__((always_inline)) {
      const int nb = nb_;
      unsigned pw[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) pw[j] = 0;
      if (wave_live) {
        tile_scores(tile, nb_, use_mask);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          if (j < nb) {
            const float top = __builtin_fmaxf(__builtin_fmaxf(__int_as_float(acc[j][0]), __int_as_float(acc[j][1])),
                                              __builtin_fmaxf(__int_as_float(acc[j][2]), __int_as_float(acc[j][3])));
            if (__builtin_amdgcn_ballot_w64(top - m > skip_below) != 0) {
              unsigned w = 0;
#pragma unroll
              for (int v = 0; v < 4; ++v) {
                const float pq = __builtin_rintf(exp_nonpos(__int_as_float(acc[j][v]) - m) * scale);  // in [0, 127]
                w |= (unsigned)(int)pq << (8 * v);
              }
              pw[j] = w;
            }
          }
        }
      }
      if constexpr (PV) {
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
          // (a slice of 64 keys whose probabilities are zero in all sixteen rows of the wave adds nothing: its V^T
          // fragments are not even read)
          if (4 * sl < nb &&
              __builtin_amdgcn_ballot_w64((pw[4 * sl] | pw[4 * sl + 1] | pw[4 * sl + 2] | pw[4 * sl + 3]) != 0) != 0) {
            const v4i pa = {(int)pw[4 * sl], (int)pw[4 * sl + 1], (int)pw[4 * sl + 2], (int)pw[4 * sl + 3]};
#pragma unroll
            for (int c = 0; c < CH; ++c) {
              const char* src = vrow + c * 16 * AL_VPITCH + 64 * sl;
              const v4i vf = {*reinterpret_cast<const int*>(src), *reinterpret_cast<const int*>(src + 16),
                              *reinterpret_cast<const int*>(src + 32), *reinterpret_cast<const int*>(src + 48)};
              o[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(vf, pa, o[c], 0, 0, 0);
            }
          }
        }
      } else {
        // four consecutive keys per lane and block; dead tiles and blocks store their zeros
        int* dst = reinterpret_cast<int*>(prow + tile * AL_TILE) + g;
        if (t < T) {
#pragma unroll
          for (int j = 0; j < 16; ++j)
            if (j < nb) dst[4 * j] = (int)pw[j];
        }
      }
    };
    TI_FOR_BLOCKS_OF(tile, body2);
  }
  if constexpr (PV) {
    if (t < T) {
      const long long b = bh / heads, h = bh - b * heads;
      int* crow = reinterpret_cast<int*>(ctx + ((b * T + t) * heads + h) * (long long)dr) + g;
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        unsigned w = 0;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          w |= (unsigned)(unsigned char)Epi<EPI_S8_SCALE>::apply(o[c][v], 0.0f, alpha_pv) << (8 * v);
        if (!PART || 16 * c < dr) crow[4 * c] = (int)w;
      }
    }
  }
}

// D = the head size in memory: any multiple of 16 up to 128 (LDS rows of 64 bytes up to 64, of 128 beyond)
bool attn_long_supported(long long T, long long S, long long D) {
  return T >= 1 && D >= 16 && D <= 128 && D % 16 == 0 && S >= 16 && S % 16 == 0 && S <= (long long)AL_TILE * AL_MAX_TILES;
}

template <int D, bool PV, bool MASKED, bool PART>
static int launch_al(dim3 grid, hipStream_t stream, const int8_t* q, const int8_t* k, const float* mask, int8_t* probs,
                     int T, int S, long long stride_q, long long stride_k, int heads, int row_blocks, float alpha,
                     const int8_t* vt, int8_t* ctx, float alpha_pv, const unsigned char* cls, int dr) {
  auto kern = attn_long_kernel<D, PV, MASKED, PART>;
  constexpr int lds = AL_ROWS * D + AL_TILE * D + (PV ? D * AL_VPITCH : 0) + 16;
  static_assert(2 * lds <= 160 * 1024, "two workgroups per CU");
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_long: LDS limit: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, q, k, mask, probs, T, S, stride_q, stride_k, heads, row_blocks,
                     alpha, vt, ctx, alpha_pv, cls, dr);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_long launch: %s", hipGetErrorString(e));
  return TI_OK;
}

// vt == nullptr: probabilities into probs ([BH, T, S]).  Otherwise context into ctx ([BH / heads, T, heads * D]).
int launch_attn_long(const int8_t* q, const int8_t* k, const float* mask, int8_t* probs, long long BH, long long T,
                     long long S, long long D, long long stride_q, long long stride_k, long long heads, float alpha,
                     const int8_t* vt, int8_t* ctx, float alpha_pv, hipStream_t stream, const unsigned char* cls) {
  if (BH == 0 || T == 0) return TI_OK;
  // the UNIFORM class stands for "adding alpha acc to the mask value leaves the mask value": not for absurd scales
  if (mask == nullptr || !(alpha >= -1e12f && alpha <= 1e12f)) cls = nullptr;
  if (!attn_long_supported(T, S, D))
    return fail(TI_ERR_INVALID_ARG, "attn_long: unsupported shape (T=%lld S=%lld head_dim=%lld)", T, S, D);
  const long long row_blocks = (T + AL_ROWS - 1) / AL_ROWS;
  if (BH * row_blocks > 0x7fffffffLL || T > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "attn_long: too many row blocks (%lld)", BH * row_blocks);
  const dim3 grid((unsigned)(BH * row_blocks));
#define TI_AL_ARGS(c) \
  grid, stream, q, k, mask, probs, (int)T, (int)S, stride_q, stride_k, (int)heads, (int)row_blocks, alpha, vt, ctx, alpha_pv, c, (int)D
#define TI_AL(DD, PV, PART) \
  return mask != nullptr ? launch_al<DD, PV, true, PART>(TI_AL_ARGS(cls)) : launch_al<DD, PV, false, PART>(TI_AL_ARGS(nullptr))
  if (D == 128) {
    if (vt == nullptr) TI_AL(128, false, false);
    TI_AL(128, true, false);
  }
  if (D > 64) {
    if (vt == nullptr) TI_AL(128, false, true);
    TI_AL(128, true, true);
  }
  if (D == 64) {
    if (vt == nullptr) TI_AL(64, false, false);
    TI_AL(64, true, false);
  }
  if (vt == nullptr) TI_AL(64, false, true);
  TI_AL(64, true, true);
#undef TI_AL
#undef TI_AL_ARGS
}

// Bytes of the class array of a mask [batch, 1, T, S] (0: the shape takes no classes), and the launch that fills it.
long long attn_mask_classes_bytes(long long batch, long long T, long long S) {
  if (batch <= 0 || T <= 0 || S < 16 || S % 16 != 0 || S > (long long)AL_TILE * AL_MAX_TILES) return 0;
  return batch * ((T + AL_ROWS - 1) / AL_ROWS) * ((S + AL_TILE - 1) / AL_TILE);
}
int launch_attn_mask_classes(const float* mask, unsigned char* cls, long long batch, long long T, long long S,
                             hipStream_t stream) {
  const long long n = attn_mask_classes_bytes(batch, T, S);
  if (n == 0) return fail(TI_ERR_INVALID_ARG, "attn_mask_classes: unsupported shape (batch=%lld T=%lld S=%lld)", batch, T, S);
  if (n > 0x7fffffffLL) return fail(TI_ERR_INVALID_ARG, "attn_mask_classes: too many blocks (%lld)", n);
  hipLaunchKernelGGL(mask_classes_kernel, dim3((unsigned)n), dim3(256), 0, stream, mask, cls, (int)T, (int)S,
                     (int)((T + AL_ROWS - 1) / AL_ROWS), (int)((S + AL_TILE - 1) / AL_TILE));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_mask_classes launch: %s", hipGetErrorString(e));
  return TI_OK;
}

#undef TI_FOR_BLOCKS_OF
#undef TI_AL_TILE_READY
}  // namespace ti

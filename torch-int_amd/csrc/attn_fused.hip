// Q.K^T fused with the mask, the softmax and the int8 quantisation of the probabilities, for prefill with
// up to 576 key positions and head sizes up to 128 (any multiple of 16; the LDS rows are 64 or 128 bytes, zero-filled
// beyond the head size, so OPT-2.7B's 80 needs no padded copies of q, k and V^T): probs = round(127 softmax(max(alpha q.k^T + mask, lowest))).
// The fp32 scores (4 bytes per query-key pair written and read again by the two-kernel form) never leave
// the registers.  Arithmetic and summation order are those of attn_softmax_q on the scores of
// bmm_s8t_s8n_f32t, so the bytes are the same.
//
// One workgroup of four waves per (batch * head, block of 64 query rows).  The 64 query rows and all S key
// rows are copied to LDS once (head size 128: 128-byte rows, chunk c of row r at position c ^ ((r >> 1) & 7); head
// size 64: 64-byte rows as they are - the 16 rows a fragment read touches are one contiguous KiB).  A wave owns
// 16 query rows and all S keys: S/16 blocks of v_mfma_i32_16x16x64_i8 (keys as the row operand), after which
// lane (r, g) = (lane & 15, lane >> 4) holds, for block j, the scores of query row r and keys 16j + 4g .. +3.
// A score row is therefore spread over four lanes, each holding whole chunks of four consecutive keys, which is
// what the reference summation order is made of: chunk c belongs to partial sum c % 64, partial sums meet in a
// xor butterfly 32, 16, 8, 4, 2, 1.  Chunk c = 4j + g, so partial sum index = 4 (j % 16) + g: levels 32..4 of
// the butterfly combine values of one lane (j ^ 8, j ^ 4, j ^ 2, j ^ 1), levels 2 and 1 are the lane exchanges
// lane ^ 32 and lane ^ 16.
#include "ti_common.h"
#include "softmax_math.h"

namespace ti {

#define TI_GLOBAL_AS __attribute__((address_space(1)))
#define TI_LDS_AS __attribute__((address_space(3)))

constexpr int AF_ROWS = 64;   // query rows per workgroup
constexpr int AF_D = 128;     // largest head size (sizes the LDS limit)
constexpr int AF_MAX_S = 576;  // (64 + 576) rows of 128 bytes = 80 KiB: two workgroups per CU

// NB = key blocks of 16 the registers are sized for, a multiple of 4: 16 * (NB - 3) <= S <= 16 * NB.  All but the
// last three blocks exist whatever S is, so every test on them folds away at compile time, which leaves straight-line
// code: the fragment reads, the matrix instructions and the mask loads of different blocks overlap instead of waiting
// for one another block by block.  The last three are multiplied and evaluated like the others (on whatever the LDS
// holds beyond the K panel) and, where S ends before them, their scores are replaced by -infinity: they then take no
// part in the row maximum, their exponentials are exact zeros that are never added (a block without a live value is
// skipped), and their probabilities are zeros that meet whatever the V^T panel holds beyond S.
// PV: instead of storing the probabilities, multiply them with V right away: vt is V transposed,
// [batch*heads, head size, S]; it is copied into the LDS the K panel occupied while the softmax runs (row pitch =
// S rounded up to whole slices of 64 keys, + 16 against bank conflicts; the bytes of a row beyond S are whatever the
// LDS held and meet probabilities that are zero).  The probabilities of a 64-key slice sit in a lane as four dwords
// (keys 16i + 4g .. +3, i = 0..3); used as they are for the 16 operand bytes of lane (r, g), they fix a
// permutation of the 64 keys inside the slice, and the V fragments are gathered with the same permutation (four
// 4-byte reads), so the integer sum over the slice is the same.  The context rows are written already merged:
// ctx is [batch, T, heads * 128].
// SPEC: 1 / 2 = with / without a mask.  PAD = false: S == 16 * NB, the last three blocks exist like the others (the
// forms for 128, 256, 512 ... keys are 2 to 4 % faster without the three tests).
template <int NB, bool PV, int SPEC, int D = 128, bool PAD = true>
__global__ __launch_bounds__(256, 2) void attn_qk_softmax_q_kernel(const int8_t* __restrict__ q,
                                                                   const int8_t* __restrict__ k,
                                                                   const float* __restrict__ mask,
                                                                   int8_t* __restrict__ probs, int T, int S,
                                                                   long long stride_q, long long stride_k, int heads,
                                                                   int row_blocks, float alpha,
                                                                   const int8_t* __restrict__ vt,
                                                                   int8_t* __restrict__ ctx, float alpha_pv, int dr) {
  // dr = the head size of q, k, vt and ctx in memory (a multiple of 16, D / 2 < dr <= D); D = the LDS row size
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Workgroups are dispatched in blockIdx order: the last row blocks first (under a causal mask they have the
  // most live keys), one per (batch, head), then the next ones, so that the light blocks fill the tail.
  const int n_bh = gridDim.x / row_blocks;
  const long long bh = blockIdx.x % n_bh;
  const int t0 = (row_blocks - 1 - (int)(blockIdx.x / n_bh)) * AF_ROWS;
  static_assert(NB % 4 == 0 && (SPEC == 1 || SPEC == 2), "forms");
  const int nb = S >> 4;
  constexpr bool has_mask = SPEC == 1;
  auto exists = [&](int j) { return !PAD || j < NB - 3 || j < nb; };  // block j holds keys (j < NB)

  // ---- copies: slab i = 8 rows of [Q tile (64 rows) | K panel (S rows)], 1 KiB per wave instruction
  const int8_t* qb = q + bh * stride_q;
  const int8_t* kb = k + bh * stride_k;
  static_assert(D == 64 || D == 128, "head size");
  constexpr int CPR = D / 16;        // 16-byte chunks per row
  constexpr int RPS = 64 / CPR;      // rows per 1 KiB slab
  constexpr int SWZ = D == 128 ? 7 : 0;
  const int nc = dr >> 4;  // 16-byte chunks of a row in memory; LDS chunks beyond them hold zeros
  const int slabs = (AF_ROWS + S) / RPS;
  for (int i = wave; i < slabs; i += 4) {
    const int row = i * RPS + lane / CPR;  // row of the stacked panels
    const int pos = lane % CPR;
    const int8_t* src;
    int chunk;
    if (row < AF_ROWS) {
      const int t = t0 + row < T ? t0 + row : T - 1;  // rows past the end repeat the last one; never stored
      chunk = pos ^ ((row >> 1) & SWZ);
      src = qb + (long long)t * dr + (chunk << 4);
    } else {
      const int kr = row - AF_ROWS;
      chunk = pos ^ ((kr >> 1) & SWZ);
      src = kb + (long long)kr * dr + (chunk << 4);
    }
    if (chunk < nc)
      __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)src,
                                       (TI_LDS_AS void*)((TI_LDS_AS char*)smem + i * 1024), 16, 0, 0);
    else
      *reinterpret_cast<v4i*>(smem + i * 1024 + lane * 16) = v4i{0, 0, 0, 0};
  }
  // ---- mask rows: the values of eight blocks are fetched while the previous eight are consumed, the first
  // eight together with the operand copies
  const int r = lane & 15, g = lane >> 4;
  const int t = t0 + wave * 16 + r;
  const int tc = t < T ? t : T - 1;
  const float* mrow = has_mask ? mask + (((bh / heads) * T + tc) * (long long)S) : nullptr;
  const float lowest = -3.402823466e+38f;
  float m = lowest;
  constexpr int MG = NB < 8 || NB > 32 ? 4 : 8;  // blocks per mask group (36 blocks: the registers hold no more)
  v4f mk[2][MG];
  auto fetch_mask = [&](int j0, v4f (&dst)[MG]) {
#pragma unroll
    for (int u = 0; u < MG; ++u) {
      const int j = j0 + u;
      dst[u] = v4f{0.f, 0.f, 0.f, 0.f};
      // (a block beyond S reads the values of block 0 instead - no branch; its scores are replaced below)
      if (has_mask && j < NB) dst[u] = *reinterpret_cast<const v4f*>(mrow + (exists(j) ? 16 * j : 0) + 4 * g);
    }
  };
  fetch_mask(0, mk[0]);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");

  // ---- scores: acc[j] = q rows (16 of this wave) x key block j
  const int sw = (r >> 1) & SWZ;
  const char* qs = smem + (wave * 16 + r) * D;
  const char* ks = smem + AF_ROWS * D + r * D;
  constexpr int KS = D / 64;  // 64-byte slices of the head dimension = MFMAs per block
  v4i qf[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const v4i*>(qs + (((4 * s + g) ^ sw) << 4));
  v4i acc[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    acc[j] = v4i{0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const v4i kf = *reinterpret_cast<const v4i*>(ks + j * 16 * D + (((4 * s + g) ^ sw) << 4));
      acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf, qf[s], acc[j], 0, 0, 0);
    }
  }

  __syncthreads();  // all waves have read their fragments: the K panel may be overwritten (see the stores below)
  const int pitch = 16 * NB + 16;
  // V^T panel: D rows of pitch bytes, ending where the K panel ended (it starts inside the dead Q tile)
  char* vts = smem + (AF_ROWS + S) * D - D * pitch;
  // ---- x = max(alpha * acc + mask, lowest); row maximum
#pragma unroll
  for (int j0 = 0; j0 < NB; j0 += MG) {
    const int cur = (j0 / MG) & 1;
    if (j0 + MG < NB) fetch_mask(j0 + MG, mk[cur ^ 1]);
#pragma unroll
    for (int u = 0; u < MG; ++u) {
      const int j = j0 + u;
      if (j < NB) {
        const bool real = exists(j);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float x = Epi<EPI_F32_SCALE>::apply(acc[j][v], 0.0f, alpha);
          if (has_mask) x = x + mk[cur][u][v];
          x = __builtin_fmaxf(x, lowest);  // = x > lowest ? x : lowest, NaN included
          if (PAD && j >= NB - 3) x = real ? x : -__builtin_inff();
          m = __builtin_fmaxf(m, x);
          acc[j][v] = __float_as_int(x);
        }
      }
    }
  }
  {
    float o = __shfl_xor(m, 16, 64);
    m = m > o ? m : o;
    o = __shfl_xor(m, 32, 64);
    m = m > o ? m : o;
  }

  // V^T goes into the dead K panel now, after the last mask load: loads complete in issue order, so copies issued
  // before the mask rows would have to land before the first mask value could be used.  They run under the
  // exponentials and the quantisation and are waited for in front of P.V.
  if constexpr (PV) {
    const int8_t* vb = vt + bh * (long long)dr * S;
    const int instrs = (dr * pitch + 1023) >> 10;  // 1 KiB each; rows dr .. D-1 of the panel are never read
    for (int i = wave; i < instrs; i += 4) {
      const int o = i * 1024 + lane * 16;
      int row = o / pitch, col = o - row * pitch;
      col = col < S ? col : 0;  // the 16 pad bytes of a row receive a copy of its first chunk; never read
      if (row < dr)
        __builtin_amdgcn_global_load_lds((const TI_GLOBAL_AS void*)(vb + (long long)row * S + col),
                                         (TI_LDS_AS void*)((TI_LDS_AS char*)vts + i * 1024), 16, 0, 0);
    }
  }


  // ---- e = exp(x - m); partial sums in the reference order.  exp_nonpos returns exactly 0 below -87, so a
  // block in which no lane of the wave has anything above that (masked-out keys) skips the evaluation.
  unsigned long long live = 0;  // bit j: block j has non-zero probabilities somewhere in the wave
  float part[16];
#pragma unroll
  for (int jj = 0; jj < 16; ++jj) {
    float p = 0.0f;
#pragma unroll
    for (int h = 0; h < (NB + 15) / 16; ++h) {
      const int j = jj + 16 * h;
      if (j < NB) {
        const float top = __builtin_fmaxf(__builtin_fmaxf(__int_as_float(acc[j][0]), __int_as_float(acc[j][1])),
                                          __builtin_fmaxf(__int_as_float(acc[j][2]), __int_as_float(acc[j][3])));
        if (__builtin_amdgcn_ballot_w64(top - m > -87.0f) != 0) {
          live |= 1ull << j;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const float e = exp_nonpos(__int_as_float(acc[j][v]) - m);
            acc[j][v] = __float_as_int(e);
            p = p + e;
          }
        } else {
          // every e is 0: p + 0 = p, nothing to add
          acc[j] = v4i{0, 0, 0, 0};
        }
      }
    }
    part[jj] = p;
  }
#pragma unroll
  for (int w = 8; w >= 1; w >>= 1)
#pragma unroll
    for (int jj = 0; jj < w; ++jj) part[jj] = part[jj] + part[jj + w];
  float sum = part[0];
  sum = sum + __shfl_xor(sum, 32, 64);
  sum = sum + __shfl_xor(sum, 16, 64);
  const float scale = 127.0f / sum;

  // ---- probabilities: four consecutive keys per lane and block = one dword
  unsigned pw[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    unsigned w = 0;
    if (live >> j & 1) {
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float pq = __builtin_rintf(__int_as_float(acc[j][v]) * scale);  // in [0, 127]
        w |= (unsigned)(int)pq << (8 * v);
      }
    }
    pw[j] = w;
  }
  if constexpr (!PV) {
    // staged through the part of the K panel this wave may reuse (every wave is past the barrier above, so
    // nobody reads the panel any more) and written out as whole rows, 16 bytes per lane
    // (with 64-byte rows the four waves' 64 rows of pitch bytes are a little more than the K panel: they start in the
    // Q tile, whose fragments every wave holds in registers since before the barrier)
    char* stage = smem + (D == 128 ? AF_ROWS * D : 0) + wave * 16 * pitch;
#pragma unroll
    for (int j = 0; j < NB; ++j)
      *reinterpret_cast<unsigned*>(stage + r * pitch + 16 * j + 4 * g) = pw[j];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the wave's own LDS writes are done; its reads below follow
    const int cpr = S >> 4;                              // 16-byte chunks per row
    int8_t* pbase = probs + (bh * T + t0 + wave * 16) * (long long)S;
    for (int idx = lane; idx < 16 * cpr; idx += 64) {
      const int row = idx / cpr, c16 = idx - row * cpr;
      if (t0 + wave * 16 + row < T)
        *reinterpret_cast<v4i*>(pbase + (long long)row * S + c16 * 16) =
            *reinterpret_cast<const v4i*>(stage + row * pitch + c16 * 16);
    }
  } else {
    // ---- context = P . V: all V^T copies of the workgroup must have landed
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    v4i o[D / 16];
#pragma unroll
    for (int c = 0; c < D / 16; ++c) o[c] = v4i{0, 0, 0, 0};
    const char* vrow = vts + r * pitch + 4 * g;  // V^T row (= head-dim index) r of block c is 16c + r
#pragma unroll
    for (int sl = 0; sl < NB / 4; ++sl) {
      {
        const v4i pa = {(int)pw[4 * sl], (int)pw[4 * sl + 1], (int)pw[4 * sl + 2], (int)pw[4 * sl + 3]};
        // (blocks c >= nc multiply rows of the panel that no copy filled: whatever the LDS holds there; their
        // results are not stored.  A test on c here cost the 256-key forms their register allocation.)
#pragma unroll
        for (int c = 0; c < D / 16; ++c) {
          const char* src = vrow + c * 16 * pitch + 64 * sl;
          const v4i vf = {*reinterpret_cast<const int*>(src), *reinterpret_cast<const int*>(src + 16),
                          *reinterpret_cast<const int*>(src + 32), *reinterpret_cast<const int*>(src + 48)};
          o[c] = __builtin_amdgcn_mfma_i32_16x16x64_i8(vf, pa, o[c], 0, 0, 0);
        }
      }
    }
    if (t < T) {
      const long long b = bh / heads, h = bh - b * heads;
      int* crow = reinterpret_cast<int*>(ctx + ((b * T + t) * heads + h) * (long long)dr) + g;
#pragma unroll
      for (int c = 0; c < D / 16; ++c) {
        unsigned w = 0;
#pragma unroll
        for (int v = 0; v < 4; ++v)
          w |= (unsigned)(unsigned char)Epi<EPI_S8_SCALE>::apply(o[c][v], 0.0f, alpha_pv) << (8 * v);
        if (c < nc) crow[4 * c] = (int)w;
      }
    }
  }
}

// attn_long.hip: any number of keys up to 4096 (a multiple of 16), head size 64 or 128, three sweeps over the keys
bool attn_long_supported(long long T, long long S, long long D);
int launch_attn_long(const int8_t* q, const int8_t* k, const float* mask, int8_t* probs, long long BH, long long T,
                     long long S, long long D, long long stride_q, long long stride_k, long long heads, float alpha,
                     const int8_t* vt, int8_t* ctx, float alpha_pv, hipStream_t stream, const unsigned char* cls);

// shapes the single-sweep kernel of this file takes (all keys of a head in the LDS at once)
static bool single_sweep_ok(long long T, long long S, long long D, bool pv) {
  (void)pv;  // with or without the product with V
  return T >= 1 && D >= 16 && D <= 128 && D % 16 == 0 && S >= 16 && S <= AF_MAX_S && S % 16 == 0;
}

bool attn_qk_softmax_q_supported(long long T, long long S, long long D) {
  return single_sweep_ok(T, S, D, false) || attn_long_supported(T, S, D);
}

// the form that multiplies on with V^T
bool attn_prefill_supported(long long T, long long S, long long D) {
  return single_sweep_ok(T, S, D, true) || attn_long_supported(T, S, D);
}

template <int NB, bool PV, int SPEC, int D, bool PAD>
static int launch_af(dim3 grid, size_t lds, hipStream_t stream, const int8_t* q, const int8_t* k, const float* mask,
                     int8_t* probs, int T, int S, long long stride_q, long long stride_k, int heads, int row_blocks,
                     float alpha, const int8_t* vt, int8_t* ctx, float alpha_pv, int dr) {
  auto kern = attn_qk_softmax_q_kernel<NB, PV, SPEC, D, PAD>;
  static unsigned long long lds_ok = 0;  // bit per device: the large dynamic LDS size has been allowed
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_qk_softmax_q: no current device");
  if (dev < 64 && !(lds_ok >> dev & 1)) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (AF_ROWS + AF_MAX_S) * AF_D);
    if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_qk_softmax_q: LDS limit: %s", hipGetErrorString(e));
    lds_ok |= 1ull << dev;
  }
  hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, q, k, mask, probs, T, S, stride_q, stride_k, heads, row_blocks,
                     alpha, vt, ctx, alpha_pv, dr);
  return TI_OK;
}

// vt == nullptr: probabilities into probs.  Otherwise context into ctx ([batch, T, heads * head size]).
int launch_attn_qk_softmax_q(const int8_t* q, const int8_t* k, const float* mask, int8_t* probs, long long BH,
                             long long T, long long S, long long D, long long stride_q, long long stride_k,
                             long long heads, float alpha, const int8_t* vt, int8_t* ctx, float alpha_pv,
                             hipStream_t stream, const unsigned char* mask_classes) {
  if (BH == 0 || T == 0) return TI_OK;
  if (!single_sweep_ok(T, S, D, vt != nullptr))
    return launch_attn_long(q, k, mask, probs, BH, T, S, D, stride_q, stride_k, heads, alpha, vt, ctx, alpha_pv, stream,
                            mask_classes);
  const long long row_blocks = (T + AF_ROWS - 1) / AF_ROWS;
  if (BH * row_blocks > 0x7fffffffLL || T > 0x7fffffffLL)
    return fail(TI_ERR_INVALID_ARG, "attn_qk_softmax_q: too many row blocks (%lld)", BH * row_blocks);
  const dim3 grid((unsigned)(BH * row_blocks));
  const int row_bytes = D <= 64 ? 64 : 128;  // LDS row size = the kernel's template head size
  const int nb4 = (int)((S + 63) / 64);        // the form: NB = 4 * nb4 blocks of 16 keys
  const size_t lds = (size_t)(AF_ROWS + 64 * nb4) * row_bytes;  // the blocks beyond S are read (and not used)
  int rc;
#define TI_AF_ARGS                                                                                                   \
  (grid, lds, stream, q, k, mask, probs, (int)T, (int)S, stride_q, stride_k, (int)heads, (int)row_blocks, alpha, vt, ctx, \
   alpha_pv, (int)D)
#define TI_AF(NB, PV, SPEC)                                                                      \
  rc = row_bytes == 128 ? (S == 16 * NB ? launch_af<NB, PV, SPEC, 128, false> TI_AF_ARGS         \
                                        : launch_af<NB, PV, SPEC, 128, true> TI_AF_ARGS)         \
                        : (S == 16 * NB ? launch_af<NB, PV, SPEC, 64, false> TI_AF_ARGS          \
                                        : launch_af<NB, PV, SPEC, 64, true> TI_AF_ARGS)
#define TI_AF_NB(NB)                                  \
  case NB / 4:                                        \
    if (vt == nullptr) {                              \
      if (mask != nullptr) TI_AF(NB, false, 1);       \
      else TI_AF(NB, false, 2);                       \
    } else {                                          \
      if (mask != nullptr) TI_AF(NB, true, 1);        \
      else TI_AF(NB, true, 2);                        \
    }                                                 \
    break
  switch (nb4) {
    TI_AF_NB(4);
    TI_AF_NB(8);
    TI_AF_NB(12);
    TI_AF_NB(16);
    TI_AF_NB(20);
    TI_AF_NB(24);
    TI_AF_NB(28);
    TI_AF_NB(32);
    TI_AF_NB(36);
    default:
      return fail(TI_ERR_INVALID_ARG, "attn_qk_softmax_q: %lld keys", S);
  }
#undef TI_AF_NB
#undef TI_AF
#undef TI_AF_ARGS
  if (rc) return rc;
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TI_ERR_LAUNCH, "attn_qk_softmax_q launch: %s", hipGetErrorString(e));
  return TI_OK;
}

}  // namespace ti

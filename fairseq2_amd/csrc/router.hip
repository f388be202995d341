// Fused router: logits = x @ router (+ bias), top-k with deterministic ties, combine weights.
//
// Two logit front ends feed one selection routine:
//   * bf16: a 32-token x E tile per block on v_mfma_f32_32x32x16_bf16.  The router matrix is
//     (D, E) with E contiguous, so its tiles go through LDS and come back through the transposing
//     LDS read; products of bf16 values are exact in f32 and are summed in f32.
//   * f32: plain FMA, lane l owning experts l, l+64, ... (true f32 arithmetic, any D).
// Selection: the E logits of a token are spread across one wave (lane l holds experts l, l+64, ..),
// and the top-k is K rounds of: wave-wide maximum of a 32-bit key (an order-preserving image of the
// f32 logit; NaN ranks above +inf, as torch.topk ranks it), then a ballot of the lanes that hold
// that key, lowest expert first, so equal logits resolve to the lower expert id.
#include <cmath>
#include <cstring>

#include "common.h"
#include "dispatch_small.h"

namespace fs2moe {

__device__ __forceinline__ uint32_t order_key(float v) {
  uint32_t b = __float_as_uint(v);
  if (v != v) return 0xffffffffu;  // NaN ranks above +inf
  if (v == 0.0f) b = 0;            // -0 and +0 tie
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float order_key_inv(uint32_t k) {
  if (k == 0xffffffffu) return __uint_as_float(0x7fc00000u);
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

// One wave selects for one token.  v[j] is the logit of expert lane + 64 j (bias included).
template <int J>
__device__ __forceinline__ void select_topk(const float (&v)[J], int lane, int t, int E, int K,
                                            int score_fn, int renorm,
                                            int32_t* __restrict__ topk_idx,
                                            float* __restrict__ topk_w, int* chosen = nullptr) {
  // Keys of real logits are at least order_key(-inf) = 0x007fffff, so 0 marks "taken / no expert".
  uint32_t key[J];
#pragma unroll
  for (int j = 0; j < J; ++j) key[j] = lane + 64 * j < E ? order_key(v[j]) : 0u;
  int my_e = 0;
  float my_v = 0.f, top_v = 0.f;
  for (int r = 0; r < K; ++r) {
    uint32_t m = key[0];
#pragma unroll
    for (int j = 1; j < J; ++j) m = key[j] > m ? key[j] : m;
    const uint32_t best = wave_max_u32(m);
    // the lowest expert holding `best`: experts lane + 64 j ascend with j first
    int e = 0;
    bool found = false;
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const unsigned long long holders = __ballot(key[j] == best);
      if (!found && holders != 0ull) {
        e = 64 * j + (int)__builtin_ctzll(holders);
        found = true;
      }
    }
#pragma unroll
    for (int j = 0; j < J; ++j)
      if (lane + 64 * j == e) key[j] = 0u;
    const float val = order_key_inv(best);
    if (r == 0) top_v = val;
    if (lane == r) {
      my_e = e;
      my_v = val;
    }
  }
  float w;
  if (score_fn == FS2MOE_SCORE_SIGMOID) {
    w = 1.0f / (1.0f + expf(-my_v));
    if (renorm) {
      const float s = wave_sum_f32(lane < K ? w : 0.f);
      w = w / s;
    }
  } else {
    const float ex = expf(my_v - top_v);
    float s;
    if (renorm) {
      s = wave_sum_f32(lane < K ? ex : 0.f);
    } else {
      float part = 0.f;
#pragma unroll
      for (int j = 0; j < J; ++j)
        if (lane + 64 * j < E) part += expf(v[j] - top_v);
      s = wave_sum_f32(part);
    }
    w = ex / s;
  }
  if (lane < K) {
    topk_idx[(size_t)t * K + lane] = my_e;
    topk_w[(size_t)t * K + lane] = w;
  }
  if (chosen != nullptr) *chosen = my_e;  // lane r < K: the token's r-th expert
}

// ------------------------------------------------------------------------------------- f32 / FMA
// ---------------------------------------------------------------- RMS normalisation in front
// The pre-norm decoder layer normalises the rows before the feed-forward block
// (transformer_lm/decoder_layer.py:187-199).  The router is the first kernel to read every row, so
// it can do that on the way: each block normalises its own 32 rows into `xn`, and then routes (and
// every later stage reads) `xn`.  Arithmetic of torch.nn.functional.rms_norm, which
// RMSNorm.forward calls (nn/normalization.py:234-236): mean of squares, x * rsqrt(mean + eps) and
// the product with the weight all in f32, one rounding to the activation type at the end.
template <typename TA>
struct Pack16;  // 16 bytes of activations <-> floats
template <>
struct Pack16<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(u32x4 q, float (&v)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __uint_as_float(q[i]);
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[4]) {
    u32x4 q;
#pragma unroll
    for (int i = 0; i < 4; ++i) q[i] = __float_as_uint(v[i]);
    return q;
  }
};
template <>
struct Pack16<uint16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4 q, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(q[i] << 16);
      v[2 * i + 1] = __uint_as_float(q[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float (&v)[8]) {
    u32x4 q;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      q[i] = (uint32_t)f32_to_bf16_bits(v[2 * i]) | ((uint32_t)f32_to_bf16_bits(v[2 * i + 1]) << 16);
    return q;
  }
};

// Rows t0 .. t0 + rows - 1 of the block, columns [k_lo, k_hi) written (the mean is over the whole
// row); w may be null (no elementwise weight).  A wave takes two rows at a time so that their loads
// are in flight together; rows of up to 256 16-byte chunks stay in registers between the sum of
// squares and the product, longer ones are read a second time (from cache).
template <typename TA>
__device__ __forceinline__ void rms_norm_block_rows(const TA* x, const TA* w, float eps, TA* xn, int t0, int rows,
                                    int D, int k_lo, int k_hi) {
  using P = Pack16<TA>;
  constexpr int V = P::N;
  constexpr int CACHE = 4;  // chunks per lane held in registers
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  const uintptr_t bases = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(xn) |
                          reinterpret_cast<uintptr_t>(w);
  const bool vec = D % V == 0 && (bases & 15u) == 0 && k_lo % V == 0;
  const float inv_d = 1.0f / (float)D;
  if (vec && D / V <= CACHE * kWave) {
    const int nchunk = D / V, c_lo = k_lo / V, c_hi = (k_hi + V - 1) / V;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    u32x4 g[CACHE];
    if (w != nullptr) {
#pragma unroll
      for (int i = 0; i < CACHE; ++i) {
        const int c = lane + kWave * i;
        g[i] = (c >= c_lo && c < c_hi && c < nchunk)
                   ? *reinterpret_cast<const u32x4*>(w + (size_t)c * V) : zero4;
      }
    }
    for (int r0 = wave; r0 < rows; r0 += 2 * nwaves) {
      const int r1 = r0 + nwaves < rows ? r0 + nwaves : r0;  // a missing partner repeats r0
      const TA* xr[2] = {x + (size_t)(t0 + r0) * D, x + (size_t)(t0 + r1) * D};
      u32x4 q[2][CACHE];
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
          const int c = lane + kWave * i;
          q[h][i] = c < nchunk ? *reinterpret_cast<const u32x4*>(xr[h] + (size_t)c * V) : zero4;
        }
      float rstd[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
          float v[V];
          P::unpack(q[h][i], v);
#pragma unroll
          for (int j = 0; j < V; ++j) ss += v[j] * v[j];
        }
        rstd[h] = 1.0f / sqrtf(wave_sum_f32(ss) * inv_d + eps);
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const bool row_on = h == 0 || r1 != r0;  // wave-uniform
        TA* yr = xn + (size_t)(t0 + (h == 0 ? r0 : r1)) * D;
#pragma unroll
        for (int i = 0; i < CACHE; ++i) {
          const int c = lane + kWave * i;
          if (!row_on || c < c_lo || c >= c_hi || c >= nchunk) continue;
          float v[V], gv[V];
          P::unpack(q[h][i], v);
          if (w != nullptr) P::unpack(g[i], gv);
#pragma unroll
          for (int j = 0; j < V; ++j) {
            v[j] = v[j] * rstd[h];
            if (w != nullptr) v[j] = v[j] * gv[j];
          }
          *reinterpret_cast<u32x4*>(yr + (size_t)c * V) = P::pack(v);
        }
      }
    }
    return;
  }
  for (int r = wave; r < rows; r += nwaves) {
    const TA* xr = x + (size_t)(t0 + r) * D;
    TA* yr = xn + (size_t)(t0 + r) * D;
    float ss = 0.f;
    if (vec) {
      for (int c = lane; c < D / V; c += kWave) {
        float v[V];
        P::unpack(*reinterpret_cast<const u32x4*>(xr + (size_t)c * V), v);
#pragma unroll
        for (int i = 0; i < V; ++i) ss += v[i] * v[i];
      }
    } else {
      for (int k = lane; k < D; k += kWave) {
        const float v = Elem<TA>::load(xr + k);
        ss += v * v;
      }
    }
    const float rstd = 1.0f / sqrtf(wave_sum_f32(ss) * inv_d + eps);
    if (vec) {
      const int c_hi = (k_hi + V - 1) / V < D / V ? (k_hi + V - 1) / V : D / V;
      for (int c = k_lo / V + lane; c < c_hi; c += kWave) {
        float v[V], g[V];
        P::unpack(*reinterpret_cast<const u32x4*>(xr + (size_t)c * V), v);
        if (w != nullptr) P::unpack(*reinterpret_cast<const u32x4*>(w + (size_t)c * V), g);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          v[i] = v[i] * rstd;
          if (w != nullptr) v[i] = v[i] * g[i];
        }
        *reinterpret_cast<u32x4*>(yr + (size_t)c * V) = P::pack(v);
      }
    } else {
      const int hi = k_hi < D ? k_hi : D;
      for (int k = k_lo + lane; k < hi; k += kWave) {
        float v = Elem<TA>::load(xr + k) * rstd;
        if (w != nullptr) v = v * Elem<TA>::load(w + k);
        Elem<TA>::store(yr + k, v);
      }
    }
  }
}

// The same normalisation as a kernel of its own, four rows per block.  Used in front of the router
// when there are so few 32-token blocks that the CUs running them would do the normalisation one
// after the other while the rest of the chip idles.
constexpr int kNormRows = 4;
template <typename TA>
__global__ __launch_bounds__(kNormRows* kWave) void rms_norm_kernel(const TA* x, const TA* w,
                                                                    float eps, TA* xn, int T,
                                                                    int D) {
  const int t0 = blockIdx.x * kNormRows;
  rms_norm_block_rows<TA>(x, w, eps, xn, t0, T - t0 < kNormRows ? T - t0 : kNormRows, D, 0, D);
}

constexpr int kRouterTok = 8;     // tokens per wave
constexpr int kRouterWaves = 4;   // waves per block
// rows of the router matrix staged at a time: 64 (one per lane of the token rows' loads) while the
// f32 stage fits the 64 KB of static LDS, i.e. up to 256 experts, else 32
template <int J>
constexpr int router_chunk() { return J <= 4 ? 64 : 32; }

template <typename TA, int J>
__global__ __launch_bounds__(kRouterWaves* kWave) void router_fma_kernel(
    const TA* x, const TA* norm_w, float norm_eps, TA* xn, const TA* __restrict__ router,
    const float* __restrict__ bias, int T, int D, int E, int K, int score_fn, int renorm,
    int32_t* __restrict__ topk_idx, float* __restrict__ topk_w, float* __restrict__ logits) {
  constexpr int EP = 64 * J;
  constexpr int kRouterChunk = router_chunk<J>();
  __shared__ float s_r[kRouterChunk * EP];

  const int lane = lane_id();
  const int wave = threadIdx.x / kWave;
  const int t0 = (blockIdx.x * kRouterWaves + wave) * kRouterTok;
  if (xn != nullptr) {
    const int tb = blockIdx.x * kRouterWaves * kRouterTok;
    const int rows = T - tb < kRouterWaves * kRouterTok ? T - tb : kRouterWaves * kRouterTok;
    rms_norm_block_rows<TA>(x, norm_w, norm_eps, xn, tb, rows, D, 0, D);
    __syncthreads();  // the block's rows of xn are written and visible to all its waves
    x = xn;
  }

  float acc[kRouterTok][J];
#pragma unroll
  for (int i = 0; i < kRouterTok; ++i)
#pragma unroll
    for (int j = 0; j < J; ++j) acc[i][j] = 0.f;

  for (int d0 = 0; d0 < D; d0 += kRouterChunk) {
    __syncthreads();
    for (int i = threadIdx.x; i < kRouterChunk * EP; i += kRouterWaves * kWave) {
      int dd = i / EP, e = i - dd * EP;
      float v = 0.f;
      if (d0 + dd < D && e < E) v = Elem<TA>::load(router + (size_t)(d0 + dd) * E + e);
      s_r[i] = v;
    }
    __syncthreads();

    float xv[kRouterTok];
#pragma unroll
    for (int i = 0; i < kRouterTok; ++i) {
      int t = t0 + i, d = d0 + lane;
      xv[i] = (t < T && d < D && lane < kRouterChunk) ? Elem<TA>::load(x + (size_t)t * D + d) : 0.f;
    }
#pragma unroll
    for (int dd = 0; dd < kRouterChunk; ++dd) {
      float r[J];
#pragma unroll
      for (int j = 0; j < J; ++j) r[j] = s_r[dd * EP + lane + 64 * j];
#pragma unroll
      for (int i = 0; i < kRouterTok; ++i) {
        float xb = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(xv[i]), dd));
#pragma unroll
        for (int j = 0; j < J; ++j) acc[i][j] = fmaf(xb, r[j], acc[i][j]);
      }
    }
  }

  float b[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    int e = lane + 64 * j;
    b[j] = (bias != nullptr && e < E) ? bias[e] : 0.f;
  }
#pragma unroll
  for (int i = 0; i < kRouterTok; ++i) {
    const int t = t0 + i;
    if (t >= T) break;  // wave-uniform
    float v[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int e = lane + 64 * j;
      v[j] = acc[i][j] + b[j];
      if (logits != nullptr && e < E) logits[(size_t)t * E + e] = v[j];
    }
    select_topk<J>(v, lane, t, E, K, score_fn, renorm, topk_idx, topk_w);
  }
}

// ----------------------------------------------------------------------------------- bf16 / MFMA
namespace rmfma {
constexpr int BT = 32;      // tokens per block (one MFMA tile wide)
constexpr int PADR = 32;    // sR row padding (elements)
template <int NF>
struct Shape {
  static constexpr int GROUPS = NF == 1 ? 4 : 2;  // k-groups per block (LDS allows 2 when NF = 2)
  static constexpr int THREADS = GROUPS * 256;
  static constexpr int BK = 64;                  // model-dim chunk per stage
  static constexpr int LDX = BK + 8;             // sX row stride (elements)
  static constexpr int EP = 128 * NF;            // padded expert count
  static constexpr int LDR = EP + PADR;          // sR row stride (elements)
  static constexpr int LDL = EP + 4;             // logits row stride (floats)
  static constexpr int STAGE_BYTES = (BT * LDX + BK * LDR) * 2;
  static constexpr int LOGIT_BYTES = BT * LDL * 4;
  static constexpr int GROUP_BYTES = STAGE_BYTES > LOGIT_BYTES ? STAGE_BYTES : LOGIT_BYTES;
  static constexpr int SMEM_BYTES = GROUPS * GROUP_BYTES;
};
}  // namespace rmfma

// NF = 32-expert fragments per wave (E <= 128 * NF).  The block's waves form 4 k-groups of 4 (2 when NF = 2):
// group g walks the model-dim chunks g, g+4, g+8, .. with its own LDS stage, and wave w of a group
// owns expert fragments w, w + 4, ...  A block is bound by the latency of its load -> LDS -> MFMA
// chain, not by bandwidth (one 32-token tile per CU at the sizes this runs at), so four chains
// in parallel cut it accordingly.  The partial sums meet in LDS and are added in a fixed order.
//
// SPLIT: with few tokens there are few blocks, each walking all of D behind one load latency per
// step while most CUs idle.  Then gridDim.y blocks share a token tile, block y taking a contiguous
// range of chunks, and write their sums to `partial` [gridDim.y][T][E] instead of selecting;
// router_finish_kernel adds the ranges in ascending order and selects.
template <int NF, bool SPLIT>
__global__ __launch_bounds__(rmfma::Shape<NF>::THREADS) void router_mfma_kernel(
    const uint16_t* x, const uint16_t* norm_w, float norm_eps, uint16_t* xn,
    const uint16_t* __restrict__ router, const float* __restrict__ bias, int T, int D, int E, int K,
    int score_fn, int renorm, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
    float* __restrict__ logits, float* __restrict__ partial) {
  using namespace rmfma;
  using S = Shape<NF>;
  constexpr int BK = S::BK, LDX = S::LDX, EP = S::EP, LDR = S::LDR, LDL = S::LDL;
  constexpr int GROUPS = S::GROUPS;
  constexpr int J = EP / 64;
  constexpr int R_CHUNKS = BK * EP / 8 / 256;  // 16-byte chunks of the router tile per thread
  constexpr int X_CHUNKS = BT * BK / 8 / 256;  // = 2 or 1
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid_all = threadIdx.x;
  const int group = __builtin_amdgcn_readfirstlane(tid_all >> 8);  // 0 .. GROUPS-1
  const int tid = tid_all & 255, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // within the group
  const int lr = lane & 31, lk = lane >> 5;
  const int t0 = blockIdx.x * BT;
  uint16_t* sX = reinterpret_cast<uint16_t*>(smem + group * S::GROUP_BYTES);
  uint16_t* sR = sX + BT * LDX;
  if (xn != nullptr) {
    // the columns this block goes on to read: all of them, or (SPLIT, a single token tile: the host
    // sends more tiles than that through rms_norm_kernel first) the chunks of its share, which the
    // blocks of the tile write between them
    int k_lo = 0, k_hi = D;
    if constexpr (SPLIT) {
      const int nk_all = (D + BK - 1) / BK;
      const int share = (nk_all + (int)gridDim.y - 1) / (int)gridDim.y;
      k_lo = (int)blockIdx.y * share * BK;
      k_hi = k_lo + share * BK < D ? k_lo + share * BK : D;
    }
    if (k_lo < k_hi)
      rms_norm_block_rows<uint16_t>(x, norm_w, norm_eps, xn, t0, T - t0 < BT ? T - t0 : BT, D, k_lo, k_hi);
    __syncthreads();  // the block's part of xn is written and visible to all its waves
    x = xn;
  }

  f32x16 acc[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[f][i] = 0.f;
  // the bias of the experts this lane selects over, fetched now so that the selection does not
  // start with a memory round trip
  float b[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    b[j] = (bias != nullptr && e < E) ? bias[e] : 0.f;
  }

  // Global loads run two chunks ahead through two register sets.
  u32x4 rx[2][X_CHUNKS], rr[2][R_CHUNKS];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  const int nk = (D + BK - 1) / BK;                 // chunks in all
  // this block's chunks [kt_lo, kt_hi): all of them, or its share of them
  const int per_block = SPLIT ? (nk + (int)gridDim.y - 1) / (int)gridDim.y : nk;
  const int kt_lo = SPLIT ? (int)blockIdx.y * per_block : 0;
  const int kt_hi = kt_lo + per_block < nk ? kt_lo + per_block : nk;
  // per group; a group's step i is chunk kt_lo + GROUPS i + g
  const int steps = (per_block + GROUPS - 1) / GROUPS;
  // Every load is issued unconditionally from an address clamped into the arrays, and what lies
  // outside (chunks past this block's range, the tail of D, experts past E) is replaced by zeros
  // only when the registers are stored to LDS: with no branch around the loads and no use of their
  // results before that, the compiler can count them, and waiting for one register set leaves the
  // other in flight.
  auto load_global = [&](int set, int step) {
    const int kt = kt_lo + step * GROUPS + group;
    const int k0 = (kt < kt_hi ? kt : 0) * BK;
#pragma unroll
    for (int i = 0; i < X_CHUNKS; ++i) {
      const int c = tid + 256 * i;
      const int row = c / (BK / 8), kc = c % (BK / 8);
      int t = t0 + row;
      t = t < T ? t : T - 1;
      const int k = k0 + kc * 8;
      rx[set][i] = *reinterpret_cast<const u32x4*>(x + (size_t)t * D + (k < D ? k : D - 8));
    }
#pragma unroll
    for (int i = 0; i < R_CHUNKS; ++i) {
      const int c = tid + 256 * i;
      const int kr = c / (EP / 8), ec = c % (EP / 8);
      const int k = k0 + kr, e = ec * 8;
      rr[set][i] = *reinterpret_cast<const u32x4*>(router + (size_t)(k < D ? k : D - 1) * E +
                                                   (e < E ? e : E - 8));
    }
  };
  auto store_lds = [&](int set, int step) {
    const int kt = kt_lo + step * GROUPS + group;
    const bool live = kt < kt_hi;
    const int k0 = (live ? kt : 0) * BK;
#pragma unroll
    for (int i = 0; i < X_CHUNKS; ++i) {
      const int c = tid + 256 * i;
      const int row = c / (BK / 8), kc = c % (BK / 8);
      const bool in = live && k0 + kc * 8 < D;
      *reinterpret_cast<u32x4*>(&sX[row * LDX + kc * 8]) = in ? rx[set][i] : zero4;
    }
#pragma unroll
    for (int i = 0; i < R_CHUNKS; ++i) {
      const int c = tid + 256 * i;
      const int kr = c / (EP / 8), ec = c % (EP / 8);
      // E is a multiple of 8 on this path, so a chunk is entirely inside or outside.
      const bool in = live && k0 + kr < D && ec * 8 < E;
      *reinterpret_cast<u32x4*>(&sR[kr * LDR + ec * 8]) = in ? rr[set][i] : zero4;
    }
  };
  const int s = lane & 15, half = (lane >> 4) & 1;
  auto compute = [&]() {
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const bf16x8 xf = lds_read_frag(&sX[lr * LDX + ks * 16 + lk * 8]);
      const int kr = ks * 16 + lk * 8 + (s >> 2);
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        const int col = (wave + 4 * f) * 32 + half * 16 + (s & 3) * 4;
        const bf16x8 rf = lds_read_frag_tr(&sR[kr * LDR + col], &sR[(kr + 4) * LDR + col]);
        acc[f] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rf, xf, acc[f], 0, 0, 0);
      }
    }
  };

  // Both groups run the same number of steps (a group with one chunk fewer multiplies zeros in its
  // last step), so the barriers below are common to the block.
  load_global(0, 0);
  // keep set 0 the older one here as it is in the loop: a wait for it then leaves set 1 in flight
  __builtin_amdgcn_sched_barrier(0);
  load_global(1, 1);
  for (int st = 0; st < steps; st += 2) {
    store_lds(0, st);
    lds_barrier();
    load_global(0, st + 2);
    compute();
    lds_barrier();
    store_lds(1, st + 1);
    lds_barrier();
    load_global(1, st + 3);
    if (st + 1 < steps) compute();
    lds_barrier();
  }

  // Partial logits of each group -> its own LDS region (the stage is no longer needed).
  // Accumulator layout: lane holds token lr and experts 32 F + 8 q + 4 lk + j (F = wave + 4 f).
  float* sL = reinterpret_cast<float*>(smem + group * S::GROUP_BYTES);
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = (wave + 4 * f) * 32 + 8 * q + 4 * lk;
      f32x4 v = {acc[f][4 * q], acc[f][4 * q + 1], acc[f][4 * q + 2], acc[f][4 * q + 3]};
      *reinterpret_cast<f32x4*>(&sL[lr * LDL + e]) = v;
    }
  __syncthreads();

  if constexpr (SPLIT) {
    for (int i = tid_all; i < BT * EP; i += S::THREADS) {
      const int tl = i / EP, e = i - tl * EP;
      if (t0 + tl >= T || e >= E) continue;
      float sum = 0.f;
#pragma unroll
      for (int g2 = 0; g2 < GROUPS; ++g2)
        sum += reinterpret_cast<const float*>(smem + g2 * S::GROUP_BYTES)[tl * LDL + e];
      partial[((size_t)blockIdx.y * T + t0 + tl) * E + e] = sum;
    }
    return;
  }

  // every wave of the block selects for BT / (4 GROUPS) tokens
  constexpr int TPW = BT / (GROUPS * 4);
  const int wave_all = group * 4 + wave;
  for (int i = 0; i < TPW; ++i) {
    const int tl = wave_all * TPW + i;
    const int t = t0 + tl;
    if (t >= T) break;  // wave-uniform
    float v[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int e = lane + 64 * j;
      float sum = 0.f;
#pragma unroll
      for (int g2 = 0; g2 < GROUPS; ++g2)
        sum += reinterpret_cast<const float*>(smem + g2 * S::GROUP_BYTES)[tl * LDL + e];
      v[j] = sum + b[j];
      if (logits != nullptr && e < E) logits[(size_t)t * E + e] = v[j];
    }
    select_topk<J>(v, lane, t, E, K, score_fn, renorm, topk_idx, topk_w);
  }
}

// ------------------------------------------------------------------ bf16 / MFMA, (E, D) router matrix
// The same 32-token block with the router matrix given expert-major ((E, D): each expert's weights
// contiguous, e.g. a transposed copy the caller keeps).  Then both MFMA operands are k-contiguous:
// token rows and expert rows travel global -> LDS as 128-byte row pieces by direct loads
// (buffer_load ... lds: no staging registers, no LDS store instructions) and come back as plain
// 16-byte fragment reads, where the (D, E) form stores 20 KB per step to LDS and reads the matrix
// back through transposing reads at a quarter of the rate.  A tile is 64 of k: 32 token rows + EP
// expert rows; a step is TPS tiles, SLOTS steps in a ring, SLOTS - 1 of them in flight.  Wave w
// multiplies a tile's 16-k slice w / 4 into expert fragment w % 4 (+ 4, ..); the four slices' sums meet in
// LDS and are added in a fixed order, then every wave selects for two tokens, as above.
// Row r of a tile is 128 bytes; its 16-byte chunk c sits in slot c ^ ((r >> 1) & 7) (chosen by which
// chunk a lane fetches: the direct loads put lane l's 16 bytes at l * 16 of the piece), so the
// fragment reads of 32 rows are free of bank conflicts.
namespace rmfma_t {
constexpr int BT = 32, BK = 64;
template <int NF>
struct Shape {
  static constexpr int EP = 128 * NF;
  static constexpr int TILE_BYTES = (BT + EP) * BK * 2;  // token rows first, then expert rows
  // tiles per step, i.e. per barrier: two where the ring then still holds three steps (one tile per
  // step and seven in the ring: 18.3 us for 8192 tokens of 2048 features against 15.9 this way;
  // the transposing kernel above 19.7)
  static constexpr int TPS = NF == 1 ? 2 : 1;
  static constexpr int STEP_BYTES = TPS * TILE_BYTES;
  static constexpr int SLOTS = (148 * 1024) / STEP_BYTES;
  static constexpr int LDL = EP + 4;                     // logits row stride (floats)
  static constexpr int LOGIT_BYTES = 4 * BT * LDL * 4;   // the four slices' partial sums
  static constexpr int RING_BYTES = SLOTS * STEP_BYTES;
  static constexpr int SMEM_BYTES = RING_BYTES > LOGIT_BYTES ? RING_BYTES : LOGIT_BYTES;
};
}  // namespace rmfma_t

template <int NF>
__global__ __launch_bounds__(1024) void router_mfma_t_kernel(
    const uint16_t* x, const uint16_t* norm_w, float norm_eps, uint16_t* xn,
    const uint16_t* __restrict__ router_t, const float* __restrict__ bias, int T, int D, int E, int K,
    int score_fn, int renorm, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
    float* __restrict__ logits, uint8_t* __restrict__ tile_counts, int32_t* __restrict__ tile_rank) {
  using namespace rmfma_t;
  using S = Shape<NF>;
  constexpr int EP = S::EP, LDL = S::LDL, SLOTS = S::SLOTS, AHEAD = SLOTS - 1, J = EP / 64, TPS = S::TPS;
  static_assert(AHEAD >= 1 && (AHEAD - 1) * TPS * (NF + 1) < 64, "ring and wait counts");
  typedef __attribute__((address_space(3))) void* lds_ptr;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_t[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // 0 .. 15
  const int lr = lane & 31, lk = lane >> 5;
  const int t0 = blockIdx.x * BT;
  if (xn != nullptr) {
    rms_norm_block_rows<uint16_t>(x, norm_w, norm_eps, xn, t0, T - t0 < BT ? T - t0 : BT, D, 0, D);
    __syncthreads();  // the block's rows of xn are written and visible to all its waves
    x = xn;
  }
  float b[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    b[j] = (bias != nullptr && e < E) ? bias[e] : 0.f;
  }

  // ---- what this wave loads per step: expert pieces wave + 16 j (8 rows x 128 bytes each), and
  // waves 0..3 token piece `wave`.  Lane l fills row l / 8, slot l % 8 of its piece.
  const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(x + (size_t)t0 * D), 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t r_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(router_t), 0, -1, 0x00020000);
  const int prow = lane >> 3, pslot = lane & 7;
  // (off_r has a size that does not depend on NF on purpose: with a template-dependent argument the
  // host pass cannot check the call of the load builtin below, drops the kernel's instantiation
  // without a message, and the library ends up with an undefined kernel symbol)
  uint32_t off_r[2] = {0u, 0u}, off_x = 0;
  static_assert(NF <= 2, "off_r");
#pragma unroll
  for (int j = 0; j < NF; ++j) {
    const int row = 8 * (wave + 16 * j) + prow;  // expert
    const int kc = pslot ^ ((row >> 1) & 7);
    const int e = row < E ? row : E - 1;          // (logits of experts past E are never looked at)
    off_r[j] = (uint32_t)(((size_t)e * D + kc * 8) * 2);
  }
  const bool loads_x = wave < BT / 8;
  if (loads_x) {
    const int row = 8 * wave + prow;  // token of the tile
    const int kc = pslot ^ ((row >> 1) & 7);
    const int t = t0 + row < T ? row : T - 1 - t0;  // (rows past T are never looked at)
    off_x = (uint32_t)(((size_t)t * D + kc * 8) * 2);
  }
  const int steps = D / (BK * TPS);  // the host sends only D % (64 TPS) == 0 here
  auto issue = [&](int step) {
    uint8_t* slot = smem_t + (step % SLOTS) * S::STEP_BYTES;
#pragma unroll
    for (int tt = 0; tt < TPS; ++tt) {
      uint8_t* tile = slot + tt * S::TILE_BYTES;
      const uint32_t koff = (uint32_t)(step * TPS + tt) * (BK * 2);
      if (loads_x)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (lds_ptr)(tile + wave * 1024), 16, off_x, koff, 0, 0);
#pragma unroll
      for (int j = 0; j < NF; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(
            r_rsrc, (lds_ptr)(tile + BT * BK * 2 + (wave + 16 * j) * 1024), 16, off_r[j], koff, 0, 0);
    }
  };

  f32x16 acc[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[f][i] = 0.f;
  // fragment addresses within a tile: token row lr / expert row 32 F + lr, chunk 2 ks + lk (the key
  // is (lr >> 1) & 7 for all of them: 32 F does not change it)
  const int ks = wave >> 2, f0 = wave & 3;
  const uint32_t frag = (uint32_t)(lr * 128 + (((2 * ks + lk) ^ ((lr >> 1) & 7)) << 4));

  for (int st = 0; st < AHEAD && st < steps; ++st) issue(st);
  for (int st = 0; st < steps; ++st) {
    // this wave's loads of step st have landed once at most the loads of the AHEAD - 1 steps issued
    // after them are outstanding (vmcnt counts in issue order); towards the end fewer steps follow
    if (st + AHEAD - 1 < steps) {
      constexpr int R_ONLY = (AHEAD - 1) * TPS * NF, WITH_X = (AHEAD - 1) * TPS * (NF + 1);
      if (loads_x) __builtin_amdgcn_s_waitcnt(0x0f70 | (WITH_X & 15) | ((WITH_X >> 4) << 14));
      else __builtin_amdgcn_s_waitcnt(0x0f70 | (R_ONLY & 15) | ((R_ONLY >> 4) << 14));
    } else {
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    }
    lds_barrier();  // every wave's part of step st is in LDS; everybody is done with step st - 1
    if (st + AHEAD < steps) issue(st + AHEAD);  // into the slot of step st - 1
    const uint8_t* slot = smem_t + (st % SLOTS) * S::STEP_BYTES;
    bf16x8 xf[TPS], rf[TPS][NF];
#pragma unroll
    for (int tt = 0; tt < TPS; ++tt) {
      const uint8_t* tile = slot + tt * S::TILE_BYTES;
      xf[tt] = lds_read_frag(reinterpret_cast<const uint16_t*>(tile + frag));
#pragma unroll
      for (int f = 0; f < NF; ++f)
        rf[tt][f] = lds_read_frag(
            reinterpret_cast<const uint16_t*>(tile + BT * BK * 2 + (f0 + 4 * f) * 32 * 128 + frag));
    }
#pragma unroll
    for (int tt = 0; tt < TPS; ++tt)
#pragma unroll
      for (int f = 0; f < NF; ++f)
        acc[f] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(rf[tt][f], xf[tt], acc[f], 0, 0, 0);
  }
  __syncthreads();  // all fragment reads done: the ring becomes the partial sums' space

  // Partial logits of slice ks -> its LDS region.  Accumulator layout: lane holds token lr and
  // experts 32 F + 8 q + 4 lk + j (F = f0 + 4 f).
  float* sL = reinterpret_cast<float*>(smem_t) + ks * (BT * LDL);
#pragma unroll
  for (int f = 0; f < NF; ++f)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int e = (f0 + 4 * f) * 32 + 8 * q + 4 * lk;
      f32x4 v = {acc[f][4 * q], acc[f][4 * q + 1], acc[f][4 * q + 2], acc[f][4 * q + 3]};
      *reinterpret_cast<f32x4*>(&sL[lr * LDL + e]) = v;
    }
  // With tile_counts the block also does the counting pass of dispatch for its 32 tokens: a word
  // per expert, bit `token of the tile` set by the lane that holds the choice (an order-independent
  // OR), from which a pair's rank among the tile's pairs of its expert is a population count.
  static_assert(S::LOGIT_BYTES + EP * 4 <= S::SMEM_BYTES, "room for the tile's membership words");
  uint32_t* s_bits = reinterpret_cast<uint32_t*>(smem_t + S::LOGIT_BYTES);
  const bool counting = tile_counts != nullptr;  // block-uniform
  if (counting && tid < EP) s_bits[tid] = 0u;
  __syncthreads();

  constexpr int TPW = BT / 16;  // every wave selects for two tokens
  int chosen[TPW];
#pragma unroll
  for (int i = 0; i < TPW; ++i) {
    const int tl = wave * TPW + i;
    const int t = t0 + tl;
    chosen[i] = 0;
    if (t < T) {  // wave-uniform
      float v[J];
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const int e = lane + 64 * j;
        float sum = 0.f;
#pragma unroll
        for (int g2 = 0; g2 < 4; ++g2)
          sum += reinterpret_cast<const float*>(smem_t)[g2 * (BT * LDL) + tl * LDL + e];
        v[j] = sum + b[j];
        if (logits != nullptr && e < E) logits[(size_t)t * E + e] = v[j];
      }
      select_topk<J>(v, lane, t, E, K, score_fn, renorm, topk_idx, topk_w, &chosen[i]);
      if (counting && lane < K) atomicOr(&s_bits[chosen[i]], 1u << tl);
    }
  }
  if (!counting) return;
  __syncthreads();
#pragma unroll
  for (int i = 0; i < TPW; ++i) {
    const int tl = wave * TPW + i;
    const int t = t0 + tl;
    if (t < T && lane < K)
      tile_rank[(size_t)t * K + lane] = __popc(s_bits[chosen[i]] & ((1u << tl) - 1u));
  }
  if (tid < E) tile_counts[(size_t)blockIdx.x * E + tid] = (uint8_t)__popc(s_bits[tid]);
}

constexpr int kMaxSlices = 8;  // blocks sharing a token tile, at most

// Second half of the split router: one wave per token adds the `slices` partial logits in
// ascending order, then the bias, and selects.
template <int J>
__global__ __launch_bounds__(4 * kWave) void router_finish_kernel(
    const float* __restrict__ partial, int slices, const float* __restrict__ bias, int T, int E,
    int K, int score_fn, int renorm, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
    float* __restrict__ logits) {
  const int lane = lane_id();
  const int t = blockIdx.x * 4 + threadIdx.x / kWave;
  if (t >= T) return;  // wave-uniform
  // all loads first (at most kMaxSlices of them per expert), then the sums in ascending order
  float p[kMaxSlices][J], b[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    b[j] = (bias != nullptr && e < E) ? bias[e] : 0.f;
#pragma unroll
    for (int s = 0; s < kMaxSlices; ++s)
      p[s][j] = (s < slices && e < E) ? partial[((size_t)s * T + t) * E + e] : 0.f;
  }
  float v[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    float sum = p[0][j];
#pragma unroll
    for (int s = 1; s < kMaxSlices; ++s) sum += p[s][j];
    v[j] = sum + b[j];
    if (logits != nullptr && e < E) logits[(size_t)t * E + e] = v[j];
  }
  select_topk<J>(v, lane, t, E, K, score_fn, renorm, topk_idx, topk_w);
}

// The same for a few tokens in one block, which then goes on to dispatch them (dispatch_small_block:
// no rows copied): a decode step of a few sequences spends more on starting its kernels than on
// their work, and this is one start fewer.  A wave takes the tokens wave, wave + 16, ..  Same
// arithmetic as router_finish_kernel followed by dispatch_small_kernel, so the results are identical.
constexpr int kFinishDispatchThreads = 1024;
constexpr int kFinishDispatchTokens = 2 * kFinishDispatchThreads / kWave;
template <int J>
__global__ __launch_bounds__(kFinishDispatchThreads) void router_finish_dispatch_kernel(
    const float* __restrict__ partial, int slices, const float* __restrict__ bias, int T, int E,
    int K, int score_fn, int renorm, int32_t* topk_idx, float* topk_w, int tile_m, int64_t max_rows,
    int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* inv_perm, float* row_w) {
  extern __shared__ uint32_t s_mem[];
  __shared__ int32_t s_wave_tot[4];
  const int lane = lane_id();
  for (int t = threadIdx.x / kWave; t < T; t += kFinishDispatchThreads / kWave) {  // wave-uniform
    float p[kMaxSlices][J], b[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int e = lane + 64 * j;
      b[j] = (bias != nullptr && e < E) ? bias[e] : 0.f;
#pragma unroll
      for (int s = 0; s < kMaxSlices; ++s)
        p[s][j] = (s < slices && e < E) ? partial[((size_t)s * T + t) * E + e] : 0.f;
    }
    float v[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      float sum = p[0][j];
#pragma unroll
      for (int s = 1; s < kMaxSlices; ++s) sum += p[s][j];
      v[j] = sum + b[j];
    }
    select_topk<J>(v, lane, t, E, K, score_fn, renorm, topk_idx, topk_w);
  }
  __syncthreads();  // the tokens' experts are written and visible to the block
  // (the host sends K > 16 through router_finish_kernel and the dispatch kernels instead)
  dispatch_small_block<16>(topk_idx, T, K, E, tile_m, max_rows, counts, offsets, perm, inv_perm,
                           s_mem, s_wave_tot, threadIdx.x, kFinishDispatchThreads, true, topk_w, row_w);
}

// ------------------------------------------------------------------------------------ f32 / MFMA
// The same arrangement for f32 activations on v_mfma_f32_32x32x2_f32 (true f32 products and sums):
// a 32-token tile per block, 16 waves as 16 / FRP k-groups of FRP waves, wave f of a group owning
// the 32 experts of fragment f (E <= 32 FRP).  With few experts nearly all waves split the model
// dimension, which is what a small layer needs: its blocks are latency chains, not bandwidth.
// Operands are single floats: lane (i = l % 32, k = l / 32) reads router[k][32 f + i] and
// x[token i][k] from LDS; the x tile has an odd row stride so that the 32 rows of a column read
// fall into different banks.
namespace rmf32 {
constexpr int BT = 32;   // tokens per block
constexpr int BK = 32;   // model-dim chunk per stage
constexpr int LDX = BK + 1;
template <int FRP>
struct Shape {
  static constexpr int GROUPS = 16 / FRP;
  static constexpr int GT = 64 * FRP;       // threads per k-group
  static constexpr int EP = 32 * FRP;       // padded expert count
  static constexpr int LDL = EP + 1;        // partial-logit row stride (floats)
  static constexpr int STAGE_FLOATS = BT * LDX + BK * EP;
  static constexpr int LOGIT_FLOATS = BT * LDL;
  static constexpr int GROUP_FLOATS = STAGE_FLOATS > LOGIT_FLOATS ? STAGE_FLOATS : LOGIT_FLOATS;
  static constexpr int SMEM_BYTES = GROUPS * GROUP_FLOATS * 4;
};
}  // namespace rmf32

template <int FRP>
__global__ __launch_bounds__(1024) void router_mfma_f32_kernel(
    const float* x, const float* norm_w, float norm_eps, float* xn,
    const float* __restrict__ router, const float* __restrict__ bias, int T, int D, int E, int K,
    int score_fn, int renorm, int32_t* __restrict__ topk_idx, float* __restrict__ topk_w,
    float* __restrict__ logits) {
  using namespace rmf32;
  using S = Shape<FRP>;
  constexpr int GROUPS = S::GROUPS, GT = S::GT, EP = S::EP, LDL = S::LDL;
  constexpr int J = (EP + 63) / 64;
  constexpr int X_CHUNKS = BT * BK / 4 / GT;  // 16-byte chunks of the x tile per thread (4, 2, 1)
  constexpr int R_CHUNKS = BK * EP / 4 / GT;  // = 4
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

  const int tid_all = threadIdx.x;
  const int group = __builtin_amdgcn_readfirstlane(tid_all / GT);
  const int tid = tid_all % GT, lane = tid & 63;
  const int frag = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave within the group
  const int lr = lane & 31, lk = lane >> 5;
  const int t0 = blockIdx.x * BT;
  float* sX = reinterpret_cast<float*>(smem) + group * S::GROUP_FLOATS;
  float* sR = sX + BT * LDX;
  if (xn != nullptr) {
    rms_norm_block_rows<float>(x, norm_w, norm_eps, xn, t0, T - t0 < BT ? T - t0 : BT, D, 0, D);
    __syncthreads();  // the block's rows of xn are written and visible to all its waves
    x = xn;
  }

  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  float b[J];
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const int e = lane + 64 * j;
    b[j] = (bias != nullptr && e < E) ? bias[e] : 0.f;
  }

  // Global loads run two chunks ahead through two register sets (chunks past the end load zeros).
  f32x4 rx[2][X_CHUNKS], rr[2][R_CHUNKS];
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  const int nk = (D + BK - 1) / BK;
  const int steps = (nk + GROUPS - 1) / GROUPS;
  auto load_global = [&](int set, int step) {
    const int kt = step * GROUPS + group;
    const int k0 = (kt < nk ? kt : nk) * BK;
#pragma unroll
    for (int i = 0; i < X_CHUNKS; ++i) {
      const int c = tid + GT * i;
      const int row = c / (BK / 4), kc = c % (BK / 4);
      int t = t0 + row;
      t = t < T ? t : T - 1;
      const int k = k0 + kc * 4;
      // D is a multiple of 4 on this path, so a chunk is entirely inside or outside
      rx[set][i] = k < D ? *reinterpret_cast<const f32x4*>(x + (size_t)t * D + k) : zero4;
    }
#pragma unroll
    for (int i = 0; i < R_CHUNKS; ++i) {
      const int c = tid + GT * i;
      const int kr = c / (EP / 4), ec = c % (EP / 4);
      const int k = k0 + kr, e = ec * 4;
      rr[set][i] = (k < D && e < E) ? *reinterpret_cast<const f32x4*>(router + (size_t)k * E + e)
                                    : zero4;
    }
  };
  auto store_lds = [&](int set) {
#pragma unroll
    for (int i = 0; i < X_CHUNKS; ++i) {
      const int c = tid + GT * i;
      float* d = &sX[(c / (BK / 4)) * LDX + (c % (BK / 4)) * 4];
#pragma unroll
      for (int q = 0; q < 4; ++q) d[q] = rx[set][i][q];
    }
#pragma unroll
    for (int i = 0; i < R_CHUNKS; ++i) {
      const int c = tid + GT * i;
      *reinterpret_cast<f32x4*>(&sR[(c / (EP / 4)) * EP + (c % (EP / 4)) * 4]) = rr[set][i];
    }
  };
  auto compute = [&]() {
#pragma unroll
    for (int kk = 0; kk < BK / 2; ++kk) {
      const float rf = sR[(2 * kk + lk) * EP + frag * 32 + lr];
      const float xf = sX[lr * LDX + 2 * kk + lk];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(rf, xf, acc, 0, 0, 0);
    }
  };

  load_global(0, 0);
  load_global(1, 1);
  for (int st = 0; st < steps; st += 2) {
    store_lds(0);
    __syncthreads();
    load_global(0, st + 2);
    compute();
    __syncthreads();
    store_lds(1);
    __syncthreads();
    load_global(1, st + 3);
    if (st + 1 < steps) compute();
    __syncthreads();
  }

  // Partial logits of each group -> its own LDS region (the stage is no longer needed).
  // Accumulator layout: lane holds token lr and experts 32 frag + 8 q + 4 lk + j.
  float* sL = reinterpret_cast<float*>(smem) + group * S::GROUP_FLOATS;
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int j = 0; j < 4; ++j) sL[lr * LDL + frag * 32 + 8 * q + 4 * lk + j] = acc[4 * q + j];
  __syncthreads();

  // every wave of the block selects for two tokens; the groups' sums are added in a fixed order
  const int wave_all = tid_all >> 6;
  for (int i = 0; i < BT / 16; ++i) {
    const int tl = wave_all * (BT / 16) + i;
    const int t = t0 + tl;
    if (t >= T) break;  // wave-uniform
    float v[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
      const int e = lane + 64 * j;
      float sum = 0.f;
      if (e < EP) {
#pragma unroll
        for (int g2 = 0; g2 < GROUPS; ++g2)
          sum += reinterpret_cast<const float*>(smem)[g2 * S::GROUP_FLOATS + tl * LDL + e];
      }
      v[j] = sum + b[j];
      if (logits != nullptr && e < E) logits[(size_t)t * E + e] = v[j];
    }
    select_topk<J>(v, lane, t, E, K, score_fn, renorm, topk_idx, topk_w);
  }
}

template <int FRP>
static int launch_router_mfma_f32(const float* x, const float* norm_w, float norm_eps, float* xn,
                                  const float* router, const float* bias, int T, int D, int E,
                                  int K, int score_fn, int renorm, int32_t* topk_idx,
                                  float* topk_w, float* logits, hipStream_t stream) {
  using S = rmf32::Shape<FRP>;
  auto k = router_mfma_f32_kernel<FRP>;
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(k),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, S::SMEM_BYTES);
    if (e != hipSuccess) {
      set_error("router: cannot reserve LDS: %s", hipGetErrorString(e));
      return FS2MOE_ERR_LAUNCH;
    }
    attr_set = true;
  }
  hipLaunchKernelGGL(k, dim3((T + rmf32::BT - 1) / rmf32::BT), dim3(1024), S::SMEM_BYTES, stream, x,
                     norm_w, norm_eps, xn, router, bias, T, D, E, K, score_fn, renorm, topk_idx,
                     topk_w, logits);
  return check_launch("router_mfma_f32");
}

template <typename TA>
static int launch_router_fma(const void* x, const void* norm_w, float norm_eps, void* xn,
                             const void* router, const float* bias, int T, int D, int E, int K,
                             int score_fn, int renorm, int32_t* topk_idx, float* topk_w,
                             float* logits, hipStream_t stream) {
  const int tok_per_block = kRouterTok * kRouterWaves;
  dim3 grid((T + tok_per_block - 1) / tok_per_block), block(kRouterWaves * kWave);
  const TA* xp = static_cast<const TA*>(x);
  const TA* rp = static_cast<const TA*>(router);
  const TA* wp = static_cast<const TA*>(norm_w);
  TA* xnp = static_cast<TA*>(xn);
  const int j = (E + 63) / 64;
#define FS2_ROUTER_CASE(JJ)                                                                     \
  case JJ:                                                                                      \
    hipLaunchKernelGGL((router_fma_kernel<TA, JJ>), grid, block, 0, stream, xp, wp, norm_eps,  \
                       xnp, rp, bias, T, D, E, K, score_fn, renorm, topk_idx, topk_w, logits);  \
    break;
  switch (j) {
    FS2_ROUTER_CASE(1)
    FS2_ROUTER_CASE(2)
    FS2_ROUTER_CASE(3)
    FS2_ROUTER_CASE(4)
    FS2_ROUTER_CASE(5)
    FS2_ROUTER_CASE(6)
    FS2_ROUTER_CASE(7)
    FS2_ROUTER_CASE(8)
    default:
      set_error("router: E=%d exceeds %d", E, FS2MOE_MAX_EXPERTS);
      return FS2MOE_ERR_UNSUPPORTED;
  }
#undef FS2_ROUTER_CASE
  return check_launch("router_fma");
}

}  // namespace fs2moe

using namespace fs2moe;

// Token counts up to this are normalised by rms_norm_kernel in front of the router, larger ones by
// the router blocks themselves.  It covers every token count the split router takes.
constexpr int kNormAloneMaxTokens = 4096;

// How many blocks share a 32-token tile of the bf16 MFMA router: enough to put about 256 blocks on
// the chip, each with at least one step of its k-groups, at most 8.  1 = no split.
static int router_slices(int T, int D, int E, int act_dtype) {
  if (act_dtype != FS2MOE_BF16 || D % 8 != 0 || E % 8 != 0 || E > 256 || T < 1) return 1;
  const int tiles = (T + rmfma::BT - 1) / rmfma::BT;
  const int groups = E <= 128 ? rmfma::Shape<1>::GROUPS : rmfma::Shape<2>::GROUPS;
  const int nk = (D + 63) / 64;
  int s = 256 / tiles;
  s = s < nk / groups ? s : nk / groups;
  s = s < kMaxSlices ? s : kMaxSlices;
  return s >= 2 ? s : 1;
}

// Whether the router of this size reads an (E, D) matrix (FS2MOE_ROUTER_OUT_IN): the bf16 MFMA path
// with one block per token tile and whole steps of k.  Where several blocks would share a token tile
// (few tokens) the split kernels above are faster (64 tokens of 2048 features: 6.6 + 5.6 us against
// 16.9 us), and they read (D, E).
static bool router_takes_out_in(int T, int D, int E, int act_dtype) {
  return act_dtype == FS2MOE_BF16 && D % (rmfma_t::BK * 2) == 0 && E % 8 == 0 && E <= 256 && T > rmfma::BT &&
         (int64_t)E * D * 2 < (1ll << 31) && D <= (1 << 20) && router_slices(T, D, E, act_dtype) == 1;
}

extern "C" int64_t fs2moe_router_workspace_bytes(int32_t T, int32_t D, int32_t E,
                                                 int32_t act_dtype) {
  if (T < 0 || D < 1 || E < 1) return -1;
  const int s = router_slices(T, D, E, act_dtype);
  return s > 1 ? (int64_t)s * T * E * 4 : 0;
}

// xn null: route x as it is.  Otherwise normalise into xn first (norm_w may be null) and route xn.
static int router_entry(const void* x, const void* norm_w, float norm_eps, void* xn,
                        const void* router, const float* bias, int32_t T, int32_t D, int32_t E,
                        int32_t K, int32_t act_dtype, int32_t score_fn, int32_t renormalize,
                        int32_t* topk_idx, float* topk_w, float* logits, void* workspace,
                        int64_t workspace_bytes, DispatchAfterRouter* disp, void* stream) {
  FS2_REQUIRE(x && router && topk_idx && topk_w, "router: null pointer");
  FS2_REQUIRE(xn != x, "router: xn must not alias x");
  FS2_REQUIRE(workspace == nullptr || aligned16(workspace), "router: workspace is not 16-byte aligned");
  FS2_REQUIRE(T >= 0 && D > 0, "router: bad sizes T=%d D=%d", T, D);
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS, "router: E=%d outside [1, %d]", E,
              FS2MOE_MAX_EXPERTS);
  FS2_REQUIRE(K >= 1 && K <= E && K <= FS2MOE_MAX_TOP_K, "router: K=%d outside [1, min(E=%d, %d)]",
              K, E, FS2MOE_MAX_TOP_K);
  const bool out_in = (score_fn & FS2MOE_ROUTER_OUT_IN) != 0;
  score_fn &= ~FS2MOE_ROUTER_OUT_IN;
  FS2_REQUIRE(score_fn == FS2MOE_SCORE_SIGMOID || score_fn == FS2MOE_SCORE_SOFTMAX,
              "router: unknown score_fn %d", score_fn);
  FS2_REQUIRE(act_dtype == FS2MOE_F32 || act_dtype == FS2MOE_BF16, "router: act_dtype %d",
              act_dtype);
  FS2_REQUIRE(!out_in || (router_takes_out_in(T, D, E, act_dtype) && aligned16(x) && aligned16(router) &&
                          aligned16(xn)),
              "router: an (E, D) router matrix is read only where fs2moe_router_takes_out_in says so "
              "(T=%d D=%d E=%d), from 16-byte aligned operands", T, D, E);
  if (T == 0) return FS2MOE_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // (a single token tile of the bf16 MFMA router normalises in its own blocks, also when several
  // blocks share the tile: one launch fewer for a decode step)
  const bool one_tile = act_dtype == FS2MOE_BF16 && T <= rmfma::BT && D % 8 == 0 && E % 8 == 0 && E <= 256 &&
                        aligned16(x) && aligned16(router) && aligned16(xn);
  if (xn != nullptr && T <= kNormAloneMaxTokens && !one_tile) {
    // few token blocks: normalise with the whole chip first, then route xn as it is
    dim3 grid((T + kNormRows - 1) / kNormRows), block(kNormRows * kWave);
    if (act_dtype == FS2MOE_F32)
      hipLaunchKernelGGL(rms_norm_kernel<float>, grid, block, 0, s, static_cast<const float*>(x),
                         static_cast<const float*>(norm_w), norm_eps, static_cast<float*>(xn), T, D);
    else
      hipLaunchKernelGGL(rms_norm_kernel<uint16_t>, grid, block, 0, s,
                         static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(norm_w),
                         norm_eps, static_cast<uint16_t*>(xn), T, D);
    if (int rc = check_launch("rms_norm")) return rc;
    x = xn;
    xn = nullptr;
    norm_w = nullptr;
  }
  if (out_in) {
    auto k1 = router_mfma_t_kernel<1>;
    auto k2 = router_mfma_t_kernel<2>;
    static bool attr_set = false;  // benign race: setting the attribute is idempotent
    if (!attr_set) {
      hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(k1),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          rmfma_t::Shape<1>::SMEM_BYTES);
      hipError_t e2 = hipFuncSetAttribute(reinterpret_cast<const void*>(k2),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          rmfma_t::Shape<2>::SMEM_BYTES);
      if (e1 != hipSuccess || e2 != hipSuccess) {
        set_error("router: cannot reserve LDS: %s", hipGetErrorString(e1 != hipSuccess ? e1 : e2));
        return FS2MOE_ERR_LAUNCH;
      }
      attr_set = true;
    }
    const dim3 grid((T + rmfma_t::BT - 1) / rmfma_t::BT), threads(1024);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* wp = static_cast<const uint16_t*>(norm_w);
    uint16_t* xnp = static_cast<uint16_t*>(xn);
    // (the whole-layer call without a row copy: the tiles count their pairs themselves)
    static_assert(rmfma_t::BT == kRouterTileTok, "one routing block per counting tile");
    const bool counting = disp != nullptr && disp->ws != nullptr && (int)grid.x <= kIndexTilesMax &&
                          disp->ws_bytes >= fs2moe_dispatch_workspace_bytes(T, K, E);
    uint8_t* tile_counts = counting ? tile_counts_of(disp->ws) : nullptr;
    int32_t* tile_rank = counting ? tile_rank_of(disp->ws, T, E) : nullptr;
    if (E <= 128)
      hipLaunchKernelGGL(k1, grid, threads, rmfma_t::Shape<1>::SMEM_BYTES, s, xp, wp, norm_eps, xnp,
                         static_cast<const uint16_t*>(router), bias, T, D, E, K, score_fn, renormalize,
                         topk_idx, topk_w, logits, tile_counts, tile_rank);
    else
      hipLaunchKernelGGL(k2, grid, threads, rmfma_t::Shape<2>::SMEM_BYTES, s, xp, wp, norm_eps, xnp,
                         static_cast<const uint16_t*>(router), bias, T, D, E, K, score_fn, renormalize,
                         topk_idx, topk_w, logits, tile_counts, tile_rank);
    if (int rc = check_launch("router_mfma (E, D)")) return rc;
    if (counting) {
      if (int rc = dispatch_index_tiles(topk_idx, T, K, E, disp->tile_m, disp->max_rows, tile_counts,
                                        tile_rank, disp->counts, disp->offsets, disp->perm,
                                        disp->inv_perm, stream))
        return rc;
      disp->done = true;
    }
    return FS2MOE_OK;
  }
  if (act_dtype == FS2MOE_F32) {
    // The MFMA path moves 16-byte chunks (D and E multiples of 4, aligned bases) and holds up to
    // 128 experts; anything else takes the FMA kernel.
    if (D % 4 == 0 && E % 4 == 0 && E <= 128 && aligned16(x) && aligned16(router)) {
      const float* xp = static_cast<const float*>(x);
      const float* rp = static_cast<const float*>(router);
      const float* wp = static_cast<const float*>(norm_w);
      float* xnp = static_cast<float*>(xn);
      if (E <= 32)
        return launch_router_mfma_f32<1>(xp, wp, norm_eps, xnp, rp, bias, T, D, E, K, score_fn, renormalize, topk_idx,
                                         topk_w, logits, s);
      if (E <= 64)
        return launch_router_mfma_f32<2>(xp, wp, norm_eps, xnp, rp, bias, T, D, E, K, score_fn, renormalize, topk_idx,
                                         topk_w, logits, s);
      return launch_router_mfma_f32<4>(xp, wp, norm_eps, xnp, rp, bias, T, D, E, K, score_fn, renormalize, topk_idx,
                                       topk_w, logits, s);
    }
    return launch_router_fma<float>(x, norm_w, norm_eps, xn, router, bias, T, D, E, K, score_fn, renormalize, topk_idx,
                                    topk_w, logits, s);
  }
  // The MFMA path moves 16-byte chunks (D and E multiples of 8, aligned bases) and holds up to 256
  // experts; anything else takes the FMA kernel.
  if (D % 8 == 0 && E % 8 == 0 && E <= 256 && aligned16(x) && aligned16(router)) {
    dim3 grid((T + rmfma::BT - 1) / rmfma::BT);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    const uint16_t* rp = static_cast<const uint16_t*>(router);
    const uint16_t* wp = static_cast<const uint16_t*>(norm_w);
    uint16_t* xnp = static_cast<uint16_t*>(xn);
    auto k1 = router_mfma_kernel<1, false>;
    auto k2 = router_mfma_kernel<2, false>;
    auto k1s = router_mfma_kernel<1, true>;
    auto k2s = router_mfma_kernel<2, true>;
    static bool attr_set = false;  // benign race: setting the attribute is idempotent
    if (!attr_set) {
      const void* kernels[4] = {reinterpret_cast<const void*>(k1), reinterpret_cast<const void*>(k1s),
                                reinterpret_cast<const void*>(k2), reinterpret_cast<const void*>(k2s)};
      for (int i = 0; i < 4; ++i) {
        hipError_t e = hipFuncSetAttribute(
            kernels[i], hipFuncAttributeMaxDynamicSharedMemorySize,
            i < 2 ? rmfma::Shape<1>::SMEM_BYTES : rmfma::Shape<2>::SMEM_BYTES);
        if (e != hipSuccess) {
          set_error("router: cannot reserve LDS: %s", hipGetErrorString(e));
          return FS2MOE_ERR_LAUNCH;
        }
      }
      attr_set = true;
    }
    const int slices = router_slices(T, D, E, act_dtype);
    const dim3 threads(E <= 128 ? rmfma::Shape<1>::THREADS : rmfma::Shape<2>::THREADS);
    const int lds = E <= 128 ? rmfma::Shape<1>::SMEM_BYTES : rmfma::Shape<2>::SMEM_BYTES;
    if (slices > 1 && workspace != nullptr && workspace_bytes >= (int64_t)slices * T * E * 4) {
      // (several tiles were normalised by the kernel in front, T being within kNormAloneMaxTokens;
      // a single tile is normalised by its blocks, each the columns it reads)
      static_assert(256 * rmfma::BT / 2 <= kNormAloneMaxTokens, "split tiles are normalised in front");
      float* partial = static_cast<float*>(workspace);
      grid.y = slices;
      hipLaunchKernelGGL(E <= 128 ? k1s : k2s, grid, threads, lds, s, xp, wp, norm_eps, xnp, rp, bias,
                         T, D, E, K, score_fn, renormalize, topk_idx, topk_w, logits, partial);
      if (int rc = check_launch("router_mfma (split)")) return rc;
      const dim3 fgrid((T + 3) / 4), fblock(4 * kWave);
      const int j = (E + 63) / 64;
      if (disp != nullptr && logits == nullptr && T <= kFinishDispatchTokens && K <= 16) {
        const size_t dlds = dispatch_small_lds_words(E) * sizeof(uint32_t);
#define FS2_FINISH_CASE(JJ)                                                                       \
  case JJ:                                                                                        \
    hipLaunchKernelGGL((router_finish_dispatch_kernel<JJ>), dim3(1),                                \
                       dim3(kFinishDispatchThreads), dlds, s,                                     \
                       partial, slices, bias, T, E, K, score_fn, renormalize, topk_idx, topk_w,   \
                       disp->tile_m, disp->max_rows, disp->counts, disp->offsets, disp->perm,     \
                       disp->inv_perm, disp->row_w);                                              \
    break;
        switch (j) {
          FS2_FINISH_CASE(1)
          FS2_FINISH_CASE(2)
          FS2_FINISH_CASE(3)
          FS2_FINISH_CASE(4)
        }
#undef FS2_FINISH_CASE
        if (int rc = check_launch("router_finish_dispatch")) return rc;
        disp->done = true;
        return FS2MOE_OK;
      }
#define FS2_FINISH_CASE(JJ)                                                                      \
  case JJ:                                                                                       \
    hipLaunchKernelGGL((router_finish_kernel<JJ>), fgrid, fblock, 0, s, partial, slices, bias, T, \
                       E, K, score_fn, renormalize, topk_idx, topk_w, logits);                   \
    break;
      switch (j) {
        FS2_FINISH_CASE(1)
        FS2_FINISH_CASE(2)
        FS2_FINISH_CASE(3)
        FS2_FINISH_CASE(4)
      }
#undef FS2_FINISH_CASE
      return check_launch("router_finish");
    }
    hipLaunchKernelGGL(E <= 128 ? k1 : k2, grid, threads, lds, s, xp, wp, norm_eps, xnp, rp, bias, T,
                       D, E, K, score_fn, renormalize, topk_idx, topk_w, logits,
                       static_cast<float*>(nullptr));
    return check_launch("router_mfma");
  }
  return launch_router_fma<uint16_t>(x, norm_w, norm_eps, xn, router, bias, T, D, E, K, score_fn, renormalize, topk_idx,
                                     topk_w, logits, s);
}

extern "C" int32_t fs2moe_router_takes_out_in(int32_t T, int32_t D, int32_t E, int32_t act_dtype) {
  return router_takes_out_in(T, D, E, act_dtype) ? 1 : 0;
}

extern "C" int fs2moe_router_topk(const void* x, const void* router, const float* bias, int32_t T,
                                  int32_t D, int32_t E, int32_t K, int32_t act_dtype,
                                  int32_t score_fn, int32_t renormalize, int32_t* topk_idx,
                                  float* topk_w, float* logits, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
  return router_entry(x, nullptr, 0.f, nullptr, router, bias, T, D, E, K, act_dtype, score_fn,
                      renormalize, topk_idx, topk_w, logits, workspace, workspace_bytes, nullptr,
                      stream);
}

extern "C" int fs2moe_router_topk_norm(const void* x, const void* norm_weight, float norm_eps,
                                       void* xn, const void* router, const float* bias, int32_t T,
                                       int32_t D, int32_t E, int32_t K, int32_t act_dtype,
                                       int32_t score_fn, int32_t renormalize, int32_t* topk_idx,
                                       float* topk_w, float* logits, void* workspace,
                                       int64_t workspace_bytes, void* stream) {
  FS2_REQUIRE(xn != nullptr, "router: xn is null");
  FS2_REQUIRE(norm_eps >= 0.f, "router: norm_eps %g is negative", (double)norm_eps);
  return router_entry(x, norm_weight, norm_eps, xn, router, bias, T, D, E, K, act_dtype, score_fn,
                      renormalize, topk_idx, topk_w, logits, workspace, workspace_bytes, nullptr,
                      stream);
}

int fs2moe::router_then_dispatch(const void* x, const void* norm_w, float norm_eps, void* xn,
                                 const void* router, const float* bias, int32_t T, int32_t D,
                                 int32_t E, int32_t K, int32_t act_dtype, int32_t score_fn,
                                 int32_t renormalize, int32_t* topk_idx, float* topk_w,
                                 void* workspace, int64_t workspace_bytes,
                                 DispatchAfterRouter* disp, void* stream) {
  FS2_REQUIRE(xn == nullptr || norm_eps >= 0.f, "router: norm_eps %g is negative", (double)norm_eps);
  if (disp != nullptr) {
    FS2_REQUIRE(disp->tile_m >= 1 && disp->tile_m <= 1024, "dispatch: tile_m=%d", disp->tile_m);
    FS2_REQUIRE(disp->counts && disp->offsets && disp->perm && disp->inv_perm,
                "dispatch: null pointer");
    disp->done = false;
  }
  return router_entry(x, norm_w, norm_eps, xn, router, bias, T, D, E, K, act_dtype, score_fn,
                      renormalize, topk_idx, topk_w, nullptr, workspace, workspace_bytes, disp,
                      stream);
}

// ---- host mirror of the selection -------------------------------------------------------------------
// What select_topk does with a token's logits, on the host: same key, same rounds, same tie rule.
// Given the logits a device call returned, its indices are the device's bit for bit (also where two
// logits are closer than the accumulation error of any reference); the weights follow the same
// formulas in host float arithmetic and agree to rounding.
namespace {
inline uint32_t order_key_host(float v) {
  uint32_t b;
  memcpy(&b, &v, 4);
  if (v != v) return 0xffffffffu;
  if (v == 0.0f) b = 0;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
inline float order_key_inv_host(uint32_t k) {
  uint32_t b = k == 0xffffffffu ? 0x7fc00000u : (k & 0x80000000u) ? (k ^ 0x80000000u) : ~k;
  float v;
  memcpy(&v, &b, 4);
  return v;
}
}  // namespace

extern "C" int fs2moe_cpu_router_select(const float* logits, int32_t T, int32_t E, int32_t K,
                                        int32_t score_fn, int32_t renormalize, int32_t* topk_idx,
                                        float* topk_w) {
  FS2_REQUIRE(logits && topk_idx && topk_w, "cpu_router_select: null pointer");
  FS2_REQUIRE(T >= 0 && E >= 1 && E <= FS2MOE_MAX_EXPERTS && K >= 1 && K <= E &&
                  K <= FS2MOE_MAX_TOP_K,
              "cpu_router_select: bad sizes T=%d E=%d K=%d", T, E, K);
  FS2_REQUIRE(score_fn == FS2MOE_SCORE_SIGMOID || score_fn == FS2MOE_SCORE_SOFTMAX,
              "cpu_router_select: score_fn %d", score_fn);
  uint32_t key[FS2MOE_MAX_EXPERTS];
  float val[FS2MOE_MAX_TOP_K], w[FS2MOE_MAX_TOP_K];
  for (int t = 0; t < T; ++t) {
    const float* row = logits + (size_t)t * E;
    for (int e = 0; e < E; ++e) key[e] = order_key_host(row[e]);
    for (int r = 0; r < K; ++r) {
      int best = 0;
      for (int e = 1; e < E; ++e)
        if (key[e] > key[best]) best = e;  // strict: the lowest expert keeps a tie
      topk_idx[(size_t)t * K + r] = best;
      val[r] = order_key_inv_host(key[best]);
      key[best] = 0u;
    }
    if (score_fn == FS2MOE_SCORE_SIGMOID) {
      float s = 0.f;
      for (int r = 0; r < K; ++r) {
        w[r] = 1.0f / (1.0f + expf(-val[r]));
        s += w[r];
      }
      if (renormalize)
        for (int r = 0; r < K; ++r) w[r] /= s;
    } else {
      float s = 0.f;
      if (renormalize) {
        for (int r = 0; r < K; ++r) s += expf(val[r] - val[0]);
      } else {
        for (int e = 0; e < E; ++e) s += expf(row[e] - val[0]);
      }
      for (int r = 0; r < K; ++r) w[r] = expf(val[r] - val[0]) / s;
    }
    for (int r = 0; r < K; ++r) topk_w[(size_t)t * K + r] = w[r];
  }
  return FS2MOE_OK;
}

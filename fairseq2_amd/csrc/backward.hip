// Backward pass of the MoE feed-forward layer: the kernels that the forward pass has no use for.
//
// The gradient of out = sum_k w_k * expert_k(x) [+ shared(x)] reuses the forward machinery wherever the
// operation is the same with other operands (a grouped GEMM against the transposed weights is the
// grouped GEMM in the other weight orientation; the gather of output gradients into expert order is
// dispatch; the scatter of input gradients back to token order is combine).  What is new:
//   * grouped_wgrad_kernel   dW_e = A_e^T B_e, a GEMM whose contraction runs over the expert's rows
//   * swiglu_backward_kernel element-wise derivative of SiLU(g) * u, also restoring h
//   * pair_dot_kernel        the gradient of a combine weight: a dot product of two rows per pair
//   * router_backward_kernel combine-weight gradients -> logit gradients (sigmoid / softmax, with
//                            or without renormalisation over the selected experts)
// They are what torch.autograd derives from moe.py:102-157, experts.py:102-112 and ffn.py:374-395.
#include "common.h"
#include "tile_map.h"

namespace fs2moe {

// ---------------------------------------------------------------------------------- weight gradient
// C_e [M, N] = sum over the rows r of expert e of A[r, :M]^T B[r, :N].  A block owns a 128 x 128 tile
// of one expert's gradient and walks the expert's rows 32 at a time: both chunks go to LDS as they
// lie in memory (row = contraction index, columns contiguous) and come back through the transposing
// LDS read (bf16) or as single floats (f32), each already in MFMA operand order.  Rows past the
// expert's count are zero-filled, experts without rows get a zero gradient.
namespace wgk {
constexpr int TM = 128, TN = 128, RK = 32;
}

template <typename T>
__global__ __launch_bounds__(256) void grouped_wgrad_kernel(
    const T* __restrict__ A, const int32_t* __restrict__ a_map, int lda, const T* __restrict__ B,
    int ldb, T* __restrict__ C, int M, int N, Groups g, int m_tiles, int n_tiles) {
  using namespace wgk;
  constexpr bool BF16 = sizeof(T) == 2;
  constexpr int VEC = 16 / sizeof(T);             // elements per 16-byte chunk
  constexpr int ROW_CHUNKS = TM / VEC;            // chunks per LDS row (16 or 32)
  constexpr int PER_THREAD = RK * ROW_CHUNKS / 256;  // chunks per thread and operand (2 or 4)
  constexpr int ROWB = TM * sizeof(T);            // bytes per LDS row
  __shared__ __attribute__((aligned(16))) uint8_t sA[RK * ROWB];
  __shared__ __attribute__((aligned(16))) uint8_t sB[RK * ROWB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int per_e = m_tiles * n_tiles;
  const int e = blockIdx.x / per_e;
  const int rem = blockIdx.x - e * per_e;
  const int mt = rem / n_tiles, nt = rem - mt * n_tiles;
  const int m0 = mt * TM, n0 = nt * TN;
  const bool dense = g.counts == nullptr;
  const int off = dense ? 0 : g.offsets[e];
  const int cnt = dense ? g.dense_rows : g.counts[e];
  const int wm = wave & 1, wn = wave >> 1;  // the wave's 64 x 64 quarter of the tile
  const int lr = lane & 31, lk = lane >> 5;

  f32x16 acc[2][2];  // [tn][tm]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  u32x4 ra[PER_THREAD], rb[PER_THREAD];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  auto load_chunk = [&](int r0) {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = tid + 256 * i;
      const int k = c / ROW_CHUNKS, ch = c % ROW_CHUNKS;
      const int r = r0 + k;
      ra[i] = zero4;
      rb[i] = zero4;
      if (r < cnt) {
        const int arow = a_map != nullptr ? a_map[off + r] : off + r;
        if (m0 + ch * VEC < M)
          ra[i] = *reinterpret_cast<const u32x4*>(A + (size_t)arow * lda + m0 + ch * VEC);
        if (n0 + ch * VEC < N)
          rb[i] = *reinterpret_cast<const u32x4*>(B + (size_t)(off + r) * ldb + n0 + ch * VEC);
      }
    }
  };
  auto store_chunk = [&]() {
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = tid + 256 * i;
      const int k = c / ROW_CHUNKS, ch = c % ROW_CHUNKS;
      // bf16: chunk ch of row k sits in slot ch ^ ((k & 3) << 2), so that the four consecutive rows
      // a transposing read touches lie 64 bytes apart
      const int slot = BF16 ? (ch ^ ((k & 3) << 2)) : ch;
      *reinterpret_cast<u32x4*>(sA + k * ROWB + slot * 16) = ra[i];
      *reinterpret_cast<u32x4*>(sB + k * ROWB + slot * 16) = rb[i];
    }
  };

  // bf16 fragment address of the 32 columns from cbase on, rows 8 lk .. 8 lk + 3 (+4 for the upper half)
  auto tr_addr = [&](int cbase) {
    const int s = lane & 15, half = (lane >> 4) & 1;
    const int k = lk * 8 + (s >> 2);
    const int col = cbase + half * 16 + (s & 3) * 4;
    return k * ROWB + (((col >> 3) ^ ((k & 3) << 2)) * 16) + (col & 7) * 2;
  };
  int fa[2], fb[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    fa[t] = BF16 ? tr_addr(wm * 64 + t * 32) : (wm * 64 + t * 32 + lr) * 4;
    fb[t] = BF16 ? tr_addr(wn * 64 + t * 32) : (wn * 64 + t * 32 + lr) * 4;
  }

  if (cnt > 0) load_chunk(0);
  for (int r0 = 0; r0 < cnt; r0 += RK) {
    __syncthreads();  // the last chunk has been read
    store_chunk();
    __syncthreads();
    if (r0 + RK < cnt) load_chunk(r0 + RK);
    if constexpr (BF16) {
#pragma unroll
      for (int ks = 0; ks < RK / 16; ++ks) {
        bf16x8 af[2], bfr[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const uint8_t* pa = sA + fa[t] + ks * 16 * ROWB;
          const uint8_t* pb = sB + fb[t] + ks * 16 * ROWB;
          af[t] = lds_read_frag_tr(reinterpret_cast<const uint16_t*>(pa),
                                   reinterpret_cast<const uint16_t*>(pa + 4 * ROWB));
          bfr[t] = lds_read_frag_tr(reinterpret_cast<const uint16_t*>(pb),
                                    reinterpret_cast<const uint16_t*>(pb + 4 * ROWB));
        }
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
          for (int tm = 0; tm < 2; ++tm)
            acc[tn][tm] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
      }
    } else {
#pragma unroll 4
      for (int ks = 0; ks < RK / 2; ++ks) {
        float af[2], bfr[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          af[t] = *reinterpret_cast<const float*>(sA + (2 * ks + lk) * ROWB + fa[t]);
          bfr[t] = *reinterpret_cast<const float*>(sB + (2 * ks + lk) * ROWB + fb[t]);
        }
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
          for (int tm = 0; tm < 2; ++tm)
            acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x2f32(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
      }
    }
  }

  // Accumulator layout: the lane holds row m = lr of fragment tm and columns 8 q + 4 lk + {0..3} of
  // fragment tn in registers 4 q .. 4 q + 3.
  T* Ce = C + (size_t)e * M * N;
#pragma unroll
  for (int tm = 0; tm < 2; ++tm) {
    const int m = m0 + wm * 64 + tm * 32 + lr;
    if (m >= M) continue;
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 64 + tn * 32 + 8 * q + 4 * lk;
        if (n >= N) continue;  // N is a multiple of 4: the four columns are in or out together
        const float v0 = acc[tn][tm][4 * q], v1 = acc[tn][tm][4 * q + 1];
        const float v2 = acc[tn][tm][4 * q + 2], v3 = acc[tn][tm][4 * q + 3];
        if constexpr (BF16) {
          u32x2 o = {pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
          *reinterpret_cast<u32x2*>(Ce + (size_t)m * N + n) = o;
        } else {
          f32x4 o = {v0, v1, v2, v3};
          *reinterpret_cast<f32x4*>(Ce + (size_t)m * N + n) = o;
        }
      }
    }
  }
}

// ------------------------------------------------------------------------- SwiGLU, element-wise
// h = SiLU(g) * u;  dg = dh * u * s * (1 + g * (1 - s)),  du = dh * SiLU(g),  s = sigmoid(g).
// In f32 with one rounding per output; outputs may alias the inputs element for element.
template <typename T>
__global__ __launch_bounds__(256) void swiglu_backward_kernel(const T* g, const T* u, const T* dh,
                                                              int64_t n, T* h, T* dg, T* du) {
  constexpr int VEC = 16 / sizeof(T);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x * VEC;
  for (int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * VEC; i < n; i += stride) {
    const u32x4 gv = *reinterpret_cast<const u32x4*>(g + i);
    const u32x4 uv = *reinterpret_cast<const u32x4*>(u + i);
    const u32x4 dv = *reinterpret_cast<const u32x4*>(dh + i);
    float gf[VEC], uf[VEC], df[VEC], ho[VEC], go[VEC], uo[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      if constexpr (sizeof(T) == 2) {
        const uint32_t gw = gv[j >> 1], uw = uv[j >> 1], dw = dv[j >> 1];
        gf[j] = __uint_as_float((j & 1) ? (gw & 0xffff0000u) : (gw << 16));
        uf[j] = __uint_as_float((j & 1) ? (uw & 0xffff0000u) : (uw << 16));
        df[j] = __uint_as_float((j & 1) ? (dw & 0xffff0000u) : (dw << 16));
      } else {
        gf[j] = __uint_as_float(gv[j]);
        uf[j] = __uint_as_float(uv[j]);
        df[j] = __uint_as_float(dv[j]);
      }
      const float s = 1.0f / (1.0f + __expf(-gf[j]));
      const float silu = gf[j] * s;
      ho[j] = silu * uf[j];
      go[j] = df[j] * uf[j] * (s * (1.0f + gf[j] * (1.0f - s)));
      uo[j] = df[j] * silu;
    }
    u32x4 hv, gov, uov;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (sizeof(T) == 2) {
        hv[j] = pack_bf16x2(ho[2 * j], ho[2 * j + 1]);
        gov[j] = pack_bf16x2(go[2 * j], go[2 * j + 1]);
        uov[j] = pack_bf16x2(uo[2 * j], uo[2 * j + 1]);
      } else {
        hv[j] = __float_as_uint(ho[j]);
        gov[j] = __float_as_uint(go[j]);
        uov[j] = __float_as_uint(uo[j]);
      }
    }
    *reinterpret_cast<u32x4*>(h + i) = hv;
    *reinterpret_cast<u32x4*>(dg + i) = gov;
    *reinterpret_cast<u32x4*>(du + i) = uov;
  }
}

// ------------------------------------------------------------------- gradient of a combine weight
// out[p] = <a[a_rows[p]], b[p / K]> (+ <a2[a_rows[p]], b[p / K]>) for the T*K pairs p: one wave per
// pair, f32 accumulation in a fixed order.
template <typename T>
__global__ __launch_bounds__(256) void pair_dot_kernel(const T* __restrict__ a,
                                                       const T* __restrict__ a2,
                                                       const int32_t* __restrict__ a_rows,
                                                       const T* __restrict__ b, int pairs, int K,
                                                       int D, float* __restrict__ out) {
  const int p = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int lane = threadIdx.x & 63;
  const size_t ar = (size_t)a_rows[p] * D, br = (size_t)(p / K) * D;
  float s = 0.f;
  for (int d = lane; d < D; d += 64) {
    float av = Elem<T>::load(a + ar + d);
    if (a2 != nullptr) av += Elem<T>::load(a2 + ar + d);
    s += av * Elem<T>::load(b + br + d);
  }
  s = wave_sum_f32(s);
  if (lane == 0) out[p] = s;
}

// --------------------------------------------------------------------------------- router backward
// One wave per token: dw [K] -> dlogits [E] (zero where the score function does not reach).
//   sigmoid:              w_k = s_k,            s = sigmoid(l_k)    dl_k = dw_k s_k (1 - s_k)
//   sigmoid, renormalised w_k = s_k / S,        S = sum_sel s       dl_k = (dw_k - <dw, w>) / S * s_k (1 - s_k)
//   softmax:              w_k = p_k,            p = softmax(l)      dl_e = p_e ([e selected] dw_e - <dw, w>)
//   softmax, renormalised w_k = p_k / sum_sel p                     dl_k = w_k (dw_k - <dw, w>)
template <typename T>
__global__ __launch_bounds__(256) void router_backward_kernel(
    const float* __restrict__ logits, const int32_t* __restrict__ topk_idx,
    const float* __restrict__ topk_w, const float* __restrict__ d_w, int Tn, int E, int K,
    int score_fn, int renormalize, T* __restrict__ dlogits) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= Tn) return;
  const int lane = threadIdx.x & 63;
  const float* l = logits + (size_t)t * E;
  // <dw, w> over the selected experts
  float dot = 0.f;
  for (int k = 0; k < K; ++k) dot += d_w[(size_t)t * K + k] * topk_w[(size_t)t * K + k];
  float mx = -INFINITY, den = 0.f, ssum = 0.f;
  if (score_fn == FS2MOE_SCORE_SOFTMAX && !renormalize) {
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, l[e]);
    // wave-wide maximum through the order-preserving unsigned key of a float
    {
      const uint32_t u = __float_as_uint(mx);
      const uint32_t key = wave_max_u32((u & 0x80000000u) ? ~u : (u | 0x80000000u));
      mx = __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
    }
    for (int e = lane; e < E; e += 64) den += __expf(l[e] - mx);
    den = wave_sum_f32(den);
  }
  if (score_fn == FS2MOE_SCORE_SIGMOID && renormalize) {
    for (int k = 0; k < K; ++k) {
      const float lk = l[topk_idx[(size_t)t * K + k]];
      ssum += 1.0f / (1.0f + __expf(-lk));
    }
  }
  for (int e = lane; e < E; e += 64) {
    float dw = 0.f, w = 0.f;
    bool sel = false;
    for (int k = 0; k < K; ++k)
      if (topk_idx[(size_t)t * K + k] == e) {
        dw = d_w[(size_t)t * K + k];
        w = topk_w[(size_t)t * K + k];
        sel = true;
      }
    float dl = 0.f;
    if (score_fn == FS2MOE_SCORE_SIGMOID) {
      if (sel) {
        const float s = 1.0f / (1.0f + __expf(-l[e]));
        dl = renormalize ? (dw - dot) / ssum * s * (1.0f - s) : dw * s * (1.0f - s);
      }
    } else if (renormalize) {
      if (sel) dl = w * (dw - dot);
    } else {
      const float p = __expf(l[e] - mx) / den;
      dl = p * ((sel ? dw : 0.f) - dot);
    }
    Elem<T>::store(dlogits + (size_t)t * E + e, dl);
  }
}

}  // namespace fs2moe

using namespace fs2moe;

extern "C" int fs2moe_grouped_wgrad(const void* a, const int32_t* a_row_map, const void* b,
                                    const int32_t* counts, const int32_t* offsets, int32_t E,
                                    int32_t M, int32_t N, int64_t max_rows, int32_t dtype, void* dw,
                                    void* stream) {
  FS2_REQUIRE(a && b && dw, "grouped_wgrad: null pointer");
  FS2_REQUIRE((counts == nullptr) == (offsets == nullptr), "grouped_wgrad: counts without offsets");
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS && (counts != nullptr || E == 1),
              "grouped_wgrad: E=%d", E);
  FS2_REQUIRE(dtype == FS2MOE_F32 || dtype == FS2MOE_BF16, "grouped_wgrad: dtype %d", dtype);
  const int vec = dtype == FS2MOE_BF16 ? 8 : 4;
  FS2_REQUIRE(M > 0 && N > 0 && M % vec == 0 && N % vec == 0,
              "grouped_wgrad: M=%d and N=%d must be positive multiples of %d", M, N, vec);
  FS2_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), "grouped_wgrad: max_rows=%lld",
              (long long)max_rows);
  FS2_REQUIRE(aligned16(a) && aligned16(b) && aligned16(dw),
              "grouped_wgrad: buffers must be 16-byte aligned");
  const int m_tiles = (M + wgk::TM - 1) / wgk::TM, n_tiles = (N + wgk::TN - 1) / wgk::TN;
  const int64_t blocks = (int64_t)E * m_tiles * n_tiles;
  FS2_REQUIRE(blocks <= 0x7fffffffll, "grouped_wgrad: too many tiles");
  Groups g{counts, offsets, E, (int)max_rows};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == FS2MOE_BF16)
    hipLaunchKernelGGL(grouped_wgrad_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const uint16_t*>(a), a_row_map, M,
                       static_cast<const uint16_t*>(b), N, static_cast<uint16_t*>(dw), M, N, g,
                       m_tiles, n_tiles);
  else
    hipLaunchKernelGGL(grouped_wgrad_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const float*>(a), a_row_map, M, static_cast<const float*>(b), N,
                       static_cast<float*>(dw), M, N, g, m_tiles, n_tiles);
  return check_launch("grouped_wgrad");
}

extern "C" int fs2moe_swiglu_backward(const void* g, const void* u, const void* dh, int64_t rows,
                                      int32_t F, int32_t dtype, void* h, void* dg, void* du,
                                      void* stream) {
  FS2_REQUIRE(g && u && dh && h && dg && du, "swiglu_backward: null pointer");
  FS2_REQUIRE(dtype == FS2MOE_F32 || dtype == FS2MOE_BF16, "swiglu_backward: dtype %d", dtype);
  FS2_REQUIRE(rows >= 0 && F > 0 && F % 8 == 0, "swiglu_backward: rows=%lld, F=%d",
              (long long)rows, F);
  FS2_REQUIRE(aligned16(g) && aligned16(u) && aligned16(dh) && aligned16(h) && aligned16(dg) &&
                  aligned16(du),
              "swiglu_backward: buffers must be 16-byte aligned");
  const int64_t n = rows * F;
  if (n == 0) return FS2MOE_OK;
  const int vec = dtype == FS2MOE_BF16 ? 8 : 4;
  int64_t blocks = (n / vec + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == FS2MOE_BF16)
    hipLaunchKernelGGL(swiglu_backward_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const uint16_t*>(g), static_cast<const uint16_t*>(u),
                       static_cast<const uint16_t*>(dh), n, static_cast<uint16_t*>(h),
                       static_cast<uint16_t*>(dg), static_cast<uint16_t*>(du));
  else
    hipLaunchKernelGGL(swiglu_backward_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const float*>(g), static_cast<const float*>(u),
                       static_cast<const float*>(dh), n, static_cast<float*>(h),
                       static_cast<float*>(dg), static_cast<float*>(du));
  return check_launch("swiglu_backward");
}

extern "C" int fs2moe_pair_dot(const void* a, const void* a2, const int32_t* a_rows, const void* b,
                               int32_t T, int32_t K, int32_t D, int32_t dtype, float* out,
                               void* stream) {
  FS2_REQUIRE(a && a_rows && b && out, "pair_dot: null pointer");
  FS2_REQUIRE(dtype == FS2MOE_F32 || dtype == FS2MOE_BF16, "pair_dot: dtype %d", dtype);
  FS2_REQUIRE(T >= 0 && K >= 1 && K <= FS2MOE_MAX_TOP_K && D > 0, "pair_dot: T=%d, K=%d, D=%d", T, K,
              D);
  const int64_t pairs = (int64_t)T * K;
  FS2_REQUIRE(pairs < (1ll << 31), "pair_dot: too many pairs");
  if (pairs == 0) return FS2MOE_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned blocks = (unsigned)((pairs + 3) / 4);
  if (dtype == FS2MOE_BF16)
    hipLaunchKernelGGL(pair_dot_kernel<uint16_t>, dim3(blocks), dim3(256), 0, st,
                       static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(a2), a_rows,
                       static_cast<const uint16_t*>(b), (int)pairs, K, D, out);
  else
    hipLaunchKernelGGL(pair_dot_kernel<float>, dim3(blocks), dim3(256), 0, st,
                       static_cast<const float*>(a), static_cast<const float*>(a2), a_rows,
                       static_cast<const float*>(b), (int)pairs, K, D, out);
  return check_launch("pair_dot");
}

extern "C" int fs2moe_router_backward(const float* logits, const int32_t* topk_idx,
                                      const float* topk_w, const float* d_w, int32_t T, int32_t E,
                                      int32_t K, int32_t score_fn, int32_t renormalize,
                                      int32_t dtype, void* dlogits, void* stream) {
  FS2_REQUIRE(logits && topk_idx && topk_w && d_w && dlogits, "router_backward: null pointer");
  FS2_REQUIRE(dtype == FS2MOE_F32 || dtype == FS2MOE_BF16, "router_backward: dtype %d", dtype);
  FS2_REQUIRE(T >= 0 && E >= 1 && E <= FS2MOE_MAX_EXPERTS && K >= 1 && K <= FS2MOE_MAX_TOP_K &&
                  K <= E,
              "router_backward: T=%d, E=%d, K=%d", T, E, K);
  FS2_REQUIRE(score_fn == FS2MOE_SCORE_SIGMOID || score_fn == FS2MOE_SCORE_SOFTMAX,
              "router_backward: score_fn %d", score_fn);
  if (T == 0) return FS2MOE_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const unsigned blocks = (unsigned)((T + 3) / 4);
  if (dtype == FS2MOE_BF16)
    hipLaunchKernelGGL(router_backward_kernel<uint16_t>, dim3(blocks), dim3(256), 0, st, logits,
                       topk_idx, topk_w, d_w, T, E, K, score_fn, renormalize,
                       static_cast<uint16_t*>(dlogits));
  else
    hipLaunchKernelGGL(router_backward_kernel<float>, dim3(blocks), dim3(256), 0, st, logits,
                       topk_idx, topk_w, d_w, T, E, K, score_fn, renormalize,
                       static_cast<float*>(dlogits));
  return check_launch("router_backward");
}

// Weighted combine back to token order.
//
// A gather, not a scatter: the wave that owns token t reads its K expert rows through the inverse
// permutation and adds them in ascending expert id onto the base row (the shared expert's output
// or zero), in f32, then rounds once.  This is the order in which the reference's scatter_add_
// accumulates, reproduced without float atomics, so the result is deterministic.  An optional
// residual row (the layer input of a pre-norm decoder layer) joins the base before the expert rows,
// which saves the caller's separate addition pass over (T, D).
#include "common.h"

namespace fs2moe {

constexpr int kCombWaves = 4;

template <typename TA>
struct Chunk;  // 16 bytes of activations <-> f32 lanes
template <>
struct Chunk<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(u32x4 v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = __float_as_uint(f[i]);
    return o;
  }
};
template <>
struct Chunk<uint16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4 v, float* f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(v[i] << 16);
      f[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ u32x4 pack(const float* f) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
    return o;
  }
};

// KMAX: compile-time bound on K (slots beyond K carry row -1).  WPT: waves per token; the token's
// 16-byte chunks are dealt round-robin to its waves (WPT = 4 when there are too few tokens to fill
// the GPU with one wave each).
template <typename TA, int KMAX, int WPT>
__global__ __launch_bounds__(kCombWaves* kWave) void combine_kernel(
    const TA* __restrict__ ye, const int32_t* __restrict__ inv_perm,
    const int32_t* __restrict__ topk_idx, const float* __restrict__ topk_w, const TA* base,
    const TA* residual, int T, int K, int D, int weight_output, TA* out) {
  const int lane = lane_id();
  const int gw = blockIdx.x * kCombWaves + threadIdx.x / kWave;
  const int t = gw / WPT, part = gw % WPT;
  if (t >= T) return;

  // Order the token's slots by ascending expert id (slot index breaks ties).
  int e = 0x7fffffff, row = -1;
  float w = 0.f;
  if (lane < K) {
    e = topk_idx[(size_t)t * K + lane];
    row = inv_perm[(size_t)t * K + lane];
    w = weight_output ? topk_w[(size_t)t * K + lane] : 1.0f;
  }
  int pos = 0;
  for (int i = 0; i < K; ++i) {
    int ei = __shfl(e, i, kWave);
    pos += (ei < e || (ei == e && i < lane)) ? 1 : 0;
  }
  // Invert: lane s takes the slot whose position is s, so lanes 0..K-1 hold the sorted list.
  int src = 0;
  for (int i = 0; i < K; ++i) {
    int pi = __shfl(pos, i, kWave);
    if (pi == lane) src = i;
  }
  // lanes K .. KMAX-1 found no slot (src = 0): they must contribute nothing
  const int picked_row = __shfl(row, src, kWave);
  const int sorted_row = lane < K ? picked_row : -1;
  const float sorted_w = __shfl(w, src, kWave);
  // Wave-uniform copies of the sorted list (lanes >= K contributed row -1).
  int rj[KMAX];
  float wj[KMAX];
#pragma unroll
  for (int j = 0; j < KMAX; ++j) {
    rj[j] = __builtin_amdgcn_readlane(sorted_row, j);
    wj[j] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(sorted_w), j));
  }

  constexpr int N = Chunk<TA>::N;
  const int chunks = D / N;
  const u32x4* ye4 = reinterpret_cast<const u32x4*>(ye);
  const u32x4* base4 = reinterpret_cast<const u32x4*>(base);
  const u32x4* res4 = reinterpret_cast<const u32x4*>(residual);
  u32x4* out4 = reinterpret_cast<u32x4*>(out);
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  for (int c = lane + kWave * part; c < chunks; c += kWave * WPT) {
    // all of the chunk's loads are issued before the first add
    u32x4 v[KMAX];
#pragma unroll
    for (int j = 0; j < KMAX; ++j)
      v[j] = rj[j] >= 0 ? ye4[(size_t)rj[j] * chunks + c] : zero4;
    float acc[N];
    if (base != nullptr) {
      Chunk<TA>::unpack(base4[(size_t)t * chunks + c], acc);
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) acc[i] = 0.f;
    }
    if (residual != nullptr) {  // wave-uniform
      float r[N];
      Chunk<TA>::unpack(res4[(size_t)t * chunks + c], r);
#pragma unroll
      for (int i = 0; i < N; ++i) acc[i] += r[i];
    }
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
      if (rj[j] >= 0) {  // wave-uniform
        float y[N];
        Chunk<TA>::unpack(v[j], y);
#pragma unroll
        for (int i = 0; i < N; ++i) acc[i] += wj[j] * y[i];
      }
    }
    out4[(size_t)t * chunks + c] = Chunk<TA>::pack(acc);
  }
}

template <typename TA>
static int launch_combine(const void* ye, const int32_t* inv_perm, const int32_t* topk_idx,
                          const float* topk_w, const void* base, const void* residual, int T, int K,
                          int D, int weight_output, void* out, hipStream_t s) {
  const int wpt = T < 2048 ? 4 : 1;
  dim3 grid(((size_t)T * wpt + kCombWaves - 1) / kCombWaves), block(kCombWaves * kWave);
  const TA* yp = static_cast<const TA*>(ye);
  const TA* bp = static_cast<const TA*>(base);
  const TA* rp = static_cast<const TA*>(residual);
  TA* op = static_cast<TA*>(out);
#define FS2_COMBINE_CASE(KM)                                                                      \
  if (K <= KM) {                                                                                  \
    if (wpt == 4)                                                                                 \
      hipLaunchKernelGGL((combine_kernel<TA, KM, 4>), grid, block, 0, s, yp, inv_perm, topk_idx,  \
                         topk_w, bp, rp, T, K, D, weight_output, op);                             \
    else                                                                                          \
      hipLaunchKernelGGL((combine_kernel<TA, KM, 1>), grid, block, 0, s, yp, inv_perm, topk_idx,  \
                         topk_w, bp, rp, T, K, D, weight_output, op);                             \
    return check_launch("combine");                                                               \
  }
  FS2_COMBINE_CASE(1)
  FS2_COMBINE_CASE(2)
  FS2_COMBINE_CASE(4)
  FS2_COMBINE_CASE(8)
  FS2_COMBINE_CASE(16)
  FS2_COMBINE_CASE(32)
#undef FS2_COMBINE_CASE
  set_error("combine: K=%d exceeds %d", K, FS2MOE_MAX_TOP_K);
  return FS2MOE_ERR_UNSUPPORTED;
}

}  // namespace fs2moe

using namespace fs2moe;

static int combine_entry(const void* ye, const int32_t* inv_perm, const int32_t* topk_idx,
                         const float* topk_w, const void* base, const void* residual, int32_t T,
                         int32_t K, int32_t D, int32_t act_dtype, int32_t weight_output, void* out,
                         void* stream) {
  FS2_REQUIRE(ye && inv_perm && topk_idx && out, "combine: null pointer");
  FS2_REQUIRE(!weight_output || topk_w, "combine: weight_output needs topk_w");
  FS2_REQUIRE(T >= 0 && K >= 1 && K <= FS2MOE_MAX_TOP_K, "combine: bad T=%d K=%d", T, K);
  FS2_REQUIRE(act_dtype == FS2MOE_F32 || act_dtype == FS2MOE_BF16, "combine: act_dtype %d",
              act_dtype);
  FS2_REQUIRE(D > 0 && (D * elem_size(act_dtype)) % 16 == 0,
              "combine: D=%d rows are not a multiple of 16 bytes", D);
  FS2_REQUIRE(aligned16(ye) && aligned16(out) && aligned16(base) && aligned16(residual),
              "combine: buffers must be 16-byte aligned");
  if (T == 0) return FS2MOE_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (act_dtype == FS2MOE_F32)
    return launch_combine<float>(ye, inv_perm, topk_idx, topk_w, base, residual, T, K, D,
                                 weight_output, out, s);
  return launch_combine<uint16_t>(ye, inv_perm, topk_idx, topk_w, base, residual, T, K, D,
                                  weight_output, out, s);
}

extern "C" int fs2moe_combine(const void* ye, const int32_t* inv_perm, const int32_t* topk_idx,
                              const float* topk_w, const void* base, int32_t T, int32_t K,
                              int32_t D, int32_t act_dtype, int32_t weight_output, void* out,
                              void* stream) {
  return combine_entry(ye, inv_perm, topk_idx, topk_w, base, nullptr, T, K, D, act_dtype,
                       weight_output, out, stream);
}

extern "C" int fs2moe_combine_residual(const void* ye, const int32_t* inv_perm,
                                       const int32_t* topk_idx, const float* topk_w,
                                       const void* base, const void* residual, int32_t T, int32_t K,
                                       int32_t D, int32_t act_dtype, int32_t weight_output,
                                       void* out, void* stream) {
  FS2_REQUIRE(residual != nullptr, "combine_residual: null residual");
  return combine_entry(ye, inv_perm, topk_idx, topk_w, base, residual, T, K, D, act_dtype,
                       weight_output, out, stream);
}

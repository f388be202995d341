// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fs2moe.h"

namespace fs2moe {

constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;

// ---- bf16 <-> f32 (round to nearest even, NaN kept quiet) -------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
// Two floats -> packed bf16 pair in one v_cvt_pk_bf16_f32 (round to nearest even; lo in bits 0..15).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// Two bf16 values times an f32 weight, each product rounded to bf16: what dispatch stores when it
// copies a row scaled by its routing weight, and what a kernel that scales the row on the way in
// must compute to give the same bits.
__device__ __forceinline__ uint32_t scale_bf16x2(uint32_t v, float w) {
  return pack_bf16x2(__uint_as_float(v << 16) * w, __uint_as_float(v & 0xffff0000u) * w);
}

template <typename T>
struct Elem;
template <>
struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
};
template <>
struct Elem<uint16_t> {  // bf16 bit pattern
  static __device__ __forceinline__ float load(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  static __device__ __forceinline__ void store(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
};

// v * sigmoid(v) with the hardware reciprocal (1 ulp), not a full-precision division.
__device__ __forceinline__ float silu_f32(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
}

// ---- wave-level helpers -------------------------------------------------------------------------
__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// Wave-wide reductions on the DPP data path (no LDS round trips).  Four butterfly steps inside each
// row of 16 lanes (xor 1, xor 2, half-row mirror, row mirror), then row_bcast:15 into rows 1 and 3
// and row_bcast:31 into rows 2 and 3 leave the result in row 3; lane 63 is broadcast to all lanes.
constexpr int kDppXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // row_half_mirror
constexpr int kDppMirror = 0x140;     // row_mirror
constexpr int kDppBcast15 = 0x142;    // row_bcast:15
constexpr int kDppBcast31 = 0x143;    // row_bcast:31

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint64_t dpp_max_step_u64(uint64_t v) {
  const int lo = (int)(uint32_t)v, hi = (int)(uint32_t)(v >> 32);
  // lanes outside ROW_MASK (or without a source lane) keep their own value
  const uint32_t olo = (uint32_t)__builtin_amdgcn_update_dpp(lo, lo, CTRL, ROW_MASK, 0xf, false);
  const uint32_t ohi = (uint32_t)__builtin_amdgcn_update_dpp(hi, hi, CTRL, ROW_MASK, 0xf, false);
  const uint64_t o = ((uint64_t)ohi << 32) | olo;
  return o > v ? o : v;
}
__device__ __forceinline__ uint64_t wave_max_u64(uint64_t v) {
  v = dpp_max_step_u64<kDppXor1, 0xf>(v);
  v = dpp_max_step_u64<kDppXor2, 0xf>(v);
  v = dpp_max_step_u64<kDppHalfMirror, 0xf>(v);
  v = dpp_max_step_u64<kDppMirror, 0xf>(v);
  v = dpp_max_step_u64<kDppBcast15, 0xa>(v);
  v = dpp_max_step_u64<kDppBcast31, 0xc>(v);
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 63);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), 63);
  return ((uint64_t)hi << 32) | lo;
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_max_step_u32(uint32_t v) {
  // lanes outside ROW_MASK (or without a source lane) keep their own value
  const uint32_t o =
      (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROW_MASK, 0xf, false);
  return o > v ? o : v;
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = dpp_max_step_u32<kDppXor1, 0xf>(v);
  v = dpp_max_step_u32<kDppXor2, 0xf>(v);
  v = dpp_max_step_u32<kDppHalfMirror, 0xf>(v);
  v = dpp_max_step_u32<kDppMirror, 0xf>(v);
  v = dpp_max_step_u32<kDppBcast15, 0xa>(v);
  v = dpp_max_step_u32<kDppBcast31, 0xc>(v);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add_step_f32(float v) {
  // lanes outside ROW_MASK (or without a source lane) add zero
  const int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false);
  return v + __int_as_float(o);
}
__device__ __forceinline__ float wave_sum_f32(float v) {
  v = dpp_add_step_f32<kDppXor1, 0xf>(v);
  v = dpp_add_step_f32<kDppXor2, 0xf>(v);
  v = dpp_add_step_f32<kDppHalfMirror, 0xf>(v);
  v = dpp_add_step_f32<kDppMirror, 0xf>(v);
  v = dpp_add_step_f32<kDppBcast15, 0xa>(v);
  v = dpp_add_step_f32<kDppBcast31, 0xc>(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// ---- MFMA operand fragments from LDS ---------------------------------------------------------------
// Plain: the lane's 8 consecutive k values lie contiguously (k-contiguous tile).
// Transposing: the tile is n-contiguous; ds_read_tr16_b64 hands lane i of each 16-lane group element
// (i % 4) of lanes i/4, i/4+4, i/4+8, i/4+12, i.e. a 4(k) x 16(n) block transposed.  p_lo / p_hi point at
// this lane's 4-element source chunk in k rows [k0, k0+4) and [k0+4, k0+8).
__device__ __forceinline__ bf16x8 lds_read_frag(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ bf16x8 lds_read_frag_tr(const uint16_t* p_lo, const uint16_t* p_hi) {
  typedef __attribute__((address_space(3))) s16x4* lds_ptr;
  s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p_lo));
  s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p_hi));
  s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(bf16x8, v);
}

// Block barrier that orders LDS traffic only.  __syncthreads() also fences global memory, for which
// the compiler drains every outstanding global load (s_waitcnt vmcnt(0)); loops that keep a register
// set of loads in flight across their barriers, and synchronise on nothing that lives in global
// memory, use this one.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// 8 e4m3 codes (two dwords) -> 8 bf16 values.
__device__ __forceinline__ bf16x8 fp8x8_to_bf16x8(uint32_t lo, uint32_t hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  u32x4 out;
  const uint32_t w[2] = {lo, hi};
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], false);  // bytes 0, 1
    const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w[i], true);   // bytes 2, 3
    out[2 * i] = (__float_as_uint(a[0]) >> 16) | (__float_as_uint(a[1]) & 0xffff0000u);
    out[2 * i + 1] = (__float_as_uint(b[0]) >> 16) | (__float_as_uint(b[1]) & 0xffff0000u);
  }
  return __builtin_bit_cast(bf16x8, out);
}

// ---- host side -----------------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int elem_size(int dtype) { return dtype == FS2MOE_F32 ? 4 : dtype == FS2MOE_BF16 ? 2 : 1; }

// Where the whole-layer call wants its dispatch (no rows copied): with at most 32 bf16 tokens the
// router's finishing kernel ends with it, and where one block routes a whole tile of 32 tokens from an
// (E, D) matrix (up to kIndexTilesMax tiles) that block also counts the tile's pairs per expert and
// ranks them, which leaves one dispatch kernel to run (dispatch_index_tiles); both set `done`.  At
// any other size the router leaves `done` false and the caller runs fs2moe_dispatch.  Either way the
// arrays hold the same values.  `ws` is the dispatch workspace (fs2moe_dispatch_workspace_bytes).
struct DispatchAfterRouter {
  int tile_m;
  int64_t max_rows;
  int32_t *counts, *offsets, *perm, *inv_perm;
  void* ws;
  int64_t ws_bytes;
  // optional (bf16 decode sizes, rows scaled by the routing weight on their way into the experts
  // instead of by a copy): per expert row the weight of its pair, written next to perm
  float* row_w;
  bool done;
};
constexpr int kRouterTileTok = 32;   // tokens per tile of the MFMA routers
constexpr int kIndexTilesMax = 512;  // tiles whose counts every block of dispatch_index_tiles adds up
// The dispatch workspace as the tile-counting router fills it: per tile and expert the number of the
// tile's tokens that chose the expert (a byte: at most 32), then per pair its rank among the tile's
// pairs of the same expert.
inline uint8_t* tile_counts_of(void* ws) { return static_cast<uint8_t*>(ws); }
inline int32_t* tile_rank_of(void* ws, int T, int E) {
  const int64_t nt = (T + kRouterTileTok - 1) / kRouterTileTok;
  return reinterpret_cast<int32_t*>(static_cast<uint8_t*>(ws) + (nt * E + 255) / 256 * 256);
}
// The rest of dispatch after such a router: offsets, counts, perm and inv_perm as fs2moe_dispatch
// writes them without a row copy.  E a multiple of 8, at most 256; at most kIndexTilesMax tiles.
int dispatch_index_tiles(const int32_t* topk_idx, int32_t T, int32_t K, int32_t E, int32_t tile_m,
                         int64_t max_rows, const uint8_t* tile_counts, const int32_t* tile_rank,
                         int32_t* counts, int32_t* offsets, int32_t* perm, int32_t* inv_perm,
                         void* stream);
// fs2moe_router_topk (xn null) or fs2moe_router_topk_norm, without the logits output
int router_then_dispatch(const void* x, const void* norm_w, float norm_eps, void* xn,
                         const void* router, const float* bias, int32_t T, int32_t D, int32_t E,
                         int32_t K, int32_t act_dtype, int32_t score_fn, int32_t renormalize,
                         int32_t* topk_idx, float* topk_w, void* workspace, int64_t workspace_bytes,
                         DispatchAfterRouter* disp, void* stream);

// fs2moe_dispatch without a row copy that also writes row_w[row] = topk_w[pair] (see
// DispatchAfterRouter): at most 256 tokens and 256 experts, K <= 16 or not.
int dispatch_with_row_weights(const int32_t* topk_idx, const float* topk_w, int32_t T, int32_t K,
                              int32_t E, int32_t tile_m, int64_t max_rows, int32_t* counts,
                              int32_t* offsets, int32_t* perm, int32_t* inv_perm, float* row_w,
                              void* stream);
// Whether the grouped SwiGLU pair of these sizes runs on the kernels that stream the weights past a
// few staged rows (at most rows_per_expert of any expert), which can scale each row by row_w as
// they stage it; and that pair: fs2moe_grouped_swiglu_rows with rows read through row_map and
// multiplied by row_w[row] (rounded to bf16, as dispatch's scaled copy rounds them).
bool swiglu_streams_rows(int32_t act_dtype, int32_t w_dtype, int32_t D, int32_t F, int32_t E,
                         int32_t rows_per_expert);
int grouped_swiglu_scaled_rows(const void* x, const int32_t* row_map, const float* row_w,
                               const int32_t* counts, const int32_t* offsets, const void* w_gate,
                               const void* w_up, const void* w_down, int32_t E, int32_t D, int32_t F,
                               int64_t max_rows, void* h, void* ye, int32_t rows_per_expert,
                               void* stream);

}  // namespace fs2moe

#define FS2_REQUIRE(cond, ...)          \
  do {                                  \
    if (!(cond)) {                      \
      fs2moe::set_error(__VA_ARGS__);   \
      return FS2MOE_ERR_ARG;            \
    }                                   \
  } while (0)

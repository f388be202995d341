// Grouped SwiGLU expert GEMMs on MFMA.
//
// Both GEMMs of an expert network run as "grouped" GEMMs over the expert-contiguous row buffer:
//   H = SiLU(X Wg) * (X Wu)   (DUAL: two weight tiles share one activation tile, gate fused)
//   Y = H Wd
// A block owns a BM x BN output tile of one expert.  The tile -> (expert, row range) map is
// derived on the device from counts/offsets, so nothing is read back to the host.
//
// MFMA operand roles are swapped with respect to the textbook: the weight fragment is the "A"
// operand (rows = output channels n) and the activation fragment the "B" operand (columns = rows
// m of X), which yields the transposed tile.  In the 32x32 accumulator layout a lane then holds
// four CONSECUTIVE output channels of one row m, so results leave as 8-byte (bf16) or 16-byte
// (f32) stores without a trip through LDS.
//
// Expert weights are stored "in x out" (k-major rows, n contiguous: experts.py:53-82), but an MFMA
// operand lane needs 8 consecutive k for one n.  The tile is written to LDS as it lies in memory
// and read back with ds_read_tr16_b64, the gfx950 transposing LDS load: within 16 lanes, lane i
// receives element (i % 4) of lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 -- a 4(k) x 16(n) block
// transposed on the fly.  nn.Linear-oriented weights (the shared expert) are already k-contiguous
// and use plain 16-byte LDS reads.
#include "common.h"
#include "tile_map.h"
#include "experts_dma.h"
#include "experts_fp8.h"
#include "experts_gemv.h"

namespace fs2moe {

// ------------------------------------------------------------------------------------ bf16, 128-row tiles (any D, F multiple of 8)
namespace bf16k {
constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDA = BK + 8;    // sA row stride (elements): 144 B, conflict-free 16-byte reads
constexpr int LDB_KN = BN + 32;  // sB row stride for k-major tiles: 320 B
constexpr int LDB_NK = BK + 8;
}  // namespace bf16k

template <bool DUAL, int BLAYOUT>
__global__ __launch_bounds__(256, 2) void glu_gemm_bf16_kernel(
    const uint16_t* __restrict__ A, int lda, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, uint16_t* __restrict__ C, int ldc, int Kdim, int N, Groups g,
    int n_tiles) {
  using namespace bf16k;
  constexpr int NB = DUAL ? 2 : 1;
  constexpr bool KN = BLAYOUT == FS2MOE_W_IN_OUT;
  constexpr int SB_ELEMS = KN ? BK * LDB_KN : BN * LDB_NK;
  __shared__ __attribute__((aligned(16))) uint16_t sA[BM * LDA];
  __shared__ __attribute__((aligned(16))) uint16_t sB[NB][SB_ELEMS];

  const int tid = threadIdx.x;
  const int mt = blockIdx.x / n_tiles, nt = blockIdx.x - mt * n_tiles;
  int e, row0, row_end;
  if (!locate_tile<BM>(g, mt, e, row0, row_end)) return;
  const int n0 = nt * BN;
  const size_t wstride = (size_t)Kdim * N;
  const uint16_t* Bp[2] = {B0 + (size_t)e * wstride, DUAL ? B1 + (size_t)e * wstride : nullptr};

  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int lr = lane & 31, lk = lane >> 5;
  bool fm_active[2];
#pragma unroll
  for (int fm = 0; fm < 2; ++fm) fm_active[fm] = row0 + wm * 64 + fm * 32 < row_end;

  f32x16 acc[NB][2][2];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int fn = 0; fn < 2; ++fn)
#pragma unroll
      for (int fm = 0; fm < 2; ++fm)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[b][fn][fm][i] = 0.f;

  u32x4 ra[4], rb[NB][4];
  const u32x4 zero4 = {0u, 0u, 0u, 0u};

  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + 256 * i;
      const int row = c >> 3, kc = c & 7;
      int grow = row0 + row;
      grow = grow < row_end ? grow : row_end - 1;
      const int k = k0 + kc * 8;
      ra[i] = k < Kdim ? *reinterpret_cast<const u32x4*>(A + (size_t)grow * lda + k) : zero4;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i;
        if (KN) {
          const int k = k0 + (c >> 4), n = n0 + (c & 15) * 8;
          rb[b][i] = (k < Kdim && n < N)
                         ? *reinterpret_cast<const u32x4*>(Bp[b] + (size_t)k * N + n)
                         : zero4;
        } else {
          const int n = n0 + (c >> 3), k = k0 + (c & 7) * 8;
          rb[b][i] = (k < Kdim && n < N)
                         ? *reinterpret_cast<const u32x4*>(Bp[b] + (size_t)n * Kdim + k)
                         : zero4;
        }
      }
    }
  };
  auto store_lds = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c = tid + 256 * i;
      *reinterpret_cast<u32x4*>(&sA[(c >> 3) * LDA + (c & 7) * 8]) = ra[i];
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = tid + 256 * i;
        if (KN)
          *reinterpret_cast<u32x4*>(&sB[b][(c >> 4) * LDB_KN + (c & 15) * 8]) = rb[b][i];
        else
          *reinterpret_cast<u32x4*>(&sB[b][(c >> 3) * LDB_NK + (c & 7) * 8]) = rb[b][i];
      }
    }
  };

  const int nk = (Kdim + BK - 1) / BK;
  load_global(0);
  for (int kt = 0; kt < nk; ++kt) {
    store_lds();
    __syncthreads();
    if (kt + 1 < nk) load_global((kt + 1) * BK);
    if (fm_active[0]) {
#pragma unroll
      for (int ks = 0; ks < BK / 16; ++ks) {
        bf16x8 xf[2];
#pragma unroll
        for (int fm = 0; fm < 2; ++fm)
          xf[fm] = lds_read_frag(&sA[(wm * 64 + fm * 32 + lr) * LDA + ks * 16 + lk * 8]);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
#pragma unroll
          for (int fn = 0; fn < 2; ++fn) {
            bf16x8 wf;
            if (KN) {
              const int s = lane & 15, half = (lane >> 4) & 1;
              const int kr = ks * 16 + lk * 8 + (s >> 2);
              const int col = wn * 64 + fn * 32 + half * 16 + (s & 3) * 4;
              wf = lds_read_frag_tr(&sB[b][kr * LDB_KN + col], &sB[b][(kr + 4) * LDB_KN + col]);
            } else {
              wf = lds_read_frag(&sB[b][(wn * 64 + fn * 32 + lr) * LDB_NK + ks * 16 + lk * 8]);
            }
            acc[b][fn][0] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[0], acc[b][fn][0], 0, 0, 0);
            if (fm_active[1])
              acc[b][fn][1] =
                  __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[1], acc[b][fn][1], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();
  }

  // Epilogue: lane holds, for row m, channels n = nb + 8q + 4*lk + {0..3}, q = 0..3.
#pragma unroll
  for (int fm = 0; fm < 2; ++fm) {
    const int m = row0 + wm * 64 + fm * 32 + lr;
    if (m >= row_end) continue;
#pragma unroll
    for (int fn = 0; fn < 2; ++fn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 64 + fn * 32 + 8 * q + 4 * lk;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (DUAL)
            v[j] = silu_f32(acc[0][fn][fm][4 * q + j]) * acc[NB - 1][fn][fm][4 * q + j];
          else
            v[j] = acc[0][fn][fm][4 * q + j];
        }
        u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *reinterpret_cast<u32x2*>(C + (size_t)m * ldc + n) = o;
      }
    }
  }
}

// ------------------------------------------------------------------------------------- f32
// Same schedule with v_mfma_f32_32x32x2_f32 (true f32 FMA); tiles are smaller because the
// operands are four bytes wide.  This path serves the fp32 reference configuration.
namespace f32k {
constexpr int BM = 64, BN = 64, BK = 16;
constexpr int LDA = BK + 4;
constexpr int LDB_KN = BN + 4;
constexpr int LDB_NK = BK + 4;
}  // namespace f32k

template <bool DUAL, int BLAYOUT>
__global__ __launch_bounds__(256) void glu_gemm_f32_kernel(
    const float* __restrict__ A, int lda, const float* __restrict__ B0,
    const float* __restrict__ B1, float* __restrict__ C, int ldc, int Kdim, int N, Groups g,
    int n_tiles) {
  using namespace f32k;
  constexpr int NB = DUAL ? 2 : 1;
  constexpr bool KN = BLAYOUT == FS2MOE_W_IN_OUT;
  constexpr int SB_ELEMS = KN ? BK * LDB_KN : BN * LDB_NK;
  __shared__ __attribute__((aligned(16))) float sA[BM * LDA];
  __shared__ __attribute__((aligned(16))) float sB[NB][SB_ELEMS];

  const int tid = threadIdx.x;
  const int mt = blockIdx.x / n_tiles, nt = blockIdx.x - mt * n_tiles;
  int e, row0, row_end;
  if (!locate_tile<BM>(g, mt, e, row0, row_end)) return;
  const int n0 = nt * BN;
  const size_t wstride = (size_t)Kdim * N;
  const float* Bp[2] = {B0 + (size_t)e * wstride, DUAL ? B1 + (size_t)e * wstride : nullptr};

  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;
  const int lr = lane & 31, lk = lane >> 5;

  f32x16 acc[NB];
#pragma unroll
  for (int b = 0; b < NB; ++b)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[b][i] = 0.f;

  f32x4 ra, rb[NB];
  const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
  auto load_global = [&](int k0) {
    {
      const int row = tid >> 2, kc = tid & 3;
      int grow = row0 + row;
      grow = grow < row_end ? grow : row_end - 1;
      const int k = k0 + kc * 4;
      ra = k < Kdim ? *reinterpret_cast<const f32x4*>(A + (size_t)grow * lda + k) : zero4;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (KN) {
        const int k = k0 + (tid >> 4), n = n0 + (tid & 15) * 4;
        rb[b] = (k < Kdim && n < N) ? *reinterpret_cast<const f32x4*>(Bp[b] + (size_t)k * N + n)
                                    : zero4;
      } else {
        const int n = n0 + (tid >> 2), k = k0 + (tid & 3) * 4;
        rb[b] = (k < Kdim && n < N)
                    ? *reinterpret_cast<const f32x4*>(Bp[b] + (size_t)n * Kdim + k)
                    : zero4;
      }
    }
  };
  auto store_lds = [&]() {
    *reinterpret_cast<f32x4*>(&sA[(tid >> 2) * LDA + (tid & 3) * 4]) = ra;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if (KN)
        *reinterpret_cast<f32x4*>(&sB[b][(tid >> 4) * LDB_KN + (tid & 15) * 4]) = rb[b];
      else
        *reinterpret_cast<f32x4*>(&sB[b][(tid >> 2) * LDB_NK + (tid & 3) * 4]) = rb[b];
    }
  };

  const bool active = row0 + wm * 32 < row_end;
  const int nk = (Kdim + BK - 1) / BK;
  load_global(0);
  for (int kt = 0; kt < nk; ++kt) {
    store_lds();
    __syncthreads();
    if (kt + 1 < nk) load_global((kt + 1) * BK);
    if (active) {
#pragma unroll
      for (int ks = 0; ks < BK / 2; ++ks) {
        const int k = ks * 2 + lk;
        const float xf = sA[(wm * 32 + lr) * LDA + k];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
          const float wf = KN ? sB[b][k * LDB_KN + wn * 32 + lr] : sB[b][(wn * 32 + lr) * LDB_NK + k];
          acc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(wf, xf, acc[b], 0, 0, 0);
        }
      }
    }
    __syncthreads();
  }

  const int m = row0 + wm * 32 + lr;
  if (m >= row_end) return;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int n = n0 + wn * 32 + 8 * q + 4 * lk;
    if (n >= N) continue;
    f32x4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (DUAL) {
        const float gte = acc[0][4 * q + j];
        v[j] = (gte / (1.0f + expf(-gte))) * acc[NB - 1][4 * q + j];
      } else {
        v[j] = acc[0][4 * q + j];
      }
    }
    *reinterpret_cast<f32x4*>(C + (size_t)m * ldc + n) = v;
  }
}

// ------------------------------------------------------------------------------------ host
// Compute units of the current device, rounded down to a multiple of its 8 XCDs (0 on failure).
static int cu_count_by_xcd() {
  static int cached = 0;  // benign race: every thread computes the same value
  if (cached == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus < 8)
      return 0;
    cached = cus / 8 * 8;
  }
  return cached;
}

// e4m3 weights go to the throughput kernel from this many rows per expert on (mean over all experts)
#ifndef FS2MOE_FP8_GEMM_MIN_ROWS
#define FS2MOE_FP8_GEMM_MIN_ROWS 32
#endif
constexpr int64_t kFp8GemmMinRowsPerExpert = FS2MOE_FP8_GEMM_MIN_ROWS;

static bool dma_path_applies(int act_dtype, int D, int F) {
  return act_dtype == FS2MOE_BF16 && D % (2 * dma::BK) == 0 && F % (2 * dma::BK) == 0;
}

// The bf16 throughput kernel pair (gate/up, then down) on persistent blocks; BLAYOUT as the kernel
// takes it, scales only with dma::W_FP8_TILED.  The caller has checked that the path applies.
template <int BLAYOUT>
static int launch_dma_pair(const void* x, const int32_t* row_map, const Groups& g,
                           int64_t rows_bound, const void* w_gate, const void* w_up,
                           const void* w_down, const float* s_gate, const float* s_up,
                           const float* s_down, int D, int F, void* h, void* y,
                           hipStream_t stream, void* g_keep = nullptr, void* u_keep = nullptr) {
  using namespace dma;
  const int groups = g.counts ? g.E : 0;
  // the gate/up kernel, or its variant that also stores the two products (plain bf16 weights only)
  constexpr bool CAN_KEEP = BLAYOUT != dma::W_FP8_TILED;
  auto k1 = glu_gemm_bf16_dma_kernel<true, BLAYOUT>;
  auto k1k = glu_gemm_bf16_dma_kernel<true, BLAYOUT, CAN_KEEP>;
  auto k2 = glu_gemm_bf16_dma_kernel<false, BLAYOUT>;
  if (g_keep != nullptr && !CAN_KEEP) {
    set_error("experts: the products are kept with bf16 weights only");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    const void* ks[3] = {reinterpret_cast<const void*>(k1), reinterpret_cast<const void*>(k1k),
                         reinterpret_cast<const void*>(k2)};
    for (const void* k : ks) {
      hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
      if (e != hipSuccess) {
        set_error("experts: cannot reserve %d bytes of LDS: %s", SMEM_BYTES, hipGetErrorString(e));
        return FS2MOE_ERR_LAUNCH;
      }
    }
    attr_set = true;
  }
  // Persistent blocks: one per CU (the 128 KB ring allows no more), a multiple of the 8 XCDs.
  const int num_blocks = cu_count_by_xcd();
  if (num_blocks == 0) {
    set_error("experts: cannot query the compute-unit count");
    return FS2MOE_ERR_LAUNCH;
  }
  const int nt1 = (F + 127) / 128, nt2 = (D + 255) / 256;
  {
    const int64_t m_tiles = rows_bound / BM + groups + 1;
    if (m_tiles * nt1 > 0x7fffffffll || m_tiles * nt2 > 0x7fffffffll) {
      set_error("experts: too many tiles");
      return FS2MOE_ERR_UNSUPPORTED;
    }
  }
  const unsigned g1 = (unsigned)num_blocks, g2 = (unsigned)num_blocks;
  // (the variant that keeps the products takes their destinations in the two scale arguments)
  hipLaunchKernelGGL(g_keep != nullptr ? k1k : k1, dim3(g1), dim3(NWAVES * 64), SMEM_BYTES, stream,
                     static_cast<const uint16_t*>(x), row_map, D,
                     static_cast<const uint16_t*>(w_gate), static_cast<const uint16_t*>(w_up),
                     g_keep != nullptr ? static_cast<const float*>(g_keep) : s_gate,
                     g_keep != nullptr ? static_cast<const float*>(u_keep) : s_up,
                     static_cast<uint16_t*>(h), F, D, F, g, nt1);
  if (int rc = check_launch("glu_gemm_bf16_dma<gate,up>")) return rc;
  hipLaunchKernelGGL(k2, dim3(g2), dim3(NWAVES * 64), SMEM_BYTES, stream,
                     static_cast<const uint16_t*>(h), static_cast<const int32_t*>(nullptr), F,
                     static_cast<const uint16_t*>(w_down), static_cast<const uint16_t*>(nullptr),
                     s_down, static_cast<const float*>(nullptr), static_cast<uint16_t*>(y), D, F, D, g,
                     nt2);
  return check_launch("glu_gemm_bf16_dma<down>");
}

// The throughput kernel addresses activations and one expert's weights with 32-bit byte offsets.
static bool dma_offsets_fit(int64_t rows_bound, int D, int F) {
  const int64_t wide = D > F ? D : F;
  return rows_bound * wide * 2 <= 0xffffffffll && (int64_t)D * F * 2 <= 0xffffffffll;
}

// The streaming pair for at most `rows_hint` rows per expert: see experts_gemv.h.  Measured on the
// Qwen3 layer shape (bf16 weights, whole layer, against the GEMM tiles): 1 token 44-47 against 69 us,
// 2 tokens 52 against 70, 3 tokens 56 against 71, 4 tokens 61 against 72; from 5 rows on the vector
// ALUs fall behind (8 tokens: 95 against 84 us), so the bound stops at 4 and the matrix-pipe stream
// below takes over.
#ifndef FS2MOE_GEMV_MAX_ROWS
#define FS2MOE_GEMV_MAX_ROWS 4
#endif
static bool gemv_applies(int act_dtype, int D, int F, const Groups& g, int rows_hint) {
  // (the stream kernels find their expert with four ballots over the counts: up to 256 experts)
  if (act_dtype != FS2MOE_BF16 || g.counts == nullptr || g.E > 256 || rows_hint < 1 ||
      rows_hint > FS2MOE_GEMV_MAX_ROWS)
    return false;
  const int r = rows_hint <= 1 ? 1 : rows_hint <= 2 ? 2 : 4;
  return gemv::fits(D > F ? D : F, r);
}

template <int R>
static int launch_gemv_pair_r(const void* x, const int32_t* row_map, const float* row_w,
                              const Groups& g, const void* w_gate, const void* w_up,
                              const void* w_down, int D, int F, void* h, void* y,
                              hipStream_t stream) {
  using namespace gemv;
  auto k1 = glu_gemv_bf16_kernel<true, R>;
  auto k2 = glu_gemv_bf16_kernel<false, R>;
  auto k2d = glu_gemv_bf16_kernel<false, R, true>;  // more loads in flight over a long K
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k1),
                            hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(k2d),
                            hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(k2),
                            hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS_BYTES) != hipSuccess) {
      set_error("experts: cannot reserve %d bytes of LDS", MAX_LDS_BYTES);
      return FS2MOE_ERR_LAUNCH;
    }
    attr_set = true;
  }
  const uint16_t* xp = static_cast<const uint16_t*>(x);
  hipLaunchKernelGGL(k1, dim3((unsigned)((F + COLS - 1) / COLS), (unsigned)g.E), dim3(threads(R)),
                     (size_t)R * D * 2, stream, xp, row_map, row_w, D, static_cast<const uint16_t*>(w_gate),
                     static_cast<const uint16_t*>(w_up), static_cast<uint16_t*>(h), F, D, F,
                     g.counts, g.offsets);
  if (int rc = check_launch("glu_gemv_bf16<gate,up>")) return rc;
  hipLaunchKernelGGL(deep_applies(F, R) ? k2d : k2, dim3((unsigned)((D + COLS - 1) / COLS), (unsigned)g.E),
                     dim3(threads(R)), (size_t)R * F * 2, stream, static_cast<const uint16_t*>(h),
                     static_cast<const int32_t*>(nullptr), static_cast<const float*>(nullptr), F,
                     static_cast<const uint16_t*>(w_down),
                     static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(y), D, F, D,
                     g.counts, g.offsets);
  return check_launch("glu_gemv_bf16<down>");
}

// The same for 5 to 16 rows per expert, on the matrix pipe (glu_gemv16_bf16_kernel).  Whole layer at
// the Qwen3 shape against the GEMM tiles: 5 tokens 57 against 72 us, 8 tokens 69-71 against 79, 12
// tokens 71 against 81, 16 tokens 78 against 83.  At 3 and 4 rows it ties with the vector-ALU stream (53.5
// against 52.4 and 56.5 against 57.6 us), at 1 and 2 it loses (48 against 41, 53 against 48: half as
// many blocks per expert).
#ifndef FS2MOE_GEMV16_MAX_ROWS
#define FS2MOE_GEMV16_MAX_ROWS 16
#endif
static bool gemv16_applies(int act_dtype, int D, int F, const Groups& g, int rows_hint) {
  if (act_dtype != FS2MOE_BF16 || g.counts == nullptr || g.E > 256 ||
      rows_hint <= FS2MOE_GEMV_MAX_ROWS || rows_hint > FS2MOE_GEMV16_MAX_ROWS)
    return false;
  return gemv16::offsets_fit(D, F) && gemv16::fits(D > F ? D : F, 8);
}
// rows staged per pass: 16 when the bound asks for it and rows that long fit LDS, else 8 (an expert
// with more rows is walked again)
static int gemv16_rows(int D, int F, int rows_hint) {
  return rows_hint > 8 && gemv16::fits(D > F ? D : F, 16) ? 16 : 8;
}

template <int XR>
static int launch_gemv16_pair(const void* x, const int32_t* row_map, const float* row_w,
                              const Groups& g, const void* w_gate, const void* w_up,
                              const void* w_down, int D, int F, void* h, void* y,
                              hipStream_t stream) {
  using namespace gemv16;
  auto k1 = glu_gemv16_bf16_kernel<true, XR>;
  auto k2 = glu_gemv16_bf16_kernel<false, XR>;
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(k1),
                            hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS_BYTES) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(k2),
                            hipFuncAttributeMaxDynamicSharedMemorySize, MAX_LDS_BYTES) != hipSuccess) {
      set_error("experts: cannot reserve %d bytes of LDS", MAX_LDS_BYTES);
      return FS2MOE_ERR_LAUNCH;
    }
    attr_set = true;
  }
  hipLaunchKernelGGL(k1, dim3((unsigned)((F + COLS - 1) / COLS), (unsigned)g.E), dim3(THREADS),
                     lds_bytes(D, XR, true), stream, static_cast<const uint16_t*>(x), row_map, row_w, D,
                     static_cast<const uint16_t*>(w_gate), static_cast<const uint16_t*>(w_up),
                     static_cast<uint16_t*>(h), F, D, F, g.counts, g.offsets);
  if (int rc = check_launch("glu_gemv16_bf16<gate,up>")) return rc;
  hipLaunchKernelGGL(k2, dim3((unsigned)((D + COLS - 1) / COLS), (unsigned)g.E), dim3(THREADS),
                     lds_bytes(F, XR, false), stream, static_cast<const uint16_t*>(h),
                     static_cast<const int32_t*>(nullptr), static_cast<const float*>(nullptr), F,
                     static_cast<const uint16_t*>(w_down),
                     static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(y), D, F, D,
                     g.counts, g.offsets);
  return check_launch("glu_gemv16_bf16<down>");
}

// The dense SwiGLU (the shared expert, weights (N, K)) of up to 16 bf16 rows: dense_gemv_bf16_kernel.
// Llama-4 Scout's shared expert (D 5120, F 8192): 1 token 172 us on the GEMM tiles.
static bool dense_gemv_applies(int act_dtype, const Groups& g, int64_t rows) {
  return act_dtype == FS2MOE_BF16 && g.counts == nullptr && rows >= 1 && rows <= dgemv::MAX_ROWS;
}
static int launch_dense_gemv_pair(const void* x, int T, const void* w_gate, const void* w_up,
                                  const void* w_down, int D, int F, void* h, void* y,
                                  hipStream_t stream) {
  using namespace dgemv;
  hipLaunchKernelGGL(dense_gemv_bf16_kernel<true>, dim3((unsigned)((F + 15) / 16)), dim3(THREADS), 0,
                     stream, static_cast<const uint16_t*>(x), D, static_cast<const uint16_t*>(w_gate),
                     static_cast<const uint16_t*>(w_up), static_cast<uint16_t*>(h), F, D, F, T);
  if (int rc = check_launch("dense_gemv_bf16<gate,up>")) return rc;
  hipLaunchKernelGGL(dense_gemv_bf16_kernel<false>, dim3((unsigned)((D + 15) / 16)), dim3(THREADS), 0,
                     stream, static_cast<const uint16_t*>(h), F, static_cast<const uint16_t*>(w_down),
                     static_cast<const uint16_t*>(nullptr), static_cast<uint16_t*>(y), D, F, D, T);
  return check_launch("dense_gemv_bf16<down>");
}

// rows_hint: an upper bound on the rows of any one expert when the caller knows one (the number of
// tokens is one: a token takes an expert at most once), else 0.
template <int BLAYOUT>
static int launch_glu(const void* x, const int32_t* row_map, const Groups& g, int64_t rows_bound,
                      const void* w_gate, const void* w_up, const void* w_down, int D, int F,
                      int act_dtype, void* h, void* y, hipStream_t stream, int rows_hint = 0,
                      const float* row_w = nullptr) {
  const int groups = g.counts ? g.E : 0;
  if constexpr (BLAYOUT == FS2MOE_W_OUT_IN) {
    if (row_map == nullptr && dense_gemv_applies(act_dtype, g, rows_bound))
      return launch_dense_gemv_pair(x, (int)rows_bound, w_gate, w_up, w_down, D, F, h, y, stream);
  }
  if constexpr (BLAYOUT == FS2MOE_W_IN_OUT) {
    if (gemv_applies(act_dtype, D, F, g, rows_hint)) {
      if (rows_hint <= 1) return launch_gemv_pair_r<1>(x, row_map, row_w, g, w_gate, w_up, w_down, D, F, h, y, stream);
      if (rows_hint <= 2) return launch_gemv_pair_r<2>(x, row_map, row_w, g, w_gate, w_up, w_down, D, F, h, y, stream);
      return launch_gemv_pair_r<4>(x, row_map, row_w, g, w_gate, w_up, w_down, D, F, h, y, stream);
    }
    if (gemv16_applies(act_dtype, D, F, g, rows_hint)) {
      if (gemv16_rows(D, F, rows_hint) == 8)
        return launch_gemv16_pair<8>(x, row_map, row_w, g, w_gate, w_up, w_down, D, F, h, y, stream);
      return launch_gemv16_pair<16>(x, row_map, row_w, g, w_gate, w_up, w_down, D, F, h, y, stream);
    }
  }
  if (row_w != nullptr) {
    set_error("experts: internal: row weights given to kernels that do not scale rows");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  if (dma_path_applies(act_dtype, D, F) && dma_offsets_fit(rows_bound, D, F))
    return launch_dma_pair<BLAYOUT>(x, row_map, g, rows_bound, w_gate, w_up, w_down, nullptr, nullptr,
                                    nullptr, D, F, h, y, stream);
  if (row_map != nullptr) {
    set_error("experts: the fused gather needs bf16, D and F multiples of 64 and activation "
              "matrices below 4 GB");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  if (act_dtype == FS2MOE_BF16) {
    using namespace bf16k;
    const int64_t m_tiles = rows_bound / BM + groups + 1;
    const int nt1 = (F + BN - 1) / BN, nt2 = (D + BN - 1) / BN;
    if (m_tiles * nt1 > 0x7fffffffll || m_tiles * nt2 > 0x7fffffffll) {
      set_error("experts: grid too large");
      return FS2MOE_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL((glu_gemm_bf16_kernel<true, BLAYOUT>), dim3((unsigned)(m_tiles * nt1)),
                       dim3(256), 0, stream, static_cast<const uint16_t*>(x), D,
                       static_cast<const uint16_t*>(w_gate), static_cast<const uint16_t*>(w_up),
                       static_cast<uint16_t*>(h), F, D, F, g, nt1);
    if (int rc = check_launch("glu_gemm_bf16<gate,up>")) return rc;
    hipLaunchKernelGGL((glu_gemm_bf16_kernel<false, BLAYOUT>), dim3((unsigned)(m_tiles * nt2)),
                       dim3(256), 0, stream, static_cast<const uint16_t*>(h), F,
                       static_cast<const uint16_t*>(w_down), static_cast<const uint16_t*>(nullptr),
                       static_cast<uint16_t*>(y), D, F, D, g, nt2);
    return check_launch("glu_gemm_bf16<down>");
  }
  using namespace f32k;
  const int64_t m_tiles = rows_bound / BM + groups + 1;
  const int nt1 = (F + BN - 1) / BN, nt2 = (D + BN - 1) / BN;
  if (m_tiles * nt1 > 0x7fffffffll || m_tiles * nt2 > 0x7fffffffll) {
    set_error("experts: grid too large");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  hipLaunchKernelGGL((glu_gemm_f32_kernel<true, BLAYOUT>), dim3((unsigned)(m_tiles * nt1)),
                     dim3(256), 0, stream, static_cast<const float*>(x), D,
                     static_cast<const float*>(w_gate), static_cast<const float*>(w_up),
                     static_cast<float*>(h), F, D, F, g, nt1);
  if (int rc = check_launch("glu_gemm_f32<gate,up>")) return rc;
  hipLaunchKernelGGL((glu_gemm_f32_kernel<false, BLAYOUT>), dim3((unsigned)(m_tiles * nt2)),
                     dim3(256), 0, stream, static_cast<const float*>(h), F,
                     static_cast<const float*>(w_down), static_cast<const float*>(nullptr),
                     static_cast<float*>(y), D, F, D, g, nt2);
  return check_launch("glu_gemm_f32<down>");
}

}  // namespace fs2moe

using namespace fs2moe;

extern "C" int fs2moe_grouped_swiglu_fuses_gather(int32_t D, int32_t F, int32_t act_dtype,
                                                  int32_t w_dtype) {
  if (D <= 0 || F <= 0) return 0;
  if (w_dtype == FS2MOE_FP8_E4M3) return (act_dtype == FS2MOE_BF16 && D % 64 == 0 && F % 64 == 0) ? 1 : 0;
  return (w_dtype == act_dtype && dma_path_applies(act_dtype, D, F)) ? 1 : 0;
}

extern "C" int fs2moe_grouped_swiglu_keeps(int32_t D, int32_t F, int64_t max_rows,
                                           int32_t act_dtype) {
  if (D <= 0 || F <= 0 || max_rows < 0) return 0;
  return (dma_path_applies(act_dtype, D, F) && dma_offsets_fit(max_rows, D, F)) ? 1 : 0;
}

extern "C" int fs2moe_grouped_swiglu_keep(const void* xe, const int32_t* row_map,
                                          const int32_t* counts, const int32_t* offsets,
                                          const void* w_gate, const void* w_up, const void* w_down,
                                          int32_t E, int32_t D, int32_t F, int64_t max_rows,
                                          int32_t act_dtype, void* g, void* u, void* h, void* ye,
                                          void* stream) {
  FS2_REQUIRE(xe && counts && offsets && w_gate && w_up && w_down && g && u && h && ye,
              "grouped_swiglu_keep: null pointer");
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS, "grouped_swiglu_keep: E=%d outside [1, %d]", E,
              FS2MOE_MAX_EXPERTS);
  FS2_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), "grouped_swiglu_keep: max_rows=%lld",
              (long long)max_rows);
  if (!fs2moe_grouped_swiglu_keeps(D, F, max_rows, act_dtype)) {
    set_error("grouped_swiglu_keep: needs bf16, D and F multiples of 64 and activation matrices "
              "below 4 GB (D=%d, F=%d, act_dtype %d, max_rows=%lld)",
              D, F, act_dtype, (long long)max_rows);
    return FS2MOE_ERR_UNSUPPORTED;
  }
  FS2_REQUIRE(aligned16(xe) && aligned16(w_gate) && aligned16(w_up) && aligned16(w_down) &&
                  aligned16(g) && aligned16(u) && aligned16(h) && aligned16(ye),
              "grouped_swiglu_keep: buffers must be 16-byte aligned");
  Groups grp{counts, offsets, E, 0};
  return launch_dma_pair<FS2MOE_W_IN_OUT>(xe, row_map, grp, max_rows, w_gate, w_up, w_down, nullptr,
                                          nullptr, nullptr, D, F, h, ye,
                                          static_cast<hipStream_t>(stream), g, u);
}

static int grouped_swiglu_impl(const void* xe, const int32_t* row_map, const int32_t* counts,
                               const int32_t* offsets, const void* w_gate, const void* w_up,
                               const void* w_down, const float* s_gate, const float* s_up,
                               const float* s_down, int32_t E, int32_t D, int32_t F,
                               int64_t max_rows, int32_t act_dtype, int32_t w_dtype, void* h,
                               void* ye, int32_t rows_hint, void* stream,
                               const float* row_w = nullptr) {
  FS2_REQUIRE(xe && counts && offsets && w_gate && w_up && w_down && h && ye,
              "grouped_swiglu: null pointer");
  FS2_REQUIRE(row_w == nullptr || w_dtype == FS2MOE_BF16,
              "grouped_swiglu: internal: row weights go with bf16 weights");
  FS2_REQUIRE(rows_hint >= 0, "grouped_swiglu: rows_per_expert=%d", rows_hint);
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS, "grouped_swiglu: E=%d outside [1, %d]", E,
              FS2MOE_MAX_EXPERTS);
  FS2_REQUIRE(D > 0 && F > 0 && D % 8 == 0 && F % 8 == 0,
              "grouped_swiglu: D=%d and F=%d must be positive multiples of 8", D, F);
  FS2_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), "grouped_swiglu: max_rows=%lld",
              (long long)max_rows);
  FS2_REQUIRE(act_dtype == FS2MOE_F32 || act_dtype == FS2MOE_BF16, "grouped_swiglu: act_dtype %d",
              act_dtype);
  FS2_REQUIRE(aligned16(xe) && aligned16(w_gate) && aligned16(w_up) && aligned16(w_down) &&
                  aligned16(h) && aligned16(ye),
              "grouped_swiglu: buffers must be 16-byte aligned");
  if (w_dtype == FS2MOE_FP8_E4M3) {
    // W8A16: e4m3 codes [E, F, D] / [E, D, F] with per-output-channel f32 scales.
    FS2_REQUIRE(act_dtype == FS2MOE_BF16, "grouped_swiglu: fp8 weights need bf16 activations");
    FS2_REQUIRE(s_gate && s_up && s_down, "grouped_swiglu: fp8 weights need scales");
    FS2_REQUIRE(D % 64 == 0 && F % 64 == 0,
                "grouped_swiglu: fp8 weights need D=%d and F=%d to be multiples of 64", D, F);
    FS2_REQUIRE(aligned16(s_gate) && aligned16(s_up) && aligned16(s_down),
                "grouped_swiglu: scales must be 16-byte aligned");
    if (max_rows == 0) return FS2MOE_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // Two regimes.  With many rows per expert the layer is a GEMM: the bf16 throughput kernel, its
    // producers turning the codes into bf16 on the way to LDS (half the weight bytes of bf16, the
    // same matrix rate).  With few (decode) it is a stream over the weights: the kernels below.  The
    // row counts live on the device, so the choice goes by the mean number of rows per expert the
    // buffers are sized for.
    // (the streaming kernels build their item table with a thread per expert: up to 256 experts)
    if ((max_rows / E >= kFp8GemmMinRowsPerExpert || E > 256) && dma_offsets_fit(max_rows, D, F)) {
      Groups g{counts, offsets, E, 0};
      return launch_dma_pair<dma::W_FP8_TILED>(xe, row_map, g, max_rows, w_gate, w_up, w_down, s_gate,
                                               s_up, s_down, D, F, h, ye, st);
    }
    FS2_REQUIRE(E <= 256, "grouped_swiglu: the e4m3 streaming kernels take up to 256 experts (E=%d)", E);
    // Persistent blocks, three or four per CU (what the kernels' registers allow), walking work
    // items.
    // A long K is split over the 4 waves of a block (the chain of dependent loads per wave sets the
    // time of an item), a short one over 2 with two sets of channel groups per block.  A wave takes
    // 2 (gate/up) or 4 (down) groups of 16 channels when K is long, half that when it is short;
    // N / 16 is a multiple of 4, so the channel blocks tile N exactly.
    const int cus = cu_count_by_xcd();
    if (cus == 0) {
      set_error("experts: cannot query the compute-unit count");
      return FS2MOE_ERR_LAUNCH;
    }
    const unsigned cu_blocks = (unsigned)cus;
    {
      // work items (16-row chunks x channel blocks of at least 32 channels) are counted in 31 bits
      const int64_t chunks = max_rows / 16 + E;
      const int64_t most_blocks = (D > F ? D : F) / 32;
      if (chunks * most_blocks > 0x7fffffffll) {
        set_error("experts: too many work items");
        return FS2MOE_ERR_UNSUPPORTED;
      }
    }
    auto launch = [&](auto dual_tag, const void* a, const int32_t* map, int lda, const void* w0,
                      const void* w1, const float* s0, const float* s1, void* c, int ldc, int kdim,
                      int n) {
      constexpr bool DUAL = decltype(dual_tag)::value;
      const uint16_t* ap = static_cast<const uint16_t*>(a);
      const uint8_t* w0p = static_cast<const uint8_t*>(w0);
      const uint8_t* w1p = static_cast<const uint8_t*>(w1);
      uint16_t* cp = static_cast<uint16_t*>(c);
      const unsigned grid = (DUAL ? 4u : 3u) * cu_blocks;  // the kernels' launch bounds
      if (kdim >= 512) {
        constexpr int CGW = DUAL ? 2 : 4;
        hipLaunchKernelGGL((glu_gemm_fp8w_kernel<DUAL, 4, CGW>), dim3(grid), dim3(256), 0, st, ap,
                           map, lda, w0p, w1p, s0, s1, cp, ldc, kdim, n, counts, offsets, E,
                           n / 16 / CGW);
      } else {
        constexpr int CGW = DUAL ? 1 : 2;
        hipLaunchKernelGGL((glu_gemm_fp8w_kernel<DUAL, 2, CGW>), dim3(grid), dim3(256), 0, st, ap,
                           map, lda, w0p, w1p, s0, s1, cp, ldc, kdim, n, counts, offsets, E,
                           n / 16 / (2 * CGW));
      }
    };
    launch(std::true_type{}, xe, row_map, D, w_gate, w_up, s_gate, s_up, h, F, D, F);
    if (int rc = check_launch("glu_gemm_fp8w<gate,up>")) return rc;
    launch(std::false_type{}, h, nullptr, F, w_down, nullptr, s_down, nullptr, ye, D, F, D);
    return check_launch("glu_gemm_fp8w<down>");
  }
  if (w_dtype != act_dtype) {
    set_error("grouped_swiglu: weight dtype %d with activation dtype %d has no kernel", w_dtype,
              act_dtype);
    return FS2MOE_ERR_UNSUPPORTED;
  }
  if (max_rows == 0) return FS2MOE_OK;
  Groups g{counts, offsets, E, 0};
  return launch_glu<FS2MOE_W_IN_OUT>(xe, row_map, g, max_rows, w_gate, w_up, w_down, D, F, act_dtype,
                                     h, ye, static_cast<hipStream_t>(stream), rows_hint, row_w);
}

bool fs2moe::swiglu_streams_rows(int32_t act_dtype, int32_t w_dtype, int32_t D, int32_t F, int32_t E,
                                 int32_t rows_per_expert) {
  if (act_dtype != FS2MOE_BF16 || w_dtype != FS2MOE_BF16 || D < 8 || F < 8 || D % 8 || F % 8) return false;
  static const int32_t some = 0;  // (the predicates only ask whether the groups have counts)
  const Groups g{&some, &some, E, 0};
  return gemv_applies(act_dtype, D, F, g, rows_per_expert) || gemv16_applies(act_dtype, D, F, g, rows_per_expert);
}

int fs2moe::grouped_swiglu_scaled_rows(const void* x, const int32_t* row_map, const float* row_w,
                                       const int32_t* counts, const int32_t* offsets,
                                       const void* w_gate, const void* w_up, const void* w_down,
                                       int32_t E, int32_t D, int32_t F, int64_t max_rows, void* h,
                                       void* ye, int32_t rows_per_expert, void* stream) {
  FS2_REQUIRE(row_map && row_w, "grouped_swiglu: null pointer");
  FS2_REQUIRE(swiglu_streams_rows(FS2MOE_BF16, FS2MOE_BF16, D, F, E, rows_per_expert),
              "grouped_swiglu: internal: D=%d F=%d E=%d with %d rows an expert do not stream", D, F, E,
              rows_per_expert);
  return grouped_swiglu_impl(x, row_map, counts, offsets, w_gate, w_up, w_down, nullptr, nullptr,
                             nullptr, E, D, F, max_rows, FS2MOE_BF16, FS2MOE_BF16, h, ye,
                             rows_per_expert, stream, row_w);
}

extern "C" int fs2moe_grouped_swiglu(const void* xe, const int32_t* row_map, const int32_t* counts,
                                     const int32_t* offsets, const void* w_gate, const void* w_up,
                                     const void* w_down, const float* s_gate, const float* s_up,
                                     const float* s_down, int32_t E, int32_t D, int32_t F,
                                     int64_t max_rows, int32_t act_dtype, int32_t w_dtype, void* h,
                                     void* ye, void* stream) {
  return grouped_swiglu_impl(xe, row_map, counts, offsets, w_gate, w_up, w_down, s_gate, s_up, s_down,
                             E, D, F, max_rows, act_dtype, w_dtype, h, ye, 0, stream);
}

extern "C" int fs2moe_grouped_swiglu_rows(const void* xe, const int32_t* row_map,
                                          const int32_t* counts, const int32_t* offsets,
                                          const void* w_gate, const void* w_up, const void* w_down,
                                          const float* s_gate, const float* s_up,
                                          const float* s_down, int32_t E, int32_t D, int32_t F,
                                          int64_t max_rows, int32_t act_dtype, int32_t w_dtype,
                                          void* h, void* ye, int32_t rows_per_expert, void* stream) {
  return grouped_swiglu_impl(xe, row_map, counts, offsets, w_gate, w_up, w_down, s_gate, s_up, s_down,
                             E, D, F, max_rows, act_dtype, w_dtype, h, ye, rows_per_expert, stream);
}

// One grouped (or dense) GEMM, C = A @ B_e, on the kernels of the SwiGLU pair's second half.
template <int BLAYOUT>
static int launch_gemm(const void* a, const int32_t* row_map, const Groups& g, int64_t rows_bound,
                       const void* b, int K, int N, int dtype, void* c, hipStream_t stream) {
  const int groups = g.counts ? g.E : 0;
  if (dtype == FS2MOE_BF16 && K % (2 * dma::BK) == 0 && dma_offsets_fit(rows_bound, K, N)) {
    using namespace dma;
    auto k = glu_gemm_bf16_dma_kernel<false, BLAYOUT>;
    static bool attr_set = false;  // benign race: setting the attribute is idempotent
    if (!attr_set) {
      hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(k),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
      if (e1 != hipSuccess) {
        set_error("gemm: cannot reserve %d bytes of LDS: %s", SMEM_BYTES, hipGetErrorString(e1));
        return FS2MOE_ERR_LAUNCH;
      }
      attr_set = true;
    }
    const int num_blocks = cu_count_by_xcd();
    if (num_blocks == 0) {
      set_error("gemm: cannot query the compute-unit count");
      return FS2MOE_ERR_LAUNCH;
    }
    const int nt = (N + 255) / 256;
    if ((rows_bound / BM + groups + 1) * nt > 0x7fffffffll) {
      set_error("gemm: too many tiles");
      return FS2MOE_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(k, dim3((unsigned)num_blocks), dim3(NWAVES * 64), SMEM_BYTES, stream,
                       static_cast<const uint16_t*>(a), row_map, K, static_cast<const uint16_t*>(b),
                       static_cast<const uint16_t*>(nullptr), static_cast<const float*>(nullptr),
                       static_cast<const float*>(nullptr), static_cast<uint16_t*>(c), N, K, N, g, nt);
    return check_launch("glu_gemm_bf16_dma<single>");
  }
  if (row_map != nullptr) {
    set_error("gemm: a row map needs bf16, K a multiple of 64 and matrices below 4 GB");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  if (dtype == FS2MOE_BF16) {
    using namespace bf16k;
    const int64_t m_tiles = rows_bound / BM + groups + 1;
    const int nt = (N + BN - 1) / BN;
    if (m_tiles * nt > 0x7fffffffll) {
      set_error("gemm: grid too large");
      return FS2MOE_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL((glu_gemm_bf16_kernel<false, BLAYOUT>), dim3((unsigned)(m_tiles * nt)),
                       dim3(256), 0, stream, static_cast<const uint16_t*>(a), K,
                       static_cast<const uint16_t*>(b), static_cast<const uint16_t*>(nullptr),
                       static_cast<uint16_t*>(c), N, K, N, g, nt);
    return check_launch("glu_gemm_bf16<single>");
  }
  using namespace f32k;
  const int64_t m_tiles = rows_bound / BM + groups + 1;
  const int nt = (N + BN - 1) / BN;
  if (m_tiles * nt > 0x7fffffffll) {
    set_error("gemm: grid too large");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  hipLaunchKernelGGL((glu_gemm_f32_kernel<false, BLAYOUT>), dim3((unsigned)(m_tiles * nt)), dim3(256),
                     0, stream, static_cast<const float*>(a), K, static_cast<const float*>(b),
                     static_cast<const float*>(nullptr), static_cast<float*>(c), N, K, N, g, nt);
  return check_launch("glu_gemm_f32<single>");
}

extern "C" int fs2moe_grouped_gemm(const void* a, const int32_t* row_map, const int32_t* counts,
                                   const int32_t* offsets, const void* b, int32_t b_layout,
                                   int32_t E, int32_t K, int32_t N, int64_t max_rows, int32_t dtype,
                                   void* c, void* stream) {
  FS2_REQUIRE(a && b && c, "grouped_gemm: null pointer");
  FS2_REQUIRE((counts == nullptr) == (offsets == nullptr), "grouped_gemm: counts without offsets");
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS && (counts != nullptr || E == 1),
              "grouped_gemm: E=%d", E);
  FS2_REQUIRE(b_layout == FS2MOE_W_IN_OUT || b_layout == FS2MOE_W_OUT_IN, "grouped_gemm: layout %d",
              b_layout);
  FS2_REQUIRE(dtype == FS2MOE_F32 || dtype == FS2MOE_BF16, "grouped_gemm: dtype %d", dtype);
  FS2_REQUIRE(K > 0 && N > 0 && K % 8 == 0 && N % 8 == 0,
              "grouped_gemm: K=%d and N=%d must be positive multiples of 8", K, N);
  FS2_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), "grouped_gemm: max_rows=%lld",
              (long long)max_rows);
  FS2_REQUIRE(aligned16(a) && aligned16(b) && aligned16(c),
              "grouped_gemm: buffers must be 16-byte aligned");
  if (max_rows == 0) return FS2MOE_OK;
  Groups g{counts, offsets, E, (int)max_rows};
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (b_layout == FS2MOE_W_IN_OUT)
    return launch_gemm<FS2MOE_W_IN_OUT>(a, row_map, g, max_rows, b, K, N, dtype, c, st);
  return launch_gemm<FS2MOE_W_OUT_IN>(a, row_map, g, max_rows, b, K, N, dtype, c, st);
}

extern "C" int fs2moe_dense_swiglu_keep(const void* x, const void* w_gate, const void* w_up,
                                        const void* w_down, int32_t T, int32_t D, int32_t F,
                                        int32_t act_dtype, void* g, void* u, void* h, void* y,
                                        void* stream) {
  FS2_REQUIRE(x && w_gate && w_up && w_down && g && u && h && y, "dense_swiglu_keep: null pointer");
  FS2_REQUIRE(T >= 0, "dense_swiglu_keep: T=%d", T);
  if (!fs2moe_grouped_swiglu_keeps(D, F, T, act_dtype)) {
    set_error("dense_swiglu_keep: needs bf16, D and F multiples of 64 and activation matrices "
              "below 4 GB (D=%d, F=%d, act_dtype %d, T=%d)", D, F, act_dtype, T);
    return FS2MOE_ERR_UNSUPPORTED;
  }
  FS2_REQUIRE(aligned16(x) && aligned16(w_gate) && aligned16(w_up) && aligned16(w_down) &&
                  aligned16(g) && aligned16(u) && aligned16(h) && aligned16(y),
              "dense_swiglu_keep: buffers must be 16-byte aligned");
  if (T == 0) return FS2MOE_OK;
  Groups grp{nullptr, nullptr, 1, T};
  return launch_dma_pair<FS2MOE_W_OUT_IN>(x, nullptr, grp, T, w_gate, w_up, w_down, nullptr,
                                          nullptr, nullptr, D, F, h, y,
                                          static_cast<hipStream_t>(stream), g, u);
}

extern "C" int fs2moe_grouped_gemm_sum_supported(int32_t K, int32_t N, int64_t max_rows,
                                                 int32_t dtype) {
  if (K <= 0 || N <= 0 || max_rows < 0 || N % 8 != 0) return 0;
  return (dtype == FS2MOE_BF16 && K % (2 * dma::BK) == 0 && dma_offsets_fit(max_rows, K, N)) ? 1 : 0;
}

extern "C" int fs2moe_grouped_gemm_sum(const void* a1, const void* b1, const void* a2,
                                       const void* b2, const int32_t* counts,
                                       const int32_t* offsets, int32_t E, int32_t K, int32_t N,
                                       int64_t max_rows, int32_t dtype, void* c, void* stream) {
  FS2_REQUIRE(a1 && b1 && a2 && b2 && c, "grouped_gemm_sum: null pointer");
  FS2_REQUIRE((counts == nullptr) == (offsets == nullptr),
              "grouped_gemm_sum: counts without offsets");
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS && (counts != nullptr || E == 1),
              "grouped_gemm_sum: E=%d", E);
  FS2_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), "grouped_gemm_sum: max_rows=%lld",
              (long long)max_rows);
  if (!fs2moe_grouped_gemm_sum_supported(K, N, max_rows, dtype)) {
    set_error("grouped_gemm_sum: needs bf16, K a multiple of 64, N a multiple of 8 and matrices "
              "below 4 GB (K=%d, N=%d, dtype %d, max_rows=%lld)",
              K, N, dtype, (long long)max_rows);
    return FS2MOE_ERR_UNSUPPORTED;
  }
  FS2_REQUIRE(aligned16(a1) && aligned16(b1) && aligned16(a2) && aligned16(b2) && aligned16(c),
              "grouped_gemm_sum: buffers must be 16-byte aligned");
  if (max_rows == 0) return FS2MOE_OK;
  using namespace dma;
  Groups g{counts, offsets, E, (int)max_rows};
  auto k = glu_gemm_bf16_dma_kernel<false, FS2MOE_W_OUT_IN, false, true>;
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void*>(k),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
    if (e1 != hipSuccess) {
      set_error("grouped_gemm_sum: cannot reserve %d bytes of LDS: %s", SMEM_BYTES,
                hipGetErrorString(e1));
      return FS2MOE_ERR_LAUNCH;
    }
    attr_set = true;
  }
  const int num_blocks = cu_count_by_xcd();
  if (num_blocks == 0) {
    set_error("grouped_gemm_sum: cannot query the compute-unit count");
    return FS2MOE_ERR_LAUNCH;
  }
  const int groups = counts ? E : 0;
  const int nt = (N + 255) / 256;
  if ((max_rows / BM + groups + 1) * nt > 0x7fffffffll) {
    set_error("grouped_gemm_sum: too many tiles");
    return FS2MOE_ERR_UNSUPPORTED;
  }
  // (the second activation matrix travels in the first scale argument, the second weights in B1)
  hipLaunchKernelGGL(k, dim3((unsigned)num_blocks), dim3(NWAVES * 64), SMEM_BYTES,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(a1),
                     static_cast<const int32_t*>(nullptr), K, static_cast<const uint16_t*>(b1),
                     static_cast<const uint16_t*>(b2), static_cast<const float*>(a2),
                     static_cast<const float*>(nullptr), static_cast<uint16_t*>(c), N, K, N, g, nt);
  return check_launch("glu_gemm_bf16_dma<two sources>");
}

extern "C" int fs2moe_dense_swiglu(const void* x, const void* w_gate, const void* w_up,
                                   const void* w_down, int32_t T, int32_t D, int32_t F,
                                   int32_t act_dtype, void* h, void* y, void* stream) {
  FS2_REQUIRE(x && w_gate && w_up && w_down && h && y, "dense_swiglu: null pointer");
  FS2_REQUIRE(T >= 0 && D > 0 && F > 0 && D % 8 == 0 && F % 8 == 0,
              "dense_swiglu: T=%d, D=%d, F=%d (D and F must be positive multiples of 8)", T, D, F);
  FS2_REQUIRE(act_dtype == FS2MOE_F32 || act_dtype == FS2MOE_BF16, "dense_swiglu: act_dtype %d",
              act_dtype);
  FS2_REQUIRE(aligned16(x) && aligned16(w_gate) && aligned16(w_up) && aligned16(w_down) &&
                  aligned16(h) && aligned16(y),
              "dense_swiglu: buffers must be 16-byte aligned");
  if (T == 0) return FS2MOE_OK;
  Groups g{nullptr, nullptr, 1, T};
  return launch_glu<FS2MOE_W_OUT_IN>(x, nullptr, g, T, w_gate, w_up, w_down, D, F, act_dtype, h, y,
                                     static_cast<hipStream_t>(stream));
}

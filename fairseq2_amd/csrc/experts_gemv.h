// Grouped SwiGLU products for a handful of rows per expert, bf16 weights in the reference layout.
//
// A decode step of one to eight sequences gives every active expert at most that many rows: the
// layer is then a stream over the active experts' weights, each weight used once per row.  The
// throughput kernel handles such an expert as a tile of 256 channels walked through all of K by one
// block, i.e. a chain of K / 64 round trips on one CU with the matrix pipe all but idle (8 experts x
// 6 tiles keep 48 of 256 CUs busy for 32 us).  Here the weights never pass through LDS or the matrix
// pipe: a lane loads 16 bytes (8 channels of one k row, as they lie in memory, (K, N) with N
// contiguous), multiplies them with that k's activation of each row on the vector ALUs and keeps
// R x 8 sums (twice that for the fused gate/up product).  A block owns 64 channels of one expert:
// its eight waves split K, a wave's eight lane groups split it again (a load instruction covers
// 8 lane groups x 4 k rows of 128 contiguous bytes), and the partial sums are added in a fixed
// order: lane groups by exchange within the wave, waves through LDS.  The expert's rows sit in LDS
// as they lie in memory; a lane reads the 4 k it needs of each row with one 8-byte read.
//
// R (1, 2 or 4) is the most rows of one expert taken per pass: a template parameter that bounds the
// registers (rows an expert does not have are skipped); an expert with more rows than R is walked
// again for every further R rows (correct for any count, meant for counts up to R).  From 5 rows per
// expert on the arithmetic no longer hides behind the stream and the GEMM tiles are faster.
#pragma once

#include "common.h"

namespace fs2moe {
namespace gemv {
constexpr int COLS = 64;          // channels per block
// waves per block: a block is a short chain of round trips to memory, so K is split over eight
// waves (with four, one token took 47 instead of 44 us and four tokens 71 instead of 61)
constexpr int waves(int R) { return 8; }
constexpr int threads(int R) { return 64 * waves(R); }
constexpr int MAX_LDS_BYTES = 144 * 1024;  // (160 KB less the kernel's own partial sums, 16 KB at most)
inline bool fits(int K, int R) { return (int64_t)K * R * 2 <= MAX_LDS_BYTES; }
// Steps of K (256 rows a block) whose loads a wave issues before it multiplies any: 4 with one or
// two rows, 2 with four (registers).  DEEP: 8, for the single product with one or two rows over a
// long K, where a block is a chain of K / 256 / U round trips (Mixtral's down projection, K 14336:
// the layer at one token 225 -> 178 us, at two 286 -> 251; a short K would only issue loads that it
// then masks: Qwen3's K of 768 is three steps, and two tokens took 54 instead of 48 us with 8).
// The sums do not depend on it: a lane adds its products in the same order.
constexpr int steps_in_flight(bool dual, int R, bool deep) { return R > 2 ? 2 : (deep && !dual) ? 8 : 4; }
inline bool deep_applies(int K, int R) { return R <= 2 && K >= 4096; }
}  // namespace gemv

// The n-th expert that has rows, -1 when there are fewer (wave-uniform; every wave works it out for
// itself from the counts, without LDS or a barrier: E <= 256 is four ballots).  A block takes the
// blockIdx.y-th such expert instead of expert blockIdx.y: blocks of experts without rows would end at
// once wherever they are, but numbered this way the blocks that work are contiguous in launch order
// whatever the experts' numbers, and consecutive blocks go to consecutive XCDs.  With the real routing
// of 12 tokens (24 experts active, scattered over 128) the blocks of the block-per-CU kernel below
// crowded on some XCDs and its pair of launches took 73 instead of 54 us.
__device__ __forceinline__ int nth_active_expert(const int32_t* __restrict__ counts, int E, int n) {
  const int lane = threadIdx.x & 63;
  int c[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = lane + 64 * j;
    c[j] = counts[i < E ? i : 0];
  }
  int e = -1, seen = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const unsigned long long act = __ballot(lane + 64 * j < E && c[j] > 0);
    const int before = __popcll(act & ((1ull << lane) - 1ull));
    const unsigned long long hit = __ballot(((act >> lane) & 1ull) != 0ull && seen + before == n);
    if (e < 0 && hit != 0ull) e = 64 * j + (int)__builtin_ctzll(hit);
    seen += __popcll(act);
  }
  return e;
}

// DUAL: C[r, n] = SiLU(A[r] . B0[:, n]) * (A[r] . B1[:, n]); else C[r, n] = A[r] . B0[:, n].
// A rows are read through row_map when it is given (row r of the expert is A[row_map[offset + r]]),
// and multiplied by row_w[offset + r] on the way into LDS when that is given (rounded to bf16: the
// bits dispatch's scaled row copy would have held).
// grid: (ceil(N / 64), E).  K a multiple of 4, N a multiple of 8.
template <bool DUAL, int R, bool DEEP = false>
__global__ __launch_bounds__(gemv::threads(R)) void glu_gemv_bf16_kernel(
    const uint16_t* __restrict__ A, const int32_t* __restrict__ row_map,
    const float* __restrict__ row_w, int lda,
    const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1, uint16_t* __restrict__ C,
    int ldc, int K, int N, const int32_t* __restrict__ counts,
    const int32_t* __restrict__ offsets) {
  using namespace gemv;
  constexpr int M = DUAL ? 2 : 1;
  constexpr int NW = waves(R), THREADS = threads(R);
  constexpr int KSTEP = NW * 32;  // k rows per block and step: NW waves x 8 lane groups x 4
  extern __shared__ __attribute__((aligned(16))) uint8_t gemv_smem[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(gemv_smem);  // [R][K]
  __shared__ float red[NW][M][R][COLS];

  const int e = blockIdx.y;
  const int cnt = counts[e];
  if (cnt == 0) return;
  const int off = offsets[e];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ks = lane >> 3, cc = lane & 7;
  const int col = blockIdx.x * COLS + cc * 8;
  const bool col_ok = col < N;  // N is a multiple of 8: the lane's eight channels are in or out together
  const size_t wbase = (size_t)e * K * N + (col_ok ? col : 0);
  const uint16_t* w0 = B0 + wbase;
  const uint16_t* w1 = DUAL ? B1 + wbase : w0;

  for (int r0 = 0; r0 < cnt; r0 += R) {
    // ---- the pass's rows -> LDS (rows past the expert's count as zeros) ---------------------------
    if (r0 > 0) __syncthreads();  // the previous pass's reads of xs and red are over
    const int kchunks = K / 4;    // 8-byte pieces per row
    for (int i = tid; i < R * kchunks; i += THREADS) {
      const int r = i / kchunks, c = i - r * kchunks;
      u32x2 v = {0u, 0u};
      if (r0 + r < cnt) {
        const int row = off + r0 + r;
        const size_t src = (size_t)(row_map != nullptr ? row_map[row] : row) * lda;
        v = *reinterpret_cast<const u32x2*>(A + src + 4 * c);
        if (row_w != nullptr) {
          const float w = row_w[row];
          v = u32x2{scale_bf16x2(v[0], w), scale_bf16x2(v[1], w)};
        }
      }
      *reinterpret_cast<u32x2*>(xs + (size_t)r * K + 4 * c) = v;
    }
    __syncthreads();

    // ---- the stream over K --------------------------------------------------------------------------
    // (rows the expert does not have are skipped, block-uniformly: R only bounds the registers)
    const int rcnt = __builtin_amdgcn_readfirstlane(cnt - r0 < R ? cnt - r0 : R);
    float acc[M][R][8];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int c = 0; c < 8; ++c) acc[m][r][c] = 0.f;
    // U steps of K per iteration, all their loads issued before any arithmetic: a step is one round
    // trip to memory and little else, so the steps' round trips overlap
    constexpr int U = gemv::steps_in_flight(DUAL, R, DEEP);
    for (int kb0 = 0; kb0 < K; kb0 += U * KSTEP) {
      u32x4 wvu[U][M][4];
#pragma unroll
      for (int uu = 0; uu < U; ++uu) {
        const int k0 = kb0 + uu * KSTEP + wave * 32 + ks * 4;
        const int kk = k0 < K ? k0 : 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          wvu[uu][0][j] = *reinterpret_cast<const u32x4*>(w0 + (size_t)(kk + j) * N);
          if (DUAL) wvu[uu][M - 1][j] = *reinterpret_cast<const u32x4*>(w1 + (size_t)(kk + j) * N);
        }
      }
      // (without the fence the compiler moves every load down to its first use and waits for each
      // one there: one round trip per load instead of one per iteration)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int uu = 0; uu < U; ++uu) {
      const int k0 = kb0 + uu * KSTEP + wave * 32 + ks * 4;
      const bool k_ok = k0 < K;  // K is a multiple of 4: the lane's four rows are in or out together
      const int kk = k_ok ? k0 : 0;
      const u32x4 (&wv)[M][4] = wvu[uu];
      float xv[R][4];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (r < rcnt) {
          const u32x2 q = *reinterpret_cast<const u32x2*>(xs + (size_t)r * K + kk);
          xv[r][0] = k_ok ? __uint_as_float(q[0] << 16) : 0.f;
          xv[r][1] = k_ok ? __uint_as_float(q[0] & 0xffff0000u) : 0.f;
          xv[r][2] = k_ok ? __uint_as_float(q[1] << 16) : 0.f;
          xv[r][3] = k_ok ? __uint_as_float(q[1] & 0xffff0000u) : 0.f;
        }
      }
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float wf[8];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            wf[2 * c] = __uint_as_float(wv[m][j][c] << 16);
            wf[2 * c + 1] = __uint_as_float(wv[m][j][c] & 0xffff0000u);
          }
#pragma unroll
          for (int r = 0; r < R; ++r) {
            if (r < rcnt) {
#pragma unroll
              for (int c = 0; c < 8; ++c) acc[m][r][c] += xv[r][j] * wf[c];
            }
          }
        }
      }
    }

    // ---- lane groups (fixed order: exchange distances 8, 16, 32), then waves through LDS ------------
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (r < rcnt) {
#pragma unroll
          for (int c = 0; c < 8; ++c) {
            float v = acc[m][r][c];
            v += __shfl_xor(v, 8, kWave);
            v += __shfl_xor(v, 16, kWave);
            v += __shfl_xor(v, 32, kWave);
            acc[m][r][c] = v;
          }
        }
      }
    if (ks == 0) {
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int c = 0; c < 8; ++c) red[wave][m][r][cc * 8 + c] = acc[m][r][c];
    }
    __syncthreads();
    for (int i = tid; i < R * COLS; i += THREADS) {
      const int r = i / COLS, c = i - r * COLS;
      const int n = blockIdx.x * COLS + c;
      if (r0 + r >= cnt || n >= N) continue;
      float g = 0.f, u = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        g += red[w][0][r][c];
        if (DUAL) u += red[w][M - 1][r][c];
      }
      if (DUAL) g = silu_f32(g) * u;
      C[(size_t)(off + r0 + r) * ldc + n] = f32_to_bf16_bits(g);
    }
  }
}


// ---------------------------------------------------------------------------------------------------
// The same stream for 5 to 16 rows per expert, with the arithmetic on the matrix pipe and still no
// LDS transposition of the weights.  v_mfma_f32_16x16x32_bf16 wants, per lane, eight k of ONE
// channel; a lane's 16-byte load holds eight channels of ONE k.  But the 32 k slots of the
// instruction are just 32 products summed per (channel, row) pair: which k sits in which slot is
// free as long as both operands agree.  So a lane (c16 = l % 16, g = l / 16) loads its eight
// channels 8 c16 .. 8 c16 + 7 at eight k rows (two steps of four consecutive rows), and one byte
// permute per pair of rows turns that 8 x 8 block of its OWN registers into eight operands, one per
// channel, each holding the lane's eight k in its eight slots.  MFMA number c of a step then multiplies
// channels {8 r + c : r = 0..15} (one per lane of a group) with up to 16 rows of the expert over
// 4 groups x 8 k, and the lane (row m = l % 16, q = l / 16) ends up with channels 8 (4 q + i) + c,
// i = 0..3.  The rows' operand is what lies in LDS: the 2 x 4 consecutive k of row m.
//
// A block owns 128 channels of one expert; its eight waves split K (a step of the block is 128 k
// rows) and their partial sums meet in LDS in a fixed order ((0+4)+(2+6))+((1+5)+(3+7)).  XR (8 or
// 16) is how many rows are staged in LDS: a pass takes up to XR rows, an expert with more is walked
// again.  Rows lie K + 4 elements apart so that the sixteen rows' reads fall into different banks.
namespace gemv16 {
constexpr int COLS = 128;     // channels per block: 16 lanes x 8
constexpr int WAVES = 8, THREADS = WAVES * 64;
constexpr int KSTEP = WAVES * 16;  // k rows per step of the block: waves x 4 lane groups x 4
constexpr int MAX_LDS_BYTES = 160 * 1024;
__host__ __device__ inline int stride(int K) { return K + 4; }
inline size_t lds_bytes(int K, int XR, bool dual) {
  const size_t xs = ((size_t)XR * stride(K) + 4) * 2;
  const size_t red = (size_t)4 * (dual ? 2 : 1) * 32 * 64 * 4;
  return xs > red ? xs : red;
}
inline bool fits(int K, int XR) { return lds_bytes(K, XR, true) <= (size_t)MAX_LDS_BYTES; }
// (one expert's matrix is addressed with 32-bit byte offsets)
inline bool offsets_fit(int D, int F) { return (int64_t)D * F * 2 <= 0xffffffffll; }
}  // namespace gemv16

// Arguments as glu_gemv_bf16_kernel.  grid: (ceil(N / 128), E).  K and N multiples of 8.
// (The second launch bound is waves per SIMD: the single product is held to 128 registers so that
// two blocks share a CU -- the down projection of 20 active experts is 320 blocks, which at one block
// per CU ran as a full round and a quarter-full one: 4 us of 75 at 8 tokens.)
template <bool DUAL, int XR>
__global__ __launch_bounds__(gemv16::THREADS, DUAL ? 2 : 4) void glu_gemv16_bf16_kernel(
    const uint16_t* __restrict__ A, const int32_t* __restrict__ row_map,
    const float* __restrict__ row_w, int lda,
    const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1, uint16_t* __restrict__ C,
    int ldc, int K, int N, const int32_t* __restrict__ counts,
    const int32_t* __restrict__ offsets) {
  using namespace gemv16;
  constexpr int M = DUAL ? 2 : 1;
  constexpr int PAIRS = DUAL ? 1 : 2;  // pairs of steps per iteration: 16 loads in flight per lane
  extern __shared__ __attribute__((aligned(16))) uint8_t gemv16_smem[];
  uint16_t* xs = reinterpret_cast<uint16_t*>(gemv16_smem);  // [XR][K + 4], then 4 zeros
  float* red = reinterpret_cast<float*>(gemv16_smem);       // [4][M][32][64], after the stream

  const int e = nth_active_expert(counts, (int)gridDim.y, (int)blockIdx.y);
  if (e < 0) return;
  const int cnt = counts[e];
  const int off = offsets[e];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, g = lane >> 4;
  const int ldx = stride(K);
  const int col = blockIdx.x * COLS + c16 * 8;
  const bool col_ok = col < N;  // N is a multiple of 8: the lane's eight channels are in or out together
  // the expert's matrices as uniform bases, a lane's place in them as a 32-bit byte offset (one
  // register per address, shared by gate and up)
  const uint8_t* w0 = reinterpret_cast<const uint8_t*>(B0 + (size_t)e * K * N);
  const uint8_t* w1 = DUAL ? reinterpret_cast<const uint8_t*>(B1 + (size_t)e * K * N) : w0;
  const uint32_t lane_col = (uint32_t)(col_ok ? col : 0);
  const uint16_t* xzero = xs + (size_t)XR * ldx;
  const uint16_t* xrow = xs + (size_t)c16 * ldx;  // row m = c16 of the pass, if it is staged
  const bool row_ok = c16 < XR;

  for (int r0 = 0; r0 < cnt; r0 += XR) {
    // ---- the pass's rows -> LDS (rows past the expert's count as zeros) ---------------------------
    if (r0 > 0) __syncthreads();  // the previous pass's sums have left LDS
    // (a row per group of threads, so that the row's place is looked up once and a thread's loads
    // are all in flight together; K is a multiple of 8 here: 16-byte pieces)
    {
      constexpr int TPR = THREADS / XR, INFLIGHT = 4;
      const int r = tid / TPR, c0 = tid - r * TPR;
      const int kchunks = K / 8;
      const bool has = r0 + r < cnt;
      size_t src = 0;
      float w = 1.f;
      if (has) {
        const int row = off + r0 + r;
        src = (size_t)(row_map != nullptr ? row_map[row] : row) * lda;
        if (row_w != nullptr) w = row_w[row];
      }
      for (int cb = c0; cb < kchunks; cb += TPR * INFLIGHT) {
        u32x4 v[INFLIGHT];
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u) {
          const int c = cb + u * TPR;
          v[u] = *reinterpret_cast<const u32x4*>(A + src + 8 * (c < kchunks ? c : 0));
        }
#pragma unroll
        for (int u = 0; u < INFLIGHT; ++u) {
          const int c = cb + u * TPR;
          if (c >= kchunks) continue;
          if (!has) v[u] = u32x4{0u, 0u, 0u, 0u};
          if (row_w != nullptr)  // (block-uniform; as dispatch's scaled copy rounds)
            v[u] = u32x4{scale_bf16x2(v[u][0], w), scale_bf16x2(v[u][1], w), scale_bf16x2(v[u][2], w),
                         scale_bf16x2(v[u][3], w)};
          u32x2* dst = reinterpret_cast<u32x2*>(xs + (size_t)r * ldx + 8 * c);  // 8-byte aligned
          dst[0] = u32x2{v[u][0], v[u][1]};
          dst[1] = u32x2{v[u][2], v[u][3]};
        }
      }
    }
    if (tid < 4) xs[(size_t)XR * ldx + tid] = 0;
    __syncthreads();

    // ---- the stream over K --------------------------------------------------------------------------
    f32x4 acc[M][8];
#pragma unroll
    for (int m = 0; m < M; ++m)
#pragma unroll
      for (int c = 0; c < 8; ++c) acc[m][c] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int kb0 = 0; kb0 < K; kb0 += 2 * PAIRS * KSTEP) {
      u32x4 wq[2 * PAIRS][M][4];
      u32x2 xq[2 * PAIRS];
#pragma unroll
      for (int s = 0; s < 2 * PAIRS; ++s) {
        const int k0 = kb0 + s * KSTEP + wave * 16 + g * 4;
        const bool k_ok = k0 < K;  // K is a multiple of 4: the lane's four rows are in or out together
        const int kk = k_ok ? k0 : 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t at = ((uint32_t)(kk + j) * (uint32_t)N + lane_col) * 2u;
          wq[s][0][j] = *reinterpret_cast<const u32x4*>(w0 + at);
          if (DUAL) wq[s][M - 1][j] = *reinterpret_cast<const u32x4*>(w1 + at);
        }
        // (k rows past K meet zeros: chosen by address, a select on the value would become a branch)
        xq[s] = *reinterpret_cast<const u32x2*>(k_ok && row_ok ? xrow + k0 : xzero);
      }
      // (without the fence the compiler moves every load down to its first use and waits for each
      // one there: one round trip per load instead of one per iteration)
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int p = 0; p < PAIRS; ++p) {
        const u32x4 xo = {xq[2 * p][0], xq[2 * p][1], xq[2 * p + 1][0], xq[2 * p + 1][1]};
        const bf16x8 xop = __builtin_bit_cast(bf16x8, xo);
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int c = 0; c < 8; ++c) {
            // channel c of the lane: the low (c even) or high (c odd) half of dword c / 2 of each row
            const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
            const u32x4(&a)[4] = wq[2 * p][m];
            const u32x4(&b)[4] = wq[2 * p + 1][m];
            const u32x4 wo = {__builtin_amdgcn_perm(a[1][c >> 1], a[0][c >> 1], sel),
                              __builtin_amdgcn_perm(a[3][c >> 1], a[2][c >> 1], sel),
                              __builtin_amdgcn_perm(b[1][c >> 1], b[0][c >> 1], sel),
                              __builtin_amdgcn_perm(b[3][c >> 1], b[2][c >> 1], sel)};
            acc[m][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wo), xop,
                                                                 acc[m][c], 0, 0, 0);
            // (operands are formed four channels ahead at most: formed all at once they cost 64
            // registers and the kernel spills)
            if ((c & 3) == 3) __builtin_amdgcn_sched_barrier(0);
          }
      }
    }

    // ---- the waves' sums meet in LDS: (w + 4) onto w, then (w + 2) onto w, then 1 onto 0 ------------
    __syncthreads();  // every wave is done reading the rows: the sums take their place
#pragma unroll
    for (int half = 4; half >= 1; half >>= 1) {
      // (one address register per wave and constant offsets from it)
      if (wave >= half && wave < 2 * half) {
        float* rp = red + (wave - half) * (M * 32 * 64) + lane;
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) rp[(m * 32 + c * 4 + i) * 64] = acc[m][c][i];
      }
      __syncthreads();
      if (wave < half) {
        const float* rp = red + wave * (M * 32 * 64) + lane;
#pragma unroll
        for (int m = 0; m < M; ++m)
#pragma unroll
          for (int c = 0; c < 8; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[m][c][i] += rp[(m * 32 + c * 4 + i) * 64];
      }
      if (half > 1) __syncthreads();
    }
    // ---- wave 0: row m = l % 16, channels 8 (4 q + i) + c ---------------------------------------------
    if (wave == 0 && row_ok && r0 + c16 < cnt) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = blockIdx.x * COLS + (4 * g + i) * 8;
        if (n >= N) continue;
        u32x4 o;
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          float v0 = acc[0][2 * h][i], v1 = acc[0][2 * h + 1][i];
          if (DUAL) {
            v0 = silu_f32(v0) * acc[M - 1][2 * h][i];
            v1 = silu_f32(v1) * acc[M - 1][2 * h + 1][i];
          }
          o[h] = (uint32_t)f32_to_bf16_bits(v0) | ((uint32_t)f32_to_bf16_bits(v1) << 16);
        }
        *reinterpret_cast<u32x4*>(C + (size_t)(off + r0 + c16) * ldc + n) = o;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// The shared expert (a dense SwiGLU, weights as nn.Linear holds them: (N, K) with K contiguous) for
// up to 16 rows: at a decode step its three matrices are streamed once like an expert's, and the
// GEMM tiles make that a chain of K / 64 round trips per tile (Llama-4 Scout, one token: 172 us for
// 252 MB).  Here 16 bytes of a weight row ARE eight k of one channel, which is what
// v_mfma_f32_16x16x32_bf16 takes from lane (n = l % 16, g = l / 16) as it stands; the matching lane
// (m = l % 16, g) loads the same eight k of row m straight from memory (the rows stay in L2; a row
// the call does not have repeats the last one, its results are not stored).  A block owns 16
// channels, its eight waves split K in steps of 32 and add their sums in LDS in ascending order.
namespace dgemv {
constexpr int WAVES = 8, THREADS = WAVES * 64;
constexpr int U = 8;  // steps of 32 k a wave has in flight
constexpr int MAX_ROWS = 16;
}  // namespace dgemv

// DUAL: C[r, n] = SiLU(A[r] . B0[n]) * (A[r] . B1[n]); else C[r, n] = A[r] . B0[n].
// A [T][lda], B0/B1 [N][K], C [T][ldc]; T <= 16; K and N multiples of 8.  grid: ceil(N / 16).
template <bool DUAL>
__global__ __launch_bounds__(dgemv::THREADS) void dense_gemv_bf16_kernel(
    const uint16_t* __restrict__ A, int lda, const uint16_t* __restrict__ B0,
    const uint16_t* __restrict__ B1, uint16_t* __restrict__ C, int ldc, int K, int N, int T) {
  using namespace dgemv;
  constexpr int M = DUAL ? 2 : 1;
  __shared__ f32x4 red[WAVES][M][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n = n0 + r16 < N ? n0 + r16 : N - 1;  // a channel past N repeats the last one: not stored
  const int row = r16 < T ? r16 : T - 1;
  const uint16_t* w0 = B0 + (size_t)n * K;
  const uint16_t* w1 = DUAL ? B1 + (size_t)n * K : w0;
  const uint16_t* xr = A + (size_t)row * lda;
  f32x4 acc[M];
#pragma unroll
  for (int m = 0; m < M; ++m) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};
  // step s of the block is the 32 k from 32 s; wave w takes the steps w, w + 8, ..
  for (int s0 = wave; s0 * 32 < K; s0 += WAVES * U) {
    u32x4 wq[U][M], xq[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (s0 + u * WAVES) * 32 + g * 8;
      const int kk = k < K ? k : 0;  // K is a multiple of 8: the lane's eight k are in or out together
      wq[u][0] = *reinterpret_cast<const u32x4*>(w0 + kk);
      if (DUAL) wq[u][M - 1] = *reinterpret_cast<const u32x4*>(w1 + kk);
      xq[u] = *reinterpret_cast<const u32x4*>(xr + kk);
    }
    // (all the loads are issued before the first is waited for)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (s0 + u * WAVES) * 32 + g * 8;
      u32x4 xv = xq[u];
      if (k >= K) xv = u32x4{0u, 0u, 0u, 0u};
      const bf16x8 xop = __builtin_bit_cast(bf16x8, xv);
#pragma unroll
      for (int m = 0; m < M; ++m)
        acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wq[u][m]), xop,
                                                         acc[m], 0, 0, 0);
    }
  }
#pragma unroll
  for (int m = 0; m < M; ++m) red[wave][m][lane] = acc[m];
  __syncthreads();
  if (wave != 0) return;
  // lane (row m = l % 16, q = l / 16) holds channels n0 + 4 q + i, i = 0..3
  f32x4 sum[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    sum[m] = red[0][m][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum[m] += red[w][m][lane];
  }
  const int nc = n0 + 4 * g;
  if (r16 < T && nc < N) {  // N is a multiple of 8: four channels are in or out together
    float v[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = DUAL ? silu_f32(sum[0][i]) * sum[M - 1][i] : sum[0][i];
    u32x2 o = {(uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16),
               (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16)};
    *reinterpret_cast<u32x2*>(C + (size_t)r16 * ldc + nc) = o;
  }
}

}  // namespace fs2moe

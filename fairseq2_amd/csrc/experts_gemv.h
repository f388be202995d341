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
constexpr int MAX_LDS_BYTES = 65536;
inline bool fits(int K, int R) { return (int64_t)K * R * 2 <= MAX_LDS_BYTES; }
}  // namespace gemv

// DUAL: C[r, n] = SiLU(A[r] . B0[:, n]) * (A[r] . B1[:, n]); else C[r, n] = A[r] . B0[:, n].
// A rows are read through row_map when it is given (row r of the expert is A[row_map[offset + r]]).
// grid: (ceil(N / 64), E).  K a multiple of 4, N a multiple of 8.
template <bool DUAL, int R>
__global__ __launch_bounds__(gemv::threads(R)) void glu_gemv_bf16_kernel(
    const uint16_t* __restrict__ A, const int32_t* __restrict__ row_map, int lda,
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
    constexpr int U = R <= 2 ? 4 : 2;
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

}  // namespace fs2moe

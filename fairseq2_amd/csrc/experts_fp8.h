// Grouped SwiGLU GEMMs with fp8 (OCP e4m3) weights and bf16 activations (W8A16).
//
// Built for the decode regime: a few rows per expert, so the layer is a stream over the active
// experts' weights and the bound is HBM.  Weights are quantised per output channel and stored in
// 1 KB tiles of 16 output channels x 64 in-features, [expert][channel / 16][feature / 64][16][64]:
// a wave's load instruction reads one whole tile and a wave's stream for 16 channels over its part
// of K is one contiguous byte range, which is what HBM likes best.
//
// Work items.  An item is (expert, block of 16 * CGW * (4 / KS) channels, chunk of 16 rows); experts
// without rows have no items.  Every block builds the same item table from the counts (one prefix
// sum) and walks the items blockIdx, blockIdx + gridDim, ..: the grid is sized to the GPU (three
// blocks per CU), not to E, so nothing is spent on starting blocks for the idle experts of a
// decode batch, and an expert with many rows is spread over as many blocks as it has chunks
// instead of being one long chain of dependent loads.  The chunks of one (expert, channel block)
// are items 8 apart, which run at the same time on the same XCD (block b runs on XCD b % 8): its L2
// fetches their common weights once.
//
// Inside an item.  A set of KS waves owns CGW groups of 16 output channels (gate and the same up
// channels for the fused gate/up GEMM); the waves split K into KS parts and add their partial sums in
// LDS in a fixed order; a block holds 4 / KS such sets.  (With a wave per 16 channels and all of K, a
// wave is a chain of K / 256 dependent memory latencies, and that chain, not bandwidth, set the
// kernel time.)  A wave walks its part in blocks of 64: lane (n = l % 16, g = l / 16) loads the 16
// bytes [64 kb + 16 g, +16) of weight row n and converts them to two bf16x8 operands in registers
// (e4m3 -> f32 is exact and an e4m3 value fits bf16 exactly).  The matching activation lane
// (m = l % 16, g) loads the same 16 k of row m, so the two v_mfma_f32_16x16x32_bf16 steps of a
// block see consistently permuted k; the wave's channel groups share these activation loads.
// Activations come straight from global memory (an expert's few rows stay in L2).  The per-channel
// scale multiplies the f32 accumulator once, in the epilogue.  With weights as the "A" operand a
// lane ends up with four consecutive channels of one row, stored as 8 bytes.
#pragma once

#include <type_traits>

#include "common.h"

namespace fs2moe {

// Partial sums of one 16-row chunk of an expert over k-blocks [kb_lo, kb_hi) for CW groups of 16
// channels (the groups share the activation loads).  K is walked 4 blocks of 64 at a time with all
// of a step's loads issued before any conversion or MFMA: every step is one round trip to memory,
// with 4 * (CW * (DUAL ? 2 : 1) + 2) loads of 1 KB in flight per wave.
template <bool DUAL, int CW>
__device__ __forceinline__ void fp8w_partial(const uint16_t* __restrict__ xr,
                                             const uint8_t* __restrict__ wg,
                                             const uint8_t* __restrict__ wu, size_t group_stride,
                                             int kb_lo, int kb_hi, f32x4 (&accg)[CW],
                                             f32x4 (&accu)[CW]) {
  constexpr int KU = 4;
  auto step = [&](int kb0, auto ku_tag) {
    constexpr int U = decltype(ku_tag)::value;
    u32x4 qg[U][CW], qu[U][CW], xa[U][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int c = 0; c < CW; ++c) {
        const size_t off = c * group_stride + (size_t)(kb0 + u) * 1024;
        qg[u][c] = *reinterpret_cast<const u32x4*>(wg + off);
        if (DUAL) qu[u][c] = *reinterpret_cast<const u32x4*>(wu + off);
      }
      const u32x4* p = reinterpret_cast<const u32x4*>(xr + (size_t)(kb0 + u) * 64);
      xa[u][0] = p[0];
      xa[u][1] = p[1];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bf16x8 x0 = __builtin_bit_cast(bf16x8, xa[u][0]);
      const bf16x8 x1 = __builtin_bit_cast(bf16x8, xa[u][1]);
#pragma unroll
      for (int c = 0; c < CW; ++c) {
        const bf16x8 g0 = fp8x8_to_bf16x8(qg[u][c][0], qg[u][c][1]);
        const bf16x8 g1 = fp8x8_to_bf16x8(qg[u][c][2], qg[u][c][3]);
        accg[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g0, x0, accg[c], 0, 0, 0);
        accg[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(g1, x1, accg[c], 0, 0, 0);
        if (DUAL) {
          const bf16x8 u0 = fp8x8_to_bf16x8(qu[u][c][0], qu[u][c][1]);
          const bf16x8 u1 = fp8x8_to_bf16x8(qu[u][c][2], qu[u][c][3]);
          accu[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u0, x0, accu[c], 0, 0, 0);
          accu[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(u1, x1, accu[c], 0, 0, 0);
        }
      }
    }
  };
  int kb = kb_lo;
#pragma unroll 1
  for (; kb + KU <= kb_hi; kb += KU) step(kb, std::integral_constant<int, KU>{});
  // the remainder in one step as well
  const int rest = kb_hi - kb;  // wave-uniform, < KU
  if (rest == 3) {
    step(kb, std::integral_constant<int, 3>{});
  } else if (rest == 2) {
    step(kb, std::integral_constant<int, 2>{});
  } else if (rest == 1) {
    step(kb, std::integral_constant<int, 1>{});
  }
}

// row_map (may be null): activation row r is read from A[row_map[r]] instead of A[r].
// A [rows, Kdim] bf16; W0/W1 tiled e4m3 [E][N/16][Kdim/64][16][64]; S0/S1 [E, N] f32; C [rows, N] bf16.
// n_blocks = N / (16 * CGW * (4 / KS)) channel blocks per expert (the host picks KS and CGW so that
// this divides); any grid size works, E <= 256 = the block size.
template <bool DUAL, int KS, int CGW>
__global__ __launch_bounds__(256, DUAL ? 4 : 3) void glu_gemm_fp8w_kernel(
    const uint16_t* __restrict__ A, const int32_t* __restrict__ row_map, int lda,
    const uint8_t* __restrict__ W0, const uint8_t* __restrict__ W1,
    const float* __restrict__ S0, const float* __restrict__ S1,
    uint16_t* __restrict__ C, int ldc, int Kdim, int N, const int32_t* __restrict__ counts,
    const int32_t* __restrict__ offsets, int E, int n_blocks) {
  constexpr int CG = 4 / KS;  // sets of CGW channel groups per block
  // partial sums: [wave][channel group][gate | up][lane] as f32x4
  __shared__ f32x4 s_part[4][CGW][2][64];
  __shared__ int32_t s_start[FS2MOE_MAX_EXPERTS + 1], s_cnt[FS2MOE_MAX_EXPERTS],
      s_off[FS2MOE_MAX_EXPERTS];
  __shared__ int32_t s_wave_tot[4];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // ---- item table: expert e has n_blocks * ceil(count / 16) items --------------------------------
  {
    const int cnt = tid < E ? counts[tid] : 0;
    const int items = n_blocks * ((cnt + 15) >> 4);
    int incl = items;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int v = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += v;
    }
    if (lane == 63) s_wave_tot[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += s_wave_tot[w];
    if (tid < E) {
      s_start[tid] = base + incl - items;
      s_cnt[tid] = cnt;
      s_off[tid] = offsets[tid];
    }
    if (tid == E - 1) s_start[E] = base + incl;
    __syncthreads();
  }
  const int total = s_start[E];

  const int cg = wave / KS, ks = wave % KS;  // set of channel groups in the block, part of K
  const int groups = N / 16;                 // N is a multiple of 16
  const int nkb = Kdim / 64;  // the host guarantees Kdim % 64 == 0
  const size_t group_stride = (size_t)Kdim * 16;  // bytes between the tiles of consecutive groups
  const int kb_lo = ks * nkb / KS, kb_hi = (ks + 1) * nkb / KS;

  for (int item = blockIdx.x; item < total; item += gridDim.x) {
    // (what follows from the lane number is worked out per item from an opaque copy of it: hoisted
    // out of this loop, the addresses' lane parts took registers the inner loop has no room for and
    // were spilled to scratch and reloaded for every item)
    int lane_l = tid & 63;
    asm volatile("" : "+v"(lane_l));
    const int lane = lane_l, ln = lane & 15, g = lane >> 4;
    // expert of the item (wave-uniform)
    int e = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int ei = e0 + lane;
      const bool hit = ei < E && s_start[ei] <= item && item < s_start[ei + 1];
      const unsigned long long m = __ballot(hit);
      if (m) e = e0 + (int)__builtin_ctzll(m);
    }
    e = __builtin_amdgcn_readfirstlane(e);
    const int cnt = s_cnt[e], row0 = s_off[e];
    const int chunks = (cnt + 15) >> 4;
    const int l = item - s_start[e];
    // chunk-minor order in steps of 8 items when the channel blocks come in eights (see above)
    int nbi, rc;
    if ((n_blocks & 7) == 0) {
      rc = (l >> 3) % chunks;
      nbi = (l / (8 * chunks)) * 8 + (l & 7);
    } else {
      nbi = l / chunks;
      rc = l - nbi * chunks;
    }
    const int m0 = rc * 16;
    const int gq = (nbi * CG + cg) * CGW;  // first of the wave's channel groups; gq + CGW <= groups

    // tile (group, kb) of expert e starts at ((e * N/16 + group) * Kdim/64 + kb) * 1024
    const size_t wrow = ((size_t)e * groups + gq) * group_stride + ln * 64 + 16 * g;
    int r = m0 + ln;
    r = r < cnt ? r : cnt - 1;  // clamped rows are computed but never stored
    // fused gather: rows below cnt are real pairs, so their map entries are tokens
    const int src = row_map != nullptr ? row_map[row0 + r] : row0 + r;
    f32x4 accg[CGW], accu[CGW];
#pragma unroll
    for (int c = 0; c < CGW; ++c) {
      accg[c] = f32x4{0.f, 0.f, 0.f, 0.f};
      accu[c] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    fp8w_partial<DUAL, CGW>(A + (size_t)src * lda + 16 * g, W0 + wrow, DUAL ? W1 + wrow : W0,
                            group_stride, kb_lo, kb_hi, accg, accu);
    if (item != (int)blockIdx.x) __syncthreads();  // the last item's partial sums have been consumed
#pragma unroll
    for (int c = 0; c < CGW; ++c) {
      s_part[wave][c][0][lane] = accg[c];
      if (DUAL) s_part[wave][c][1][lane] = accu[c];
    }
    __syncthreads();
    // The KS waves of a set share out its channel groups: wave ks finishes group ks: the KS partial
    // sums in wave order, scale, gate, store.
    static_assert(CGW <= KS, "a wave finishes at most one channel group");
    if (ks < CGW) {
      const int c = ks;
      const int n0 = (gq + c) * 16;
      const int w0 = cg * KS;
      f32x4 tg = s_part[w0][c][0][lane], tu = tg;
      if (DUAL) tu = s_part[w0][c][1][lane];
#pragma unroll
      for (int w = 1; w < KS; ++w) {
        tg += s_part[w0 + w][c][0][lane];
        if (DUAL) tu += s_part[w0 + w][c][1][lane];
      }
      if (m0 + ln < cnt) {
        // Accumulator layout: lane holds channels n0 + 4g + {0..3} of row m0 + ln.
        const f32x4 sg = *reinterpret_cast<const f32x4*>(S0 + (size_t)e * N + n0 + 4 * g);
        f32x4 su = sg;
        if (DUAL) su = *reinterpret_cast<const f32x4*>(S1 + (size_t)e * N + n0 + 4 * g);
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float a = tg[j] * sg[j];
          v[j] = DUAL ? silu_f32(a) * (tu[j] * su[j]) : a;
        }
        u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        *reinterpret_cast<u32x2*>(C + (size_t)(row0 + m0 + ln) * ldc + n0 + 4 * g) = o;
      }
    }
  }
}

}  // namespace fs2moe

// Output-tile scheduling of the grouped GEMMs: which expert and row range a block works on.
#pragma once

#include "common.h"

namespace fs2moe {

struct Groups {
  const int32_t* counts;   // [E] tokens per expert, or nullptr for one dense group
  const int32_t* offsets;  // [E + 1] first row of each expert
  int E;
  int dense_rows;
};

// Finds the (expert, row range) of m-tile `mt`.  All 256 threads of the block must call it.
template <int BM>
__device__ __forceinline__ bool locate_tile(const Groups& g, int mt, int& e, int& row0,
                                            int& row_end) {
  if (g.counts == nullptr) {
    e = 0;
    row0 = mt * BM;
    row_end = g.dense_rows;
    return row0 < row_end;
  }
  __shared__ int s_wave_tot[2][4];
  __shared__ int s_tile[3];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) s_tile[0] = -1;
  // the experts 256 at a time (one per thread), carrying the tiles of the rounds before
  int carried = 0;
  for (int e0 = 0; e0 < g.E; e0 += 256) {
    const int ex = e0 + tid, par = (e0 >> 8) & 1;
    const int cnt = ex < g.E ? g.counts[ex] : 0;
    const int tiles = (cnt + BM - 1) / BM;
    int incl = tiles;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      int v = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += v;
    }
    if (lane == 63) s_wave_tot[par][wave] = incl;
    __syncthreads();
    int base = carried;
    for (int w = 0; w < wave; ++w) base += s_wave_tot[par][w];
    const int excl = base + incl - tiles;
    if (tiles > 0 && mt >= excl && mt < excl + tiles) {
      const int off = g.offsets[ex];
      s_tile[0] = ex;
      s_tile[1] = off + (mt - excl) * BM;
      s_tile[2] = off + cnt;
    }
    for (int w = 0; w < 4; ++w) carried += s_wave_tot[par][w];
  }
  __syncthreads();
  e = s_tile[0];
  row0 = s_tile[1];
  row_end = s_tile[2];
  return e >= 0;
}

}  // namespace fs2moe

// All of dispatch for at most 256 tokens when no rows are copied: count, scan and index by one block.
// A device function, because two kernels end with it: dispatch_small_kernel (fs2moe_dispatch) and
// the router's finishing kernel for a few tokens, which selects the experts and dispatches in one
// launch.
#pragma once

#include "common.h"

namespace fs2moe {

constexpr int kDispTok = 256;  // tokens per block in the counting pass
constexpr int kDispWords = kDispTok / 32;

// LDS words dispatch_small_block needs at s_mem
__host__ __device__ inline size_t dispatch_small_lds_words(int E) {
  return (size_t)E * kDispWords * 2 + E + 1;
}

// write: the results go to memory (else they are only left in LDS: s_bits, s_pref, s_off at s_mem).
// KCAP: a compile-time bound on K.  E <= 256 (a thread per expert in the scan).
// Called by every thread of a block of `nthreads` >= 256 threads (a multiple of 64); threads 0..255
// are the tokens' threads, the others only help with the loops over LDS and pass the barriers.
// topk_idx (and topk_w, read only when row_w is given) may have been written by this block before a
// barrier.
template <int KCAP>
__device__ __forceinline__ void dispatch_small_block(
    const int32_t* topk_idx, int T, int K, int E, int tile_m, int64_t max_rows, int32_t* counts,
    int32_t* offsets, int32_t* perm, int32_t* inv_perm, uint32_t* s_mem, int32_t* s_wave_tot,
    int tid, int nthreads, bool write = true, const float* topk_w = nullptr,
    float* row_w = nullptr) {
  uint32_t* s_bits = s_mem;                    // [E][kDispWords] membership bitmaps
  uint32_t* s_pref = s_mem + E * kDispWords;   // [E][kDispWords] members in the words below
  int32_t* s_off = reinterpret_cast<int32_t*>(s_pref + E * kDispWords);  // [E + 1]
  const int lane = tid & 63, wave = tid >> 6;
  const int t = tid;
  const bool has_token = t < T && tid < kDispTok;
  // The token's experts, loaded first and unconditionally (from the first token's where this thread
  // has no token or k is past K), so that all the loads are in flight together behind the clearing
  // of the bitmaps; what does not count is set to -1 afterwards.
  int ek[KCAP];
  {
    const int32_t* mine = topk_idx + (has_token ? (size_t)t * K : 0);
#pragma unroll
    for (int k = 0; k < KCAP; ++k)
      ek[k] = mine[k < K ? k : 0];
  }
  for (int i = tid; i < E * kDispWords; i += nthreads) s_bits[i] = 0u;
  __syncthreads();
  const int word = tid >> 5;
  const uint32_t bit = 1u << (tid & 31);
#pragma unroll
  for (int k = 0; k < KCAP; ++k) {
    const int e = ek[k];
    ek[k] = (has_token && k < K && e >= 0 && e < E) ? e : -1;
    if (ek[k] >= 0) atomicOr(&s_bits[ek[k] * kDispWords + word], bit);
  }
  __syncthreads();
  for (int i = tid; i < E * kDispWords; i += nthreads) {
    const int e = i / kDispWords, w = i % kDispWords;
    uint32_t c = 0;
    for (int j = 0; j < w; ++j) c += __popc(s_bits[e * kDispWords + j]);
    s_pref[i] = c;
  }
  __syncthreads();
  // counts and tile-padded offsets: thread e, a block-wide exclusive scan (E <= 256 = block size)
  int cnt = 0, padded = 0;
  if (tid < E) {
    const int i = tid * kDispWords + kDispWords - 1;
    cnt = (int)(s_pref[i] + __popc(s_bits[i]));
    if (write) counts[tid] = cnt;
    padded = (cnt + tile_m - 1) / tile_m * tile_m;
  }
  int incl = padded;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int v = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += v;
  }
  if (lane == 63 && wave < 4) s_wave_tot[wave] = incl;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave && w < 4; ++w) base += s_wave_tot[w];
  if (tid < E) {
    if (write) offsets[tid] = base + incl - padded;
    s_off[tid] = base + incl - padded;
  }
  if (tid == E - 1) {
    if (write) offsets[E] = base + incl;
    s_off[E] = base + incl;
  }
  __syncthreads();
  // (write false: the bitmaps, prefixes and offsets stay in LDS for the caller, nothing goes to memory)
  if (!write) return;
  // pairs
#pragma unroll
  for (int k = 0; k < KCAP; ++k) {
    if (k < K && t < T && tid < kDispTok) {
      const size_t p = (size_t)t * K + k;
      if (ek[k] < 0) {
        inv_perm[p] = -1;
      } else {
        const int i = ek[k] * kDispWords + word;
        const int row = s_off[ek[k]] + (int)(s_pref[i] + __popc(s_bits[i] & (bit - 1u)));
        inv_perm[p] = row;
        perm[row] = t;
        // (for kernels that scale a row by its routing weight while they read it through perm)
        if (row_w != nullptr) row_w[row] = topk_w[p];
      }
    }
  }
  // padding rows of expert tid, then the rows beyond offsets[E]
  if (tid < E)
    for (int r = s_off[tid] + cnt; r < s_off[tid + 1]; ++r) perm[r] = -1;
  for (int64_t r = (int64_t)s_off[E] + tid; r < max_rows; r += nthreads) perm[r] = -1;
}

}  // namespace fs2moe

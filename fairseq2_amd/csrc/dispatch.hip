// Token dispatch: per-expert histogram, tile-padded exclusive scan, stable permutation and the
// gather of token rows into expert-contiguous order.
//
// Determinism: the row of pair (expert e, token t) is offsets[e] + |{t' < t : e selected by t'}|.
// Each block of 256 consecutive tokens records, per expert, a 256-bit membership bitmap in LDS
// (atomicOr: order-independent), so a pair's rank inside its block is a population count of the
// bits below its token, and the block's base is a prefix over the per-block counts.  No float or
// order-dependent atomics are involved; the result is the expert-major, token-ascending order.
#include "common.h"
#include "dispatch_small.h"

namespace fs2moe {

// The experts of token t, -1 where there is none (t past T, k past K, an index outside [0, E)).
// Every load is issued, from an address inside the array, before any result is looked at: a load
// behind a condition is waited for on the spot, one round trip per k.
// KCAP: a compile-time bound on K (16 covers every published layer; 32 is the library's limit).
template <int KCAP>
__device__ __forceinline__ void load_token_experts(const int32_t* __restrict__ topk_idx, int t,
                                                   int T, int K, int E, int (&ek)[KCAP]) {
  const bool has_token = t < T;
  const int32_t* mine = topk_idx + (has_token ? (size_t)t * K : 0);
#pragma unroll
  for (int k = 0; k < KCAP; ++k) ek[k] = mine[k < K ? k : 0];
#pragma unroll
  for (int k = 0; k < KCAP; ++k) {
    const int e = ek[k];
    ek[k] = (has_token && k < K && e >= 0 && e < E) ? e : -1;
  }
}

template <int KCAP>
__global__ __launch_bounds__(kDispTok) void dispatch_count_kernel(
    const int32_t* __restrict__ topk_idx, int T, int K, int E, int32_t* __restrict__ block_counts,
    int32_t* __restrict__ rank) {
  extern __shared__ uint32_t s_mem[];
  uint32_t* s_bits = s_mem;                    // [E][kDispWords] membership bitmaps
  uint32_t* s_pref = s_mem + E * kDispWords;   // [E][kDispWords] members in the words below
  const int tid = threadIdx.x;
  for (int i = tid; i < E * kDispWords; i += kDispTok) s_bits[i] = 0u;
  __syncthreads();
  const int t = blockIdx.x * kDispTok + tid;
  const int word = tid >> 5;
  const uint32_t bit = 1u << (tid & 31);
  // the token's experts stay in registers between the two passes
  int ek[KCAP];
  load_token_experts<KCAP>(topk_idx, t, T, K, E, ek);
#pragma unroll
  for (int k = 0; k < KCAP; ++k)
    if (ek[k] >= 0) atomicOr(&s_bits[ek[k] * kDispWords + word], bit);
  __syncthreads();
  for (int i = tid; i < E * kDispWords; i += kDispTok) {
    const int e = i / kDispWords, w = i % kDispWords;
    uint32_t c = 0;
    for (int j = 0; j < w; ++j) c += __popc(s_bits[e * kDispWords + j]);
    s_pref[i] = c;
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < KCAP; ++k) {
    if (k < K && t < T) {
      int r = 0;
      if (ek[k] >= 0) {
        const int i = ek[k] * kDispWords + word;
        r = (int)(s_pref[i] + __popc(s_bits[i] & (bit - 1u)));
      }
      rank[(size_t)t * K + k] = r;
    }
  }
  for (int e = tid; e < E; e += kDispTok) {
    const int i = e * kDispWords + kDispWords - 1;
    block_counts[(size_t)blockIdx.x * E + e] = (int)(s_pref[i] + __popc(s_bits[i]));
  }
}

// One block of 256 threads, the experts 256 at a time (one per thread, the rows of the rounds before
// carried along).  Turns per-block counts into per-block exclusive prefixes (in place), and writes
// counts and the tile-padded offsets (a block-wide exclusive scan).
__global__ __launch_bounds__(256) void dispatch_scan_kernel(int32_t* __restrict__ block_counts,
                                                            int num_blocks, int E, int tile_m,
                                                            int32_t* __restrict__ counts,
                                                            int32_t* __restrict__ offsets) {
  __shared__ int32_t s_wave_tot[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int carried = 0;
  for (int e0 = 0; e0 < E; e0 += 256) {
    const int ex = e0 + tid, par = (e0 >> 8) & 1;
    int padded = 0;
    if (ex < E) {
      // chunks of 8 blocks: the loads of a chunk are independent of its stores and go out together
      int run = 0;
      for (int b0 = 0; b0 < num_blocks; b0 += 8) {
        int c[8];
#pragma unroll
        for (int i = 0; i < 8; ++i)
          c[i] = b0 + i < num_blocks ? block_counts[(size_t)(b0 + i) * E + ex] : 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (b0 + i < num_blocks) block_counts[(size_t)(b0 + i) * E + ex] = run;
          run += c[i];
        }
      }
      counts[ex] = run;
      padded = (run + tile_m - 1) / tile_m * tile_m;
    }
    int incl = padded;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      int v = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += v;
    }
    if (lane == 63) s_wave_tot[par][wave] = incl;
    __syncthreads();
    int base = carried;
    for (int w = 0; w < wave; ++w) base += s_wave_tot[par][w];
    if (ex < E) offsets[ex] = base + incl - padded;
    if (ex == E - 1) offsets[E] = base + incl;
    for (int w = 0; w < 4; ++w) carried += s_wave_tot[par][w];
  }
}

template <typename TA>
__device__ __forceinline__ u32x4 scale_chunk(u32x4 v, float w);
template <>
__device__ __forceinline__ u32x4 scale_chunk<float>(u32x4 v, float w) {
  u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = __float_as_uint(__uint_as_float(v[i]) * w);
  return o;
}
template <>
__device__ __forceinline__ u32x4 scale_chunk<uint16_t>(u32x4 v, float w) {
  u32x4 o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = scale_bf16x2(v[i], w);
  return o;
}

// Blocks [0, pair_blocks): one wave per (token, slot) pair computes the pair's row and copies the
// token's row there.  Block pair_blocks + e: marks the padding rows of expert e (perm = -1) and
// zero-fills them.  Remaining blocks: perm = -1 for the rows beyond offsets[E].  The three row sets
// are disjoint, so no ordering between the blocks is needed.
template <typename TA>
__global__ __launch_bounds__(256) void dispatch_permute_kernel(
    const int32_t* __restrict__ topk_idx, const float* __restrict__ topk_w,
    const TA* __restrict__ x, int T, int K, int E, int D, int scale_input, int64_t max_rows,
    unsigned pair_blocks, const int32_t* __restrict__ counts, const int32_t* __restrict__ offsets,
    const int32_t* __restrict__ block_prefix, const int32_t* __restrict__ rank,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm, TA* __restrict__ xe) {
  const int lane = lane_id();
  const int chunks = D * (int)sizeof(TA) / 16;
  if (blockIdx.x >= pair_blocks) {
    const int idx = blockIdx.x - pair_blocks;
    const int tid = threadIdx.x;
    if (idx < E) {
      const int64_t lo = (int64_t)offsets[idx] + counts[idx], hi = offsets[idx + 1];
      for (int64_t r = lo + tid; r < hi; r += 256) perm[r] = -1;
      if (xe != nullptr) {
        const int64_t n = (hi - lo) * chunks;
        u32x4* dst = reinterpret_cast<u32x4*>(xe + lo * D);
        const u32x4 z = {0u, 0u, 0u, 0u};
        for (int64_t i = tid; i < n; i += 256) dst[i] = z;
      }
    } else {
      const int64_t r = (int64_t)offsets[E] + (int64_t)(idx - E) * 256 + tid;
      if (r < max_rows) perm[r] = -1;
    }
    return;
  }
  const int64_t p = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
  if (p >= (int64_t)T * K) return;
  const int t = (int)(p / K);
  const int e = topk_idx[p];
  if (e < 0 || e >= E) {
    if (lane == 0) inv_perm[p] = -1;
    return;
  }
  const int row = offsets[e] + block_prefix[(size_t)(t / kDispTok) * E + e] + rank[p];
  if (lane == 0) {
    inv_perm[p] = row;
    perm[row] = t;
  }
  if (xe == nullptr) return;
  const u32x4* src = reinterpret_cast<const u32x4*>(x + (size_t)t * D);
  u32x4* dst = reinterpret_cast<u32x4*>(xe + (size_t)row * D);
  if (scale_input) {
    const float w = topk_w[p];
    for (int c = lane; c < chunks; c += kWave) dst[c] = scale_chunk<TA>(src[c], w);
  } else {
    for (int c = lane; c < chunks; c += kWave) dst[c] = src[c];
  }
}

// The bookkeeping of dispatch_permute_kernel without the row copy (xe == NULL: the caller reads the
// rows through perm): one thread per (token, slot) pair, then per padding row.
__global__ __launch_bounds__(256) void dispatch_index_kernel(
    const int32_t* __restrict__ topk_idx, int T, int K, int E, int64_t max_rows,
    unsigned pair_blocks, const int32_t* __restrict__ counts, const int32_t* __restrict__ offsets,
    const int32_t* __restrict__ block_prefix, const int32_t* __restrict__ rank,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm) {
  const int tid = threadIdx.x;
  if (blockIdx.x >= pair_blocks) {
    const int idx = blockIdx.x - pair_blocks;
    if (idx < E) {
      const int64_t lo = (int64_t)offsets[idx] + counts[idx], hi = offsets[idx + 1];
      for (int64_t r = lo + tid; r < hi; r += 256) perm[r] = -1;
    } else {
      const int64_t r = (int64_t)offsets[E] + (int64_t)(idx - E) * 256 + tid;
      if (r < max_rows) perm[r] = -1;
    }
    return;
  }
  const int64_t p = (int64_t)blockIdx.x * 256 + tid;
  if (p >= (int64_t)T * K) return;
  const int t = (int)(p / K);
  const int e = topk_idx[p];
  if (e < 0 || e >= E) {
    inv_perm[p] = -1;
    return;
  }
  const int row = offsets[e] + block_prefix[(size_t)(t / kDispTok) * E + e] + rank[p];
  inv_perm[p] = row;
  perm[row] = t;
}

// dispatch_scan_kernel and dispatch_index_kernel in one launch, for up to kIndexScanBlocks counting
// blocks: the table of per-block counts is a few KB in L2, so EVERY block of the index pass works the
// scan out for itself in LDS (a microsecond, all blocks at once) instead of waiting for a launch of
// one block to do it; block 0 writes counts and offsets for the kernels that follow.  block_counts
// stays as the counting pass wrote it.  Same integers as the two kernels.
constexpr int kIndexScanBlocks = 64;
__global__ __launch_bounds__(256) void dispatch_index_scan_kernel(
    const int32_t* __restrict__ topk_idx, int T, int K, int E, int tile_m, int64_t max_rows,
    unsigned pair_blocks, const int32_t* __restrict__ block_counts, int num_blocks,
    const int32_t* __restrict__ rank, int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm) {
  extern __shared__ int32_t s_tab[];
  int32_t* s_off = s_tab;           // [E + 1]
  int32_t* s_cnt = s_off + E + 1;   // [E]
  int32_t* s_pre = s_cnt + E;       // [2][E]: rows of the counting blocks before b0 and before b0 + 1
  __shared__ int32_t s_wave_tot[2][4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool pair_block = blockIdx.x < pair_blocks;
  // the block's 256 pairs belong to at most 256 tokens, i.e. to counting blocks b0 and b0 + 1
  const int b0 = pair_block ? (int)(((int64_t)blockIdx.x * 256 / K) / kDispTok) : 0;
  int carried = 0;
  for (int e0 = 0; e0 < E; e0 += 256) {
    const int ex = e0 + tid, par = (e0 >> 8) & 1;
    int padded = 0;
    if (ex < E) {
      int run = 0, pre0 = 0, pre1 = 0;
      for (int i0 = 0; i0 < num_blocks; i0 += 16) {
        int c[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
          c[i] = block_counts[(size_t)(i0 + i < num_blocks ? i0 + i : 0) * E + ex];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          if (i0 + i == b0) pre0 = run;
          if (i0 + i == b0 + 1) pre1 = run;
          if (i0 + i < num_blocks) run += c[i];
        }
      }
      s_cnt[ex] = run;
      s_pre[ex] = pre0;
      s_pre[E + ex] = pre1;
      padded = (run + tile_m - 1) / tile_m * tile_m;
    }
    int incl = padded;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      int v = __shfl_up(incl, off, kWave);
      if (lane >= off) incl += v;
    }
    if (lane == 63) s_wave_tot[par][wave] = incl;
    __syncthreads();
    int base = carried;
    for (int w = 0; w < wave; ++w) base += s_wave_tot[par][w];
    if (ex < E) s_off[ex] = base + incl - padded;
    if (ex == E - 1) s_off[E] = base + incl;
    for (int w = 0; w < 4; ++w) carried += s_wave_tot[par][w];
  }
  __syncthreads();
  if (blockIdx.x == 0) {
    for (int e = tid; e < E; e += 256) {
      counts[e] = s_cnt[e];
      offsets[e] = s_off[e];
    }
    if (tid == 0) offsets[E] = s_off[E];
  }
  if (!pair_block) {
    const int idx = blockIdx.x - pair_blocks;
    if (idx < E) {
      const int64_t lo = (int64_t)s_off[idx] + s_cnt[idx], hi = s_off[idx + 1];
      for (int64_t r = lo + tid; r < hi; r += 256) perm[r] = -1;
    } else {
      const int64_t r = (int64_t)s_off[E] + (int64_t)(idx - E) * 256 + tid;
      if (r < max_rows) perm[r] = -1;
    }
    return;
  }
  const int64_t p = (int64_t)blockIdx.x * 256 + tid;
  if (p >= (int64_t)T * K) return;
  const int t = (int)(p / K);
  const int e = topk_idx[p];
  if (e < 0 || e >= E) {
    inv_perm[p] = -1;
    return;
  }
  const int row = s_off[e] + s_pre[(t / kDispTok - b0) * E + e] + rank[p];
  inv_perm[p] = row;
  perm[row] = t;
}

// The index pass after a router that counted for itself: tile_counts[tile][e] (bytes) is the number
// of tile `tile`'s 32 tokens that chose expert e and tile_rank[p] the rank of pair p among its
// tile's pairs of the same expert, token-ascending.  Block b < tile_blocks places the pairs of tile b;
// as in dispatch_index_scan_kernel every block adds the table up for itself (num_tiles x E bytes
// from L2: thread (slice, group of 8 experts) takes every S-th tile, 8 bytes a load, all of a
// round's loads issued before any is looked at), block 0 writes counts and offsets, and the blocks
// past the tiles fill the padding rows of perm.  Same integers as the other dispatch kernels.
// E a multiple of 8 and at most 256 (one thread per expert in the scan).
constexpr int kTileSumLoads = 8;
__global__ __launch_bounds__(256) void dispatch_index_tiles_kernel(
    const int32_t* __restrict__ topk_idx, int T, int K, int E, int tile_m, int64_t max_rows,
    unsigned tile_blocks, const uint8_t* __restrict__ tile_counts, int num_tiles,
    const int32_t* __restrict__ tile_rank, int32_t* __restrict__ counts,
    int32_t* __restrict__ offsets, int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm) {
  __shared__ int32_t s_part[2][2048];  // [all tiles | tiles before mine][slice][expert]: S E <= 2048
  __shared__ int32_t s_off[257], s_cnt[256], s_pre[256];
  __shared__ int32_t s_wave_tot[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const bool tile_block = blockIdx.x < tile_blocks;
  const int mine = tile_block ? (int)blockIdx.x : 0;
  const int G = E >> 3, S = 256 / G;
  const int g = tid % G, sl = tid / G;
  if (sl < S) {
    int tot[8], pre[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) tot[j] = pre[j] = 0;
    for (int t0 = sl; t0 < num_tiles; t0 += S * kTileSumLoads) {
      uint2 c[kTileSumLoads];
#pragma unroll
      for (int i = 0; i < kTileSumLoads; ++i) {
        const int tile = t0 + i * S;
        c[i] = *reinterpret_cast<const uint2*>(tile_counts + (size_t)(tile < num_tiles ? tile : 0) * E +
                                               g * 8);
      }
#pragma unroll
      for (int i = 0; i < kTileSumLoads; ++i) {
        const int tile = t0 + i * S;
        const bool in = tile < num_tiles, before = tile < mine;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int v = in ? (int)(((j < 4 ? c[i].x : c[i].y) >> (8 * (j & 3))) & 0xffu) : 0;
          tot[j] += v;
          pre[j] += before ? v : 0;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      s_part[0][sl * E + g * 8 + j] = tot[j];
      s_part[1][sl * E + g * 8 + j] = pre[j];
    }
  }
  __syncthreads();
  int padded = 0;
  if (tid < E) {
    int run = 0, pre = 0;
    for (int i = 0; i < S; ++i) {
      run += s_part[0][i * E + tid];
      pre += s_part[1][i * E + tid];
    }
    s_cnt[tid] = run;
    s_pre[tid] = pre;
    padded = (run + tile_m - 1) / tile_m * tile_m;
  }
  int incl = padded;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int v = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += v;
  }
  if (lane == 63) s_wave_tot[wave] = incl;
  __syncthreads();
  int base = 0;
  for (int w = 0; w < wave; ++w) base += s_wave_tot[w];
  if (tid < E) s_off[tid] = base + incl - padded;
  if (tid == E - 1) s_off[E] = base + incl;
  __syncthreads();
  if (blockIdx.x == 0) {
    if (tid < E) {
      counts[tid] = s_cnt[tid];
      offsets[tid] = s_off[tid];
    }
    if (tid == 0) offsets[E] = s_off[E];
  }
  if (!tile_block) {
    const int idx = blockIdx.x - tile_blocks;
    if (idx < E) {
      const int64_t lo = (int64_t)s_off[idx] + s_cnt[idx], hi = s_off[idx + 1];
      for (int64_t r = lo + tid; r < hi; r += 256) perm[r] = -1;
    } else {
      const int64_t r = (int64_t)s_off[E] + (int64_t)(idx - E) * 256 + tid;
      if (r < max_rows) perm[r] = -1;
    }
    return;
  }
  const int64_t p0 = (int64_t)mine * kRouterTileTok * K, pairs = (int64_t)T * K;
  for (int i = tid; i < kRouterTileTok * K; i += 256) {
    const int64_t p = p0 + i;
    if (p >= pairs) break;
    const int e = topk_idx[p];
    if (e < 0 || e >= E) {
      inv_perm[p] = -1;
      continue;
    }
    const int row = s_off[e] + s_pre[e] + tile_rank[p];
    inv_perm[p] = row;
    perm[row] = (int)(p / K);
  }
}

// All of dispatch for at most 256 tokens when no rows are copied (xe == NULL): count, scan and
// index in one block.  A decode step spends more on starting three kernels than on their work.
// Same arithmetic as the three kernels above, so the results are identical.
template <int KCAP>
__global__ __launch_bounds__(kDispTok) void dispatch_small_kernel(
    const int32_t* __restrict__ topk_idx, int T, int K, int E, int tile_m, int64_t max_rows,
    int32_t* __restrict__ counts, int32_t* __restrict__ offsets, int32_t* __restrict__ perm,
    int32_t* __restrict__ inv_perm, const float* __restrict__ topk_w, float* __restrict__ row_w) {
  extern __shared__ uint32_t s_mem[];
  __shared__ int32_t s_wave_tot[4];
  dispatch_small_block<KCAP>(topk_idx, T, K, E, tile_m, max_rows, counts, offsets, perm, inv_perm, s_mem,
                       s_wave_tot, threadIdx.x, kDispTok, true, topk_w, row_w);
}

// All of dispatch for at most 256 tokens WITH the row copy, in one launch: every block works out the
// bookkeeping for itself in LDS (it is a few microseconds of work, and a decode step spends more on
// starting three kernels), block 0 writes it to memory, and then the blocks do what
// dispatch_permute_kernel's do: blocks [0, pair_blocks) copy (and scale) a pair's row per wave,
// block pair_blocks + e zero-fills the padding rows of expert e.  Same arithmetic, same results.
template <typename TA, int KCAP>
__global__ __launch_bounds__(kDispTok) void dispatch_small_copy_kernel(
    const int32_t* __restrict__ topk_idx, const float* __restrict__ topk_w,
    const TA* __restrict__ x, int T, int K, int E, int D, int tile_m, int scale_input,
    int64_t max_rows, unsigned pair_blocks, int32_t* __restrict__ counts,
    int32_t* __restrict__ offsets, int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm,
    TA* __restrict__ xe) {
  extern __shared__ uint32_t s_mem[];
  __shared__ int32_t s_wave_tot[4];
  dispatch_small_block<KCAP>(topk_idx, T, K, E, tile_m, max_rows, counts, offsets, perm, inv_perm,
                             s_mem, s_wave_tot, threadIdx.x, kDispTok, blockIdx.x == 0);
  const uint32_t* s_bits = s_mem;
  const uint32_t* s_pref = s_mem + E * kDispWords;
  const int32_t* s_off = reinterpret_cast<const int32_t*>(s_pref + E * kDispWords);
  const int lane = lane_id();
  const int chunks = D * (int)sizeof(TA) / 16;
  if (blockIdx.x >= pair_blocks) {
    const int idx = blockIdx.x - pair_blocks;  // < E
    const int i = idx * kDispWords + kDispWords - 1;
    const int cnt = (int)(s_pref[i] + __popc(s_bits[i]));
    const int64_t lo = (int64_t)s_off[idx] + cnt, hi = s_off[idx + 1];
    const int64_t n = (hi - lo) * chunks;
    u32x4* dst = reinterpret_cast<u32x4*>(xe + lo * D);
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int64_t c = threadIdx.x; c < n; c += kDispTok) dst[c] = z;
    return;
  }
  const int64_t p = (int64_t)blockIdx.x * 4 + threadIdx.x / kWave;
  if (p >= (int64_t)T * K) return;
  const int t = (int)(p / K);
  const int e = topk_idx[p];
  if (e < 0 || e >= E) return;
  const int w = e * kDispWords + (t >> 5);
  const int row = s_off[e] + (int)(s_pref[w] + __popc(s_bits[w] & ((1u << (t & 31)) - 1u)));
  const u32x4* src = reinterpret_cast<const u32x4*>(x + (size_t)t * D);
  u32x4* dst = reinterpret_cast<u32x4*>(xe + (size_t)row * D);
  if (scale_input) {
    const float wt = topk_w[p];
    for (int c = lane; c < chunks; c += kWave) dst[c] = scale_chunk<TA>(src[c], wt);
  } else {
    for (int c = lane; c < chunks; c += kWave) dst[c] = src[c];
  }
}

}  // namespace fs2moe

using namespace fs2moe;

int fs2moe::dispatch_index_tiles(const int32_t* topk_idx, int32_t T, int32_t K, int32_t E,
                                 int32_t tile_m, int64_t max_rows, const uint8_t* tile_counts,
                                 const int32_t* tile_rank, int32_t* counts, int32_t* offsets,
                                 int32_t* perm, int32_t* inv_perm, void* stream) {
  const int nt = (T + kRouterTileTok - 1) / kRouterTileTok;
  FS2_REQUIRE(E % 8 == 0 && E <= 256 && nt >= 1 && nt <= kIndexTilesMax,
              "dispatch: internal: E=%d, %d tiles given to the tile form", E, nt);
  FS2_REQUIRE(max_rows >= FS2MOE_MAX_ROWS(T, K, E, tile_m) && max_rows < (1ll << 31),
              "dispatch: max_rows=%lld outside [%lld, 2^31)", (long long)max_rows,
              (long long)FS2MOE_MAX_ROWS(T, K, E, tile_m));
  const unsigned tail_blocks = (unsigned)((max_rows - (int64_t)T * K + 255) / 256);
  hipLaunchKernelGGL(dispatch_index_tiles_kernel, dim3((unsigned)nt + (unsigned)E + tail_blocks),
                     dim3(256), 0, static_cast<hipStream_t>(stream), topk_idx, T, K, E, tile_m,
                     max_rows, (unsigned)nt, tile_counts, nt, tile_rank, counts, offsets, perm,
                     inv_perm);
  return check_launch("dispatch_index_tiles");
}

int fs2moe::dispatch_with_row_weights(const int32_t* topk_idx, const float* topk_w, int32_t T,
                                      int32_t K, int32_t E, int32_t tile_m, int64_t max_rows,
                                      int32_t* counts, int32_t* offsets, int32_t* perm,
                                      int32_t* inv_perm, float* row_w, void* stream) {
  FS2_REQUIRE(topk_idx && topk_w && counts && offsets && perm && inv_perm && row_w,
              "dispatch: null pointer");
  FS2_REQUIRE(T >= 1 && T <= kDispTok && E >= 1 && E <= kDispTok && K >= 1 && K <= FS2MOE_MAX_TOP_K,
              "dispatch: internal: T=%d E=%d K=%d given to the one-block form", T, E, K);
  FS2_REQUIRE(tile_m >= 1 && tile_m <= 1024, "dispatch: tile_m=%d", tile_m);
  FS2_REQUIRE(max_rows >= FS2MOE_MAX_ROWS(T, K, E, tile_m) && max_rows < (1ll << 31),
              "dispatch: max_rows=%lld outside [%lld, 2^31)", (long long)max_rows,
              (long long)FS2MOE_MAX_ROWS(T, K, E, tile_m));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = dispatch_small_lds_words(E) * sizeof(uint32_t);
  if (K <= 16)
    hipLaunchKernelGGL(dispatch_small_kernel<16>, dim3(1), dim3(kDispTok), lds, s, topk_idx, T, K, E,
                       tile_m, max_rows, counts, offsets, perm, inv_perm, topk_w, row_w);
  else
    hipLaunchKernelGGL(dispatch_small_kernel<FS2MOE_MAX_TOP_K>, dim3(1), dim3(kDispTok), lds, s,
                       topk_idx, T, K, E, tile_m, max_rows, counts, offsets, perm, inv_perm, topk_w,
                       row_w);
  return check_launch("dispatch_small (row weights)");
}

extern "C" int64_t fs2moe_dispatch_workspace_bytes(int32_t T, int32_t K, int32_t E) {
  if (T < 0 || K < 1 || E < 1) return -1;
  const int64_t nb = (T + kDispTok - 1) / kDispTok;
  // per-block counts and per-pair ranks; twice the counts' room so that the same bytes also hold
  // the form a tile-counting router leaves (a byte per expert and tile of 32 tokens, then the
  // ranks from the next multiple of 256 bytes on: tile_rank_of)
  int64_t bytes = (2 * nb * E + (int64_t)T * K) * (int64_t)sizeof(int32_t);
  return (bytes + 255) / 256 * 256 + 256;
}

extern "C" int fs2moe_dispatch(const int32_t* topk_idx, const float* topk_w, const void* x,
                               int32_t T, int32_t K, int32_t E, int32_t D, int32_t tile_m,
                               int32_t act_dtype, int32_t scale_input, int64_t max_rows,
                               int32_t* counts, int32_t* offsets, int32_t* perm,
                               int32_t* inv_perm, void* xe, void* workspace,
                               int64_t workspace_bytes, void* stream) {
  FS2_REQUIRE(topk_idx && counts && offsets && perm && inv_perm && workspace,
              "dispatch: null pointer");
  FS2_REQUIRE(T >= 0 && K >= 1 && K <= FS2MOE_MAX_TOP_K, "dispatch: bad T=%d K=%d", T, K);
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS, "dispatch: E=%d outside [1, %d]", E,
              FS2MOE_MAX_EXPERTS);
  FS2_REQUIRE(tile_m >= 1 && tile_m <= 1024, "dispatch: tile_m=%d", tile_m);
  FS2_REQUIRE(act_dtype == FS2MOE_F32 || act_dtype == FS2MOE_BF16, "dispatch: act_dtype %d",
              act_dtype);
  FS2_REQUIRE(max_rows >= FS2MOE_MAX_ROWS(T, K, E, tile_m),
              "dispatch: max_rows=%lld below the bound %lld", (long long)max_rows,
              (long long)FS2MOE_MAX_ROWS(T, K, E, tile_m));
  FS2_REQUIRE(max_rows < (1ll << 31), "dispatch: max_rows=%lld does not fit int32",
              (long long)max_rows);
  FS2_REQUIRE(workspace_bytes >= fs2moe_dispatch_workspace_bytes(T, K, E),
              "dispatch: workspace of %lld bytes is too small", (long long)workspace_bytes);
  const int esz = elem_size(act_dtype);
  if (xe != nullptr) {
    FS2_REQUIRE(x != nullptr, "dispatch: x is null");
    FS2_REQUIRE(D > 0 && (D * esz) % 16 == 0, "dispatch: D=%d rows are not a multiple of 16 bytes",
                D);
    FS2_REQUIRE(aligned16(x) && aligned16(xe), "dispatch: x/xe must be 16-byte aligned");
    FS2_REQUIRE(!scale_input || topk_w != nullptr, "dispatch: scale_input needs topk_w");
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int nb = (T + kDispTok - 1) / kDispTok;
  int32_t* block_counts = static_cast<int32_t*>(workspace);
  int32_t* rank = block_counts + (size_t)nb * E;

  // (the one-block forms scan the experts with a thread each: up to 256 of them)
  const bool small = nb == 1 && E <= kDispTok;
  if (small && xe == nullptr) {
    const size_t lds = dispatch_small_lds_words(E) * sizeof(uint32_t);
    const float* no_w = nullptr;
    float* no_row_w = nullptr;
    if (K <= 16)
      hipLaunchKernelGGL(dispatch_small_kernel<16>, dim3(1), dim3(kDispTok), lds, s, topk_idx, T, K,
                         E, tile_m, max_rows, counts, offsets, perm, inv_perm, no_w, no_row_w);
    else
      hipLaunchKernelGGL(dispatch_small_kernel<FS2MOE_MAX_TOP_K>, dim3(1), dim3(kDispTok), lds, s,
                         topk_idx, T, K, E, tile_m, max_rows, counts, offsets, perm, inv_perm, no_w,
                         no_row_w);
    return check_launch("dispatch_small");
  }
  if (small) {
    // (xe is given: the copying form of the same)
    const unsigned pair_blocks = (unsigned)(((int64_t)T * K + 3) / 4);
    const dim3 grid(pair_blocks + (unsigned)E), block(kDispTok);
    const size_t lds = dispatch_small_lds_words(E) * sizeof(uint32_t);
#define FS2_SMALL_COPY(TA, KC)                                                                       \
  hipLaunchKernelGGL((dispatch_small_copy_kernel<TA, KC>), grid, block, lds, s, topk_idx, topk_w,    \
                     static_cast<const TA*>(x), T, K, E, D, tile_m, scale_input, max_rows,           \
                     pair_blocks, counts, offsets, perm, inv_perm, static_cast<TA*>(xe))
    if (act_dtype == FS2MOE_F32) {
      if (K <= 16) FS2_SMALL_COPY(float, 16);
      else FS2_SMALL_COPY(float, FS2MOE_MAX_TOP_K);
    } else {
      if (K <= 16) FS2_SMALL_COPY(uint16_t, 16);
      else FS2_SMALL_COPY(uint16_t, FS2MOE_MAX_TOP_K);
    }
#undef FS2_SMALL_COPY
    return check_launch("dispatch_small_copy");
  }
  if (nb > 0) {
    const size_t lds = (size_t)E * kDispWords * 2 * sizeof(uint32_t);
    if (K <= 16)
      hipLaunchKernelGGL(dispatch_count_kernel<16>, dim3(nb), dim3(kDispTok), lds, s, topk_idx, T, K,
                         E, block_counts, rank);
    else
      hipLaunchKernelGGL(dispatch_count_kernel<FS2MOE_MAX_TOP_K>, dim3(nb), dim3(kDispTok), lds, s,
                         topk_idx, T, K, E, block_counts, rank);
    if (int rc = check_launch("dispatch_count")) return rc;
  }
  // pair blocks, then E padding blocks, then blocks for the rows beyond offsets[E] (at most
  // max_rows - T*K of them, since offsets[E] >= T*K)
  const int64_t pairs = (int64_t)T * K;
  const unsigned tail_blocks = (unsigned)((max_rows - pairs + 255) / 256);
  if (xe == nullptr && nb <= kIndexScanBlocks) {
    const unsigned pair_blocks = (unsigned)((pairs + 255) / 256);
    const size_t lds = (size_t)(4 * E + 1) * sizeof(int32_t);
    hipLaunchKernelGGL(dispatch_index_scan_kernel, dim3(pair_blocks + (unsigned)E + tail_blocks),
                       dim3(256), lds, s, topk_idx, T, K, E, tile_m, max_rows, pair_blocks,
                       block_counts, nb, rank, counts, offsets, perm, inv_perm);
    return check_launch("dispatch_index_scan");
  }
  hipLaunchKernelGGL(dispatch_scan_kernel, dim3(1), dim3(256), 0, s, block_counts, nb, E, tile_m,
                     counts, offsets);
  if (int rc = check_launch("dispatch_scan")) return rc;
  if (xe == nullptr) {
    const unsigned pair_blocks = (unsigned)((pairs + 255) / 256);
    hipLaunchKernelGGL(dispatch_index_kernel, dim3(pair_blocks + (unsigned)E + tail_blocks),
                       dim3(256), 0, s, topk_idx, T, K, E, max_rows, pair_blocks, counts, offsets,
                       block_counts, rank, perm, inv_perm);
    return check_launch("dispatch_index");
  }
  const unsigned pair_blocks = (unsigned)((pairs + 3) / 4);
  dim3 grid(pair_blocks + (unsigned)E + tail_blocks), block(256);
  if (act_dtype == FS2MOE_F32)
    hipLaunchKernelGGL(dispatch_permute_kernel<float>, grid, block, 0, s, topk_idx, topk_w,
                       static_cast<const float*>(x), T, K, E, D, scale_input, max_rows, pair_blocks,
                       counts, offsets, block_counts, rank, perm, inv_perm, static_cast<float*>(xe));
  else
    hipLaunchKernelGGL(dispatch_permute_kernel<uint16_t>, grid, block, 0, s, topk_idx, topk_w,
                       static_cast<const uint16_t*>(x), T, K, E, D, scale_input, max_rows,
                       pair_blocks, counts, offsets, block_counts, rank, perm, inv_perm,
                       static_cast<uint16_t*>(xe));
  if (int rc = check_launch("dispatch_permute")) return rc;
  return FS2MOE_OK;
}

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
#include <type_traits>

#include "common.h"
#include "tile_map.h"

namespace fs2moe {

// ---------------------------------------------------------------------------------- weight gradient
// C_e [M, N] = sum over the rows r of expert e of A[r, :M]^T B[r, :N].  A block owns a 256 x 256 tile
// of one expert's gradient and walks the expert's rows RK at a time (32 for bf16, 16 for f32).  Eight
// consumer waves multiply (a wave 128 x 64: 4 x 2 MFMA tiles); four producer waves, one per SIMD,
// move the data: a wave that waits for memory issues nothing else, so loads issued by the waves that
// multiply cost matrix-pipe time.  Both chunks go to LDS as they lie in memory (row = contraction
// index, columns contiguous) and come back through the transposing LDS read (bf16) or as single
// floats (f32), each already in MFMA operand order.  LDS holds two chunks: while one is multiplied
// the producers write the next from registers and the two after that are on their way from memory
// in two sets of registers, so there is one barrier per chunk, which orders LDS traffic only.
// (Chunks of twice the rows, a half per register set and one barrier per chunk, were slower: 277
// against 244 us on 8 experts of 8192 rows.)  Rows past the expert's count are zero-filled,
// experts without rows get a zero gradient.
namespace wgk {
constexpr int TM = 256, TN = 256, CONSUMERS = 8, PRODUCERS = 4, WAVES = CONSUMERS + PRODUCERS;
constexpr int SMEM_BYTES = 65536;  // two chunks of both operands
}
// what a load past the end of an operand reads
__device__ __attribute__((aligned(16))) uint32_t kZero16[4] = {0u, 0u, 0u, 0u};  // (not const: a global address, so the loads stay global loads)

// MAPPED: A's rows are read through a_map.  A template parameter, not a test of the pointer: behind
// a condition the map entry's load is waited for with every other load of the wave (the counter
// cannot tell them apart at the join), which serialises a chunk's loads into round trips.
template <typename T, bool MAPPED>
__global__ __launch_bounds__(wgk::WAVES * 64) void grouped_wgrad_kernel(
    const T* __restrict__ A, const int32_t* __restrict__ a_map, int lda, const T* __restrict__ B,
    int ldb, T* __restrict__ C, int M, int N, Groups g, int m_tiles, int n_tiles, int seg_rows,
    float* __restrict__ partial, int paired) {
  using namespace wgk;
  constexpr bool BF16 = sizeof(T) == 2;
  constexpr int RK = BF16 ? 32 : 16;              // rows per chunk
  constexpr int VEC = 16 / sizeof(T);             // elements per 16-byte chunk
  constexpr int ROW_CHUNKS = TM / VEC;            // 16-byte chunks per LDS row (32 or 64)
  constexpr int PLANES = PRODUCERS * 64;          // lanes that move data
  constexpr int PER_THREAD = RK * ROW_CHUNKS / PLANES;  // chunks per producer lane and operand (4)
  constexpr int ROWB = TM * sizeof(T);            // bytes per LDS row (512 or 1024)
  constexpr int OPB = RK * ROWB;                  // bytes per operand chunk (16 KB)
  static_assert(4 * OPB == SMEM_BYTES, "two chunks of two operands");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // Which tile: slots (an expert, by rank as below, or a segment of the one group's rows) in launch
  // order, and within a slot row block minor: blocks reach the 8 XCDs round-robin (block b runs on
  // XCD b % 8, each with its own L2), so with 8 row blocks the tiles of a slot that share an XCD
  // share their block of A's columns.
  const int per_e = m_tiles * n_tiles;
  int slot, mt, nt;
  if (paired) {
    // Two slots share 2 per_e consecutive blocks, i.e. (per_e being a multiple of 4) whole rounds
    // of the 8 XCDs: four XCDs per slot, each taking a quarter of the row blocks (or of the column
    // blocks) with all blocks of the other kind, so that a slot's operand slabs are fetched by 4
    // L2s with 5 slabs each instead of by 8 with 4 each.  Which half of the XCDs takes the pair's
    // larger slot alternates from pair to pair.
    const int pair = blockIdx.x / (2 * per_e);
    const int i = blockIdx.x - pair * 2 * per_e;
    const int xcd = i & 7, j = i >> 3, x4 = xcd & 3;
    slot = 2 * pair + (((xcd >> 2) ^ pair) & 1);
    if (m_tiles % 4 == 0) {
      const int q = m_tiles / 4;
      mt = x4 * q + j % q;
      nt = j / q;
    } else {
      const int q = n_tiles / 4;
      nt = x4 * q + j % q;
      mt = j / q;
    }
    if (slot >= g.E) return;  // the partner of the last of an odd number of slots
  } else {
    slot = blockIdx.x / per_e;
    const int rem = blockIdx.x - slot * per_e;
    nt = rem / m_tiles;
    mt = rem - nt * m_tiles;
  }
  const int m0 = mt * TM, n0 = nt * TN;
  const bool dense = g.counts == nullptr;
  // Grouped: the experts are taken in descending order of their row counts (ties: lower index
  // first), so that the longest chains of chunks start first and the short ones fill the end of the
  // launch.  Every block finds the expert of its rank itself: a thread per expert, one comparison loop over
  // the E counts (the block has 768 threads, the library's limit is 512 experts).
  // One group: the rows are cut into segments of seg_rows, one slot each, whose partial sums go to
  // `partial` [segments, M, N] in f32 for wgrad_reduce_kernel to add in order.
  int e = 0, off, cnt;
  if (dense) {
    off = slot * seg_rows;
    cnt = g.dense_rows - off < seg_rows ? g.dense_rows - off : seg_rows;
  } else {
    __shared__ int s_expert, s_cnt[FS2MOE_MAX_EXPERTS], s_off[FS2MOE_MAX_EXPERTS];
    const int mine = tid < g.E ? g.counts[tid] : 0;
    if (tid < g.E) {
      s_cnt[tid] = mine;
      s_off[tid] = g.offsets[tid];  // with the counts: not a second round trip once the expert is known
    }
    __syncthreads();
    if (tid < g.E) {
      int rank = 0;
      for (int j = 0; j < g.E; ++j) {
        const int cj = s_cnt[j];
        rank += (cj > mine || (cj == mine && j < tid)) ? 1 : 0;
      }
      if (rank == slot) s_expert = tid;
    }
    __syncthreads();
    e = s_expert;
    off = s_off[e];
    cnt = s_cnt[e];
  }
  const int wm = wave & 1, wn = (wave >> 1) & 3;  // a consumer's 128 (m) x 64 (n) part of the tile
  const bool producer = wave >= CONSUMERS;
  const int ptid = tid - CONSUMERS * 64;  // a producer lane's index among the PLANES
  const int lr = lane & 31, lk = lane >> 5;

  f32x16 acc[2][4];  // [tn][tm]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[a][b][i] = 0.f;

  // Loads are unconditional; what lies past the expert's rows or the matrix's columns is read from
  // 16 zero bytes instead (the address is selected, not the data: any instruction on the loaded
  // registers other than the LDS store gets scheduled early and waits for the load there).
  // Two sets of registers in the producers, so that two chunks are on their way from memory at any
  // time (one chunk's loads take about as long as its MFMAs do: with a single set every chunk waited
  // for its loads).
  u32x4 ra[2][PER_THREAD], rb[2][PER_THREAD];
  const T* zero_src = reinterpret_cast<const T*>(kZero16);
  auto load_chunk = [&](auto set_c, int r0) {
    constexpr int set = decltype(set_c)::value;
    int rr[PER_THREAD], arow[PER_THREAD];
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int r = r0 + (ptid + PLANES * i) / ROW_CHUNKS;
      rr[i] = off + (r < cnt ? r : cnt - 1);  // cnt > 0 here
      arow[i] = rr[i];
    }
    if constexpr (MAPPED) {  // all the map entries first, then all the rows
#pragma unroll
      for (int i = 0; i < PER_THREAD; ++i) arow[i] = a_map[rr[i]];
    }
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = ptid + PLANES * i;
      const int k = c / ROW_CHUNKS, ch = c % ROW_CHUNKS;
      const bool row_ok = r0 + k < cnt;
      const bool a_ok = row_ok && m0 + ch * VEC < M, b_ok = row_ok && n0 + ch * VEC < N;
      const T* pa = a_ok ? A + (size_t)arow[i] * lda + m0 + ch * VEC : zero_src;
      const T* pb = b_ok ? B + (size_t)rr[i] * ldb + n0 + ch * VEC : zero_src;
      ra[set][i] = *reinterpret_cast<const u32x4*>(pa);
      rb[set][i] = *reinterpret_cast<const u32x4*>(pb);
    }
  };
  auto store_chunk = [&](auto set_c, int buf) {
    constexpr int set = decltype(set_c)::value;
    uint8_t* sA = smem + buf * 2 * OPB;
    uint8_t* sB = sA + OPB;
#pragma unroll
    for (int i = 0; i < PER_THREAD; ++i) {
      const int c = ptid + PLANES * i;
      const int k = c / ROW_CHUNKS, ch = c % ROW_CHUNKS;
      // bf16: chunk ch of row k sits in slot ch ^ ((k & 3) << 2), so that the four consecutive rows
      // a transposing read touches lie 64 bytes apart
      const int slot = BF16 ? (ch ^ ((k & 3) << 2)) : ch;
      *reinterpret_cast<u32x4*>(sA + k * ROWB + slot * 16) = ra[set][i];
      *reinterpret_cast<u32x4*>(sB + k * ROWB + slot * 16) = rb[set][i];
    }
  };

  // bf16 fragment address of the 32 columns from cbase on, rows 8 lk .. 8 lk + 3 (+4 for the upper half)
  auto tr_addr = [&](int cbase) {
    const int s = lane & 15, half = (lane >> 4) & 1;
    const int k = lk * 8 + (s >> 2);
    const int col = cbase + half * 16 + (s & 3) * 4;
    return k * ROWB + (((col >> 3) ^ ((k & 3) << 2)) * 16) + (col & 7) * 2;
  };
  int fa[4], fb[2];
#pragma unroll
  for (int t = 0; t < 4; ++t)
    fa[t] = BF16 ? tr_addr(wm * 128 + t * 32) : (wm * 128 + t * 32 + lr) * 4;
#pragma unroll
  for (int t = 0; t < 2; ++t)
    fb[t] = BF16 ? tr_addr(wn * 64 + t * 32) : (wn * 64 + t * 32 + lr) * 4;

  auto compute_chunk = [&](int buf) {
    const uint8_t* sA = smem + buf * 2 * OPB;
    const uint8_t* sB = sA + OPB;
    if constexpr (BF16) {
#pragma unroll
      for (int ks = 0; ks < RK / 16; ++ks) {
        bf16x8 af[4], bfr[2];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint8_t* pa = sA + fa[t] + ks * 16 * ROWB;
          af[t] = lds_read_frag_tr(reinterpret_cast<const uint16_t*>(pa),
                                   reinterpret_cast<const uint16_t*>(pa + 4 * ROWB));
        }
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const uint8_t* pb = sB + fb[t] + ks * 16 * ROWB;
          bfr[t] = lds_read_frag_tr(reinterpret_cast<const uint16_t*>(pb),
                                    reinterpret_cast<const uint16_t*>(pb + 4 * ROWB));
        }
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
          for (int tm = 0; tm < 4; ++tm)
            acc[tn][tm] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
      }
    } else {
#pragma unroll 2
      for (int ks = 0; ks < RK / 2; ++ks) {
        float af[4], bfr[2];
#pragma unroll
        for (int t = 0; t < 4; ++t)
          af[t] = *reinterpret_cast<const float*>(sA + (2 * ks + lk) * ROWB + fa[t]);
#pragma unroll
        for (int t = 0; t < 2; ++t)
          bfr[t] = *reinterpret_cast<const float*>(sB + (2 * ks + lk) * ROWB + fb[t]);
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
          for (int tm = 0; tm < 4; ++tm)
            acc[tn][tm] = __builtin_amdgcn_mfma_f32_32x32x2f32(bfr[tn], af[tm], acc[tn][tm], 0, 0, 0);
      }
    }
  };

  // Chunk i is multiplied from LDS buffer i & 1 while chunk i + 1 goes from register set (i + 1) & 1
  // into the other buffer (read last during chunk i - 1: the barrier that ended it has passed), chunk
  // i + 3 is loaded into the set this frees, and chunk i + 2 is still on its way in the other set.
  const int chunks = (cnt + RK - 1) / RK;
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  // Every load and store of the loop is unconditional (chunks past the last one load clamped rows
  // and store zeros into the buffer nobody reads any more): behind a condition the compiler cannot
  // count the loads in flight, and waits for all of them, the other set's included, before a store.
  if (producer) {
    if (chunks > 0) {
      load_chunk(Set0{}, 0);
      load_chunk(Set1{}, RK);
      store_chunk(Set0{}, 0);
      load_chunk(Set0{}, 2 * RK);
      lds_barrier();
    }
    auto step = [&](int i, auto next_set) {
      store_chunk(next_set, (i + 1) & 1);
      load_chunk(next_set, (i + 3) * RK);
      lds_barrier();  // the loads of the next chunks stay in flight
    };
    int ci = 0;
    for (; ci + 1 < chunks; ci += 2) {
      step(ci, Set1{});
      step(ci + 1, Set0{});
    }
    if (ci < chunks) step(ci, Set1{});
    return;  // the consumers write the tile
  }
  if (chunks > 0) lds_barrier();
  for (int i = 0; i < chunks; ++i) {
    compute_chunk(i & 1);
    lds_barrier();
  }

  // Accumulator layout: the lane holds row m = lr of fragment tm and columns 8 q + 4 lk + {0..3} of
  // fragment tn in registers 4 q .. 4 q + 3.
  T* Ce = C + (size_t)e * M * N;
  float* Pe = partial != nullptr ? partial + (size_t)slot * M * N : nullptr;
  if constexpr (BF16) {
    if (Pe == nullptr) {
      // Through LDS (free after the loop's last barrier), so that a store instruction writes 8 rows
      // of 128 contiguous bytes instead of 32 rows of 16: the wave puts a 32 (m) x 64 (n) fragment
      // row into its own 4.25 KB as bf16, rows 136 bytes apart, and reads it back 16 bytes per lane.
      constexpr int LDE = 136;
      uint8_t* sw = smem + wave * 8192;
      const int rrow = lane >> 3, rcol = lane & 7;
#pragma unroll
      for (int tm = 0; tm < 4; ++tm) {
#pragma unroll
        for (int tn = 0; tn < 2; ++tn)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            u32x2 o = {pack_bf16x2(acc[tn][tm][4 * q], acc[tn][tm][4 * q + 1]),
                       pack_bf16x2(acc[tn][tm][4 * q + 2], acc[tn][tm][4 * q + 3])};
            *reinterpret_cast<u32x2*>(sw + lr * LDE + (tn * 32 + 8 * q + 4 * lk) * 2) = o;
          }
        // the wave's own LDS traffic runs in order; the compiler must not move the reads (other
        // lanes' data) above the writes, nor the next round's writes above these reads
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        const int n = n0 + wn * 64 + rcol * 8;
#pragma unroll
        for (int p8 = 0; p8 < 4; ++p8) {
          const int row = p8 * 8 + rrow;
          const u32x2 lo = *reinterpret_cast<const u32x2*>(sw + row * LDE + rcol * 16);
          const u32x2 hi = *reinterpret_cast<const u32x2*>(sw + row * LDE + rcol * 16 + 8);
          const int m = m0 + wm * 128 + tm * 32 + row;
          if (m < M && n < N) {  // N is a multiple of 8: the eight columns are in or out together
            u32x4 o = {lo[0], lo[1], hi[0], hi[1]};
            *reinterpret_cast<u32x4*>(Ce + (size_t)m * N + n) = o;
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
      return;
    }
  }
#pragma unroll
  for (int tm = 0; tm < 4; ++tm) {
    const int m = m0 + wm * 128 + tm * 32 + lr;
    if (m >= M) continue;
#pragma unroll
    for (int tn = 0; tn < 2; ++tn) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = n0 + wn * 64 + tn * 32 + 8 * q + 4 * lk;
        if (n >= N) continue;  // N is a multiple of 4: the four columns are in or out together
        const float v0 = acc[tn][tm][4 * q], v1 = acc[tn][tm][4 * q + 1];
        const float v2 = acc[tn][tm][4 * q + 2], v3 = acc[tn][tm][4 * q + 3];
        if (Pe != nullptr) {
          f32x4 o = {v0, v1, v2, v3};
          *reinterpret_cast<f32x4*>(Pe + (size_t)m * N + n) = o;
        } else if constexpr (BF16) {
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

// out[i] = sum over the segments, in order, of partial[s][i]; one rounding.
template <typename T>
__global__ __launch_bounds__(256) void wgrad_reduce_kernel(const float* __restrict__ partial,
                                                           int segments, int64_t n,
                                                           T* __restrict__ out) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= n) return;  // n is a multiple of 4
  f32x4 acc = *reinterpret_cast<const f32x4*>(partial + i);
  for (int s = 1; s < segments; ++s) acc += *reinterpret_cast<const f32x4*>(partial + (size_t)s * n + i);
  if constexpr (sizeof(T) == 2) {
    u32x2 o = {pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3])};
    *reinterpret_cast<u32x2*>(out + i) = o;
  } else {
    *reinterpret_cast<f32x4*>(out + i) = acc;
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
                                                       int D, int vec_ok, float* __restrict__ out) {
  const int p = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int lane = threadIdx.x & 63;
  // A pair whose expert id was out of range has no row (dispatch wrote -1 for it, and combine
  // skips it): its weight contributed nothing, so its gradient is zero.  Uniform over the wave.
  const int row = a_rows[p];
  if (row < 0) {
    if (lane == 0) out[p] = 0.f;
    return;
  }
  const size_t ar = (size_t)row * D, br = (size_t)(p / K) * D;
  float s = 0.f;
  constexpr int VEC = 16 / sizeof(T);
  if (vec_ok) {
    // 16 bytes per lane and load
    for (int d = lane * VEC; d < D; d += 64 * VEC) {
      const u32x4 av = *reinterpret_cast<const u32x4*>(a + ar + d);
      const u32x4 bv = *reinterpret_cast<const u32x4*>(b + br + d);
      u32x4 cv = {0u, 0u, 0u, 0u};
      if (a2 != nullptr) cv = *reinterpret_cast<const u32x4*>(a2 + ar + d);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (sizeof(T) == 2) {
          float x0 = __uint_as_float(av[j] << 16), x1 = __uint_as_float(av[j] & 0xffff0000u);
          if (a2 != nullptr) {
            x0 += __uint_as_float(cv[j] << 16);
            x1 += __uint_as_float(cv[j] & 0xffff0000u);
          }
          s += x0 * __uint_as_float(bv[j] << 16);
          s += x1 * __uint_as_float(bv[j] & 0xffff0000u);
        } else {
          float x0 = __uint_as_float(av[j]);
          if (a2 != nullptr) x0 += __uint_as_float(cv[j]);
          s += x0 * __uint_as_float(bv[j]);
        }
      }
    }
  } else {
    for (int d = lane; d < D; d += 64) {
      float av = Elem<T>::load(a + ar + d);
      if (a2 != nullptr) av += Elem<T>::load(a2 + ar + d);
      s += av * Elem<T>::load(b + br + d);
    }
  }
  s = wave_sum_f32(s);
  if (lane == 0) out[p] = s;
}

// ------------------------------------------------------------------- RMS normalisation backward
// y = x r w with r = rsqrt(mean(x^2) + eps) (nn/normalization.py:234-236).  With gy = dy w:
//   dx = r gy - x r^3 <gy, x> / D        dw[j] = sum_t dy[t, j] x[t, j] r_t
// One wave per row, two passes over it (the second finds the row in cache); everything in f32,
// one rounding per stored element.  The row's r goes to rstd (may be null) for the weight gradient.
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_backward_rows_kernel(
    const T* __restrict__ x, const T* __restrict__ w, float eps, const T* __restrict__ dy, int rows,
    int D, T* __restrict__ dx, float* __restrict__ rstd) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  constexpr int VEC = 16 / sizeof(T);
  const bool vec = D % VEC == 0;  // the host checks the alignment of the bases
  const float inv_d = 1.0f / (float)D;
  for (int t = blockIdx.x * 4 + wave; t < rows; t += gridDim.x * 4) {
    const T* xr = x + (size_t)t * D;
    const T* gr = dy + (size_t)t * D;
    T* outr = dx + (size_t)t * D;
    float ss = 0.f, sg = 0.f;
    if (vec) {
      for (int d = lane * VEC; d < D; d += 64 * VEC) {
        const u32x4 xv = *reinterpret_cast<const u32x4*>(xr + d);
        const u32x4 gv = *reinterpret_cast<const u32x4*>(gr + d);
        u32x4 wv = {0u, 0u, 0u, 0u};
        if (w != nullptr) wv = *reinterpret_cast<const u32x4*>(w + d);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (sizeof(T) == 2) {
            const float x0 = __uint_as_float(xv[j] << 16), x1 = __uint_as_float(xv[j] & 0xffff0000u);
            float g0 = __uint_as_float(gv[j] << 16), g1 = __uint_as_float(gv[j] & 0xffff0000u);
            if (w != nullptr) {
              g0 *= __uint_as_float(wv[j] << 16);
              g1 *= __uint_as_float(wv[j] & 0xffff0000u);
            }
            ss += x0 * x0;
            ss += x1 * x1;
            sg += g0 * x0;
            sg += g1 * x1;
          } else {
            const float x0 = __uint_as_float(xv[j]);
            float g0 = __uint_as_float(gv[j]);
            if (w != nullptr) g0 *= __uint_as_float(wv[j]);
            ss += x0 * x0;
            sg += g0 * x0;
          }
        }
      }
    } else {
      for (int d = lane; d < D; d += 64) {
        const float x0 = Elem<T>::load(xr + d);
        float g0 = Elem<T>::load(gr + d);
        if (w != nullptr) g0 *= Elem<T>::load(w + d);
        ss += x0 * x0;
        sg += g0 * x0;
      }
    }
    const float r = 1.0f / sqrtf(wave_sum_f32(ss) * inv_d + eps);
    const float c = r * r * r * wave_sum_f32(sg) * inv_d;
    if (rstd != nullptr && lane == 0) rstd[t] = r;
    if (vec) {
      for (int d = lane * VEC; d < D; d += 64 * VEC) {
        const u32x4 xv = *reinterpret_cast<const u32x4*>(xr + d);
        const u32x4 gv = *reinterpret_cast<const u32x4*>(gr + d);
        u32x4 wv = {0u, 0u, 0u, 0u};
        if (w != nullptr) wv = *reinterpret_cast<const u32x4*>(w + d);
        u32x4 ov;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (sizeof(T) == 2) {
            const float x0 = __uint_as_float(xv[j] << 16), x1 = __uint_as_float(xv[j] & 0xffff0000u);
            float g0 = __uint_as_float(gv[j] << 16), g1 = __uint_as_float(gv[j] & 0xffff0000u);
            if (w != nullptr) {
              g0 *= __uint_as_float(wv[j] << 16);
              g1 *= __uint_as_float(wv[j] & 0xffff0000u);
            }
            ov[j] = pack_bf16x2(r * g0 - x0 * c, r * g1 - x1 * c);
          } else {
            const float x0 = __uint_as_float(xv[j]);
            float g0 = __uint_as_float(gv[j]);
            if (w != nullptr) g0 *= __uint_as_float(wv[j]);
            ov[j] = __float_as_uint(r * g0 - x0 * c);
          }
        }
        *reinterpret_cast<u32x4*>(outr + d) = ov;
      }
    } else {
      for (int d = lane; d < D; d += 64) {
        const float x0 = Elem<T>::load(xr + d);
        float g0 = Elem<T>::load(gr + d);
        if (w != nullptr) g0 *= Elem<T>::load(w + d);
        Elem<T>::store(outr + d, r * g0 - x0 * c);
      }
    }
  }
}

// Weight gradient, first half: the rows are cut into gridDim.y slabs; a thread owns 16 bytes' worth
// of columns (one column when D does not divide that way) and adds up dy x r over the rows of its
// slab in ascending order.  partial [slabs][D] f32.
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_backward_weight_kernel(
    const T* __restrict__ x, const T* __restrict__ dy, const float* __restrict__ rstd, int rows,
    int D, float* __restrict__ partial) {
  constexpr int VEC = 16 / sizeof(T);
  const bool vec = D % VEC == 0;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= (vec ? D / VEC : D)) return;
  const int per = (rows + gridDim.y - 1) / gridDim.y;
  const int t0 = blockIdx.y * per;
  const int t1 = t0 + per < rows ? t0 + per : rows;
  float* out = partial + (size_t)blockIdx.y * D;
  if (vec) {
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
#pragma unroll 4
    for (int t = t0; t < t1; ++t) {
      const u32x4 xv = *reinterpret_cast<const u32x4*>(x + (size_t)t * D + c * VEC);
      const u32x4 gv = *reinterpret_cast<const u32x4*>(dy + (size_t)t * D + c * VEC);
      const float r = rstd[t];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (sizeof(T) == 2) {
          acc[2 * j] += __uint_as_float(gv[j] << 16) * __uint_as_float(xv[j] << 16) * r;
          acc[2 * j + 1] += __uint_as_float(gv[j] & 0xffff0000u) * __uint_as_float(xv[j] & 0xffff0000u) * r;
        } else {
          acc[j] += __uint_as_float(gv[j]) * __uint_as_float(xv[j]) * r;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) out[c * VEC + j] = acc[j];
  } else {
    float acc = 0.f;
    for (int t = t0; t < t1; ++t)
      acc += Elem<T>::load(dy + (size_t)t * D + c) * Elem<T>::load(x + (size_t)t * D + c) * rstd[t];
    out[c] = acc;
  }
}

// Second half: a block owns 32 columns; its eight groups of 32 threads add every eighth slab in
// ascending order, then the eight sums are added in order.  One rounding.
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_backward_weight_sum_kernel(
    const float* __restrict__ partial, int slabs, int D, T* __restrict__ dw) {
  __shared__ float s_sum[8][32];
  const int col = blockIdx.x * 32 + (threadIdx.x & 31), grp = threadIdx.x >> 5;
  float acc = 0.f;
  if (col < D) {
#pragma unroll 8
    for (int s = grp; s < slabs; s += 8) acc += partial[(size_t)s * D + col];
  }
  s_sum[grp][threadIdx.x & 31] = acc;
  __syncthreads();
  if (grp == 0 && col < D) {
    float total = 0.f;
#pragma unroll
    for (int q = 0; q < 8; ++q) total += s_sum[q][threadIdx.x];
    Elem<T>::store(dw + col, total);
  }
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
      // an id outside [0, E) selects nothing (the forward stages drop such a pair)
      const int id = topk_idx[(size_t)t * K + k];
      if (id < 0 || id >= E) continue;
      ssum += 1.0f / (1.0f + __expf(-l[id]));
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

// One group with fewer tiles than the chip has CUs: the rows are cut into this many segments.
static int wgrad_segments(int64_t rows, int M, int N) {
  const int64_t tiles = (int64_t)((M + wgk::TM - 1) / wgk::TM) * ((N + wgk::TN - 1) / wgk::TN);
  if (tiles >= 128) return 1;
  int64_t s = 256 / tiles;
  const int64_t most = rows / 256;  // at least 256 rows per segment
  s = s < most ? s : most;
  return s >= 2 ? (int)s : 1;
}

extern "C" int64_t fs2moe_grouped_wgrad_workspace_bytes(int32_t grouped, int32_t M, int32_t N,
                                                        int64_t max_rows) {
  if (M < 1 || N < 1 || max_rows < 0) return -1;
  if (grouped) return 0;
  const int s = wgrad_segments(max_rows, M, N);
  return s > 1 ? (int64_t)s * M * N * 4 : 0;
}

extern "C" int fs2moe_grouped_wgrad(const void* a, const int32_t* a_row_map, const void* b,
                                    const int32_t* counts, const int32_t* offsets, int32_t E,
                                    int32_t M, int32_t N, int64_t max_rows, int32_t dtype, void* dw,
                                    void* workspace, int64_t workspace_bytes, void* stream) {
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
  FS2_REQUIRE(aligned16(a) && aligned16(b) && aligned16(dw) && aligned16(workspace),
              "grouped_wgrad: buffers must be 16-byte aligned");
  const int m_tiles = (M + wgk::TM - 1) / wgk::TM, n_tiles = (N + wgk::TN - 1) / wgk::TN;
  // one group: segments of its rows (each a slot of the grid) when there is scratch for their sums
  int segments = 1;
  if (counts == nullptr) {
    segments = wgrad_segments(max_rows, M, N);
    if (workspace == nullptr || workspace_bytes < (int64_t)segments * M * N * 4) segments = 1;
  }
  const int slots = counts != nullptr ? E : segments;
  const int seg_rows = (int)(((max_rows + segments - 1) / segments + 15) / 16 * 16);
  float* partial = segments > 1 ? static_cast<float*>(workspace) : nullptr;
  // grouped, the tile grid divides over four XCDs, and there are enough experts for the two halves
  // of the XCDs to get the same work over all pairs (with 8 skewed experts they did not: Mixtral's
  // gradients took 9 % longer): slots in pairs (see the kernel)
  const int paired = counts != nullptr && E >= 32 && (m_tiles % 4 == 0 || n_tiles % 4 == 0) ? 1 : 0;
  const int64_t blocks = (int64_t)(paired ? (slots + 1) / 2 * 2 : slots) * m_tiles * n_tiles;
  FS2_REQUIRE(blocks <= 0x7fffffffll, "grouped_wgrad: too many tiles");
  Groups g{counts, offsets, E, (int)max_rows};
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool mapped = a_row_map != nullptr;
  auto kb = mapped ? grouped_wgrad_kernel<uint16_t, true> : grouped_wgrad_kernel<uint16_t, false>;
  auto kf = mapped ? grouped_wgrad_kernel<float, true> : grouped_wgrad_kernel<float, false>;
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    const void* ks[4] = {reinterpret_cast<const void*>(grouped_wgrad_kernel<uint16_t, false>),
                         reinterpret_cast<const void*>(grouped_wgrad_kernel<uint16_t, true>),
                         reinterpret_cast<const void*>(grouped_wgrad_kernel<float, false>),
                         reinterpret_cast<const void*>(grouped_wgrad_kernel<float, true>)};
    for (const void* k : ks) {
      hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, wgk::SMEM_BYTES);
      if (e != hipSuccess) {
        set_error("grouped_wgrad: cannot reserve %d bytes of LDS: %s", wgk::SMEM_BYTES,
                  hipGetErrorString(e));
        return FS2MOE_ERR_LAUNCH;
      }
    }
    attr_set = true;
  }
  if (dtype == FS2MOE_BF16)
    hipLaunchKernelGGL(kb, dim3((unsigned)blocks), dim3(wgk::WAVES * 64), wgk::SMEM_BYTES, st,
                       static_cast<const uint16_t*>(a), a_row_map, M,
                       static_cast<const uint16_t*>(b), N, static_cast<uint16_t*>(dw), M, N, g,
                       m_tiles, n_tiles, seg_rows, partial, paired);
  else
    hipLaunchKernelGGL(kf, dim3((unsigned)blocks), dim3(wgk::WAVES * 64), wgk::SMEM_BYTES, st,
                       static_cast<const float*>(a), a_row_map, M, static_cast<const float*>(b), N,
                       static_cast<float*>(dw), M, N, g, m_tiles, n_tiles, seg_rows, partial, paired);
  if (int rc = check_launch("grouped_wgrad")) return rc;
  if (segments > 1) {
    const int64_t n = (int64_t)M * N;
    const unsigned rblocks = (unsigned)((n / 4 + 255) / 256);
    if (dtype == FS2MOE_BF16)
      hipLaunchKernelGGL(wgrad_reduce_kernel<uint16_t>, dim3(rblocks), dim3(256), 0, st, partial,
                         segments, n, static_cast<uint16_t*>(dw));
    else
      hipLaunchKernelGGL(wgrad_reduce_kernel<float>, dim3(rblocks), dim3(256), 0, st, partial,
                         segments, n, static_cast<float*>(dw));
    return check_launch("wgrad_reduce");
  }
  return FS2MOE_OK;
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
  // 16-byte loads need rows that start on 16 bytes: D a multiple of the vector and aligned bases
  const int vec = 16 / elem_size(dtype);
  const int vec_ok = D % vec == 0 && aligned16(a) && aligned16(b) && (a2 == nullptr || aligned16(a2));
  if (dtype == FS2MOE_BF16)
    hipLaunchKernelGGL(pair_dot_kernel<uint16_t>, dim3(blocks), dim3(256), 0, st,
                       static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(a2), a_rows,
                       static_cast<const uint16_t*>(b), (int)pairs, K, D, vec_ok, out);
  else
    hipLaunchKernelGGL(pair_dot_kernel<float>, dim3(blocks), dim3(256), 0, st,
                       static_cast<const float*>(a), static_cast<const float*>(a2), a_rows,
                       static_cast<const float*>(b), (int)pairs, K, D, vec_ok, out);
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

// slabs of rows for the weight gradient of the normalisation: at least 32 rows each, at most 256
static int norm_weight_slabs(int64_t rows) {
  const int64_t s = rows / 32;
  return s < 1 ? 1 : (s > 256 ? 256 : (int)s);
}

extern "C" int64_t fs2moe_rms_norm_backward_workspace_bytes(int32_t T, int32_t D) {
  if (T < 0 || D < 1) return -1;
  // rstd [T] (padded to 16 bytes), then the slabs' partial sums
  return ((int64_t)T * 4 + 15) / 16 * 16 + (int64_t)norm_weight_slabs(T) * D * 4;
}

extern "C" int fs2moe_rms_norm_backward(const void* x, const void* weight, float eps,
                                        const void* dy, int32_t T, int32_t D, int32_t dtype,
                                        void* dx, void* dweight, void* workspace,
                                        int64_t workspace_bytes, void* stream) {
  FS2_REQUIRE(x && dy && dx, "rms_norm_backward: null pointer");
  FS2_REQUIRE(dtype == FS2MOE_F32 || dtype == FS2MOE_BF16, "rms_norm_backward: dtype %d", dtype);
  FS2_REQUIRE(T >= 0 && D > 0, "rms_norm_backward: T=%d, D=%d", T, D);
  FS2_REQUIRE(dweight == nullptr || weight != nullptr,
              "rms_norm_backward: a weight gradient without a weight");
  FS2_REQUIRE(dx != dy && dx != x, "rms_norm_backward: dx must not alias x or dy");
  FS2_REQUIRE(aligned16(x) && aligned16(dy) && aligned16(dx) && aligned16(weight) &&
                  aligned16(workspace),
              "rms_norm_backward: buffers must be 16-byte aligned");
  hipStream_t st = static_cast<hipStream_t>(stream);
  float* rstd = nullptr;
  float* partial = nullptr;
  if (dweight != nullptr) {
    FS2_REQUIRE(workspace != nullptr &&
                    workspace_bytes >= fs2moe_rms_norm_backward_workspace_bytes(T, D),
                "rms_norm_backward: the weight gradient needs a workspace of %lld bytes",
                (long long)fs2moe_rms_norm_backward_workspace_bytes(T, D));
    rstd = static_cast<float*>(workspace);
    partial = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) +
                                       ((int64_t)T * 4 + 15) / 16 * 16);
  }
  if (T > 0) {
    int blocks = (T + 3) / 4;
    if (blocks > 4096) blocks = 4096;
    if (dtype == FS2MOE_BF16)
      hipLaunchKernelGGL(rms_norm_backward_rows_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256),
                         0, st, static_cast<const uint16_t*>(x),
                         static_cast<const uint16_t*>(weight), eps,
                         static_cast<const uint16_t*>(dy), T, D, static_cast<uint16_t*>(dx), rstd);
    else
      hipLaunchKernelGGL(rms_norm_backward_rows_kernel<float>, dim3((unsigned)blocks), dim3(256), 0,
                         st, static_cast<const float*>(x), static_cast<const float*>(weight), eps,
                         static_cast<const float*>(dy), T, D, static_cast<float*>(dx), rstd);
    if (int rc = check_launch("rms_norm_backward")) return rc;
  }
  if (dweight == nullptr) return FS2MOE_OK;
  // (with no rows the one slab sums nothing and the gradient is zero)
  const int slabs = norm_weight_slabs(T);
  const int vec = dtype == FS2MOE_BF16 ? 8 : 4;
  const int owners = D % vec == 0 ? D / vec : D;  // threads per slab
  const dim3 grid((unsigned)((owners + 255) / 256), (unsigned)slabs);
  const unsigned sum_blocks = (unsigned)((D + 31) / 32);
  if (dtype == FS2MOE_BF16) {
    hipLaunchKernelGGL(rms_norm_backward_weight_kernel<uint16_t>, grid, dim3(256), 0, st,
                       static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(dy), rstd, T, D,
                       partial);
    hipLaunchKernelGGL(rms_norm_backward_weight_sum_kernel<uint16_t>, dim3(sum_blocks), dim3(256), 0, st,
                       partial, slabs, D, static_cast<uint16_t*>(dweight));
  } else {
    hipLaunchKernelGGL(rms_norm_backward_weight_kernel<float>, grid, dim3(256), 0, st,
                       static_cast<const float*>(x), static_cast<const float*>(dy), rstd, T, D,
                       partial);
    hipLaunchKernelGGL(rms_norm_backward_weight_sum_kernel<float>, dim3(sum_blocks), dim3(256), 0, st,
                       partial, slabs, D, static_cast<float*>(dweight));
  }
  return check_launch("rms_norm_backward (weight)");
}

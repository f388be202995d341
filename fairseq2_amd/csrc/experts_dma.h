// bf16 grouped GEMM, throughput kernel: persistent blocks, 256-row tiles, producer and consumer waves.
//
// Tile shape.  A block owns 256 rows x 256 "virtual" channels (128 gate + the same 128 up channels
// when DUAL, else 256 channels).  Its 8 consumer waves form a 4 (rows) x 2 (channels) grid; each owns
// 64 x 128, i.e. 2 x 4 MFMA 32x32x16 tiles = 128 accumulator registers, two consumers per SIMD.
//
// Specialisation.  Four more waves (one per SIMD) are producers: they only move data from global
// memory to LDS.  A wave that waits for memory issues nothing else (waves issue in order), so loads
// issued by the consumers would cost matrix-pipe time; issued by producers, they overlap the
// consumers' MFMAs.
//
// Persistence.  One block per CU walks a list of output tiles, dealt out so that every block gets
// the same amount of work and the blocks of an XCD work on neighbouring tiles (see the tile tables
// below).  The tile -> (expert, rows) map comes from counts/offsets, copied to LDS once; nothing is
// read back to the host.  Tiles that would make up a last round of a few whole tiles are dealt as
// halves (128 rows) when that lets the round end in a light tile's time.
//
// Pipeline.  K is walked in units of 64: a unit is a 256 x 64 activation block (128-byte rows: a
// 64-byte piece of a row would make the L1 fetch every 128-byte line twice and halve the fill rate)
// and two 32 x 256 weight sub-stages, 64 KB in all, and LDS holds two units.  The units of all of a
// block's tiles form ONE stream: loads run ahead of the MFMAs straight across tile boundaries, so a
// tile's epilogue overlaps the next tile's first loads.  A unit travels global -> registers -> LDS:
//     producer, unit u:  barrier;  register by register: write the piece of unit u+1 it holds into
//                        the other half (read last in unit u-1), load unit u+2's piece into it
//     consumer, unit u:  barrier;  fragments from half u % 2;  32 MFMAs
// One barrier per 64 k rather than per 32 k: after a barrier every consumer starts with LDS reads
// whose latency nothing hides (both waves of a SIMD are at the same point), and that cost is per
// barrier.  (Direct global->LDS loads would save the registers and the LDS writes, but in this
// kernel four producers get 24 bytes per cycle out of them; loads into registers reach about three
// times that.)
//
// What bounds it.  Per unit two chains of about the same length meet at the barrier: the consumers'
// 2048 clocks of MFMAs, and a producer's 16 LDS stores (a 1 KB ds_write_b128 takes a wave about 80
// clocks while the consumers read: 4 x 1 KB / 80 = 51 B/clk) and 16 loads (about 40 clocks each),
// which as two phases took 1659 + 627 clocks and interleaved take about 2050; around the barrier
// another 700 go by (the consumers' first fragment reads, the spread of twelve waves' arrival).
// Measured and not kept, each within a few percent either way: a second register set (two units in
// flight), per-wave LDS progress counters instead of the block barrier, direct global -> LDS loads
// (about 170 clocks to issue each in this kernel), units of 128 k or two units in flight for tiles
// of a few rows, consumer waves of 128 x 64, hand-pipelined and assembly consumer loops.  Under it
// all the clock: the part holds 1.7-1.9 GHz with these operands, 2.4 with all-zero ones.
//
// LDS layout.  A wave writes its piece as one contiguous 1 KB, so rows are not padded; bank
// conflicts are avoided by choosing WHICH global chunk each lane fetches (an XOR swizzle of the
// chunk index):
//   * activation blocks: rows of 8 chunks (128 B); chunk kc of row r sits in slot
//     kc ^ ((r >> 1) & 7), so the 16 rows a 16-byte fragment read touches spread over all banks;
//   * n-contiguous weight tiles (one 32 x 128 sub-tile per matrix when DUAL, else 32 x 256): chunk c
//     of k-row k sits in slot c ^ ((k & 3) << 2), so the 4 consecutive k rows a transposing read
//     touches land 64 B apart.
#pragma once

#include "common.h"
#include "tile_map.h"

namespace fs2moe {
namespace dma {
constexpr int BM = 256, BK = 32, BNV = 256;
constexpr int CONSUMERS = 8, PRODUCERS = 4, NWAVES = CONSUMERS + PRODUCERS;
constexpr int A_BYTES = BM * 2 * BK * 2;  // 32 KB: 256 rows x 64 k
constexpr int B_BYTES = BK * BNV * 2;     // 16 KB: one weight sub-stage of 32 k
constexpr int UNIT_BYTES = A_BYTES + 2 * B_BYTES;  // 64 KB
constexpr int RING_BYTES = 2 * UNIT_BYTES;         // 128 KB
#ifndef FS2MOE_GEMM_BAND
#define FS2MOE_GEMM_BAND 8
#endif
constexpr int BAND = FS2MOE_GEMM_BAND;  // row blocks per band of the tile order (see locate)
constexpr int LIGHT_ROWS = 128;  // a last tile of at most this many rows costs about half a tile
// after the ring: heavy-tile prefix [E + 1], light-tile prefix [E + 1], counts [E], offsets [E], each
// sized for the library's limit on E
constexpr int TABLE_INTS = 4 * FS2MOE_MAX_EXPERTS + 8;
// then, for e4m3 weights, the per-channel scales of two tiles (the one being multiplied and the one
// whose loads are under way): [2][256] f32
constexpr int SCALE_BYTES = 2 * BNV * 4;
constexpr int SMEM_BYTES = RING_BYTES + TABLE_INTS * 4 + SCALE_BYTES;
// A third weight layout next to FS2MOE_W_IN_OUT / FS2MOE_W_OUT_IN: e4m3 codes in 1 KB tiles of 16
// output channels x 64 in-features, [expert][channel / 16][feature / 64][16][64], with one f32 scale
// per output channel (the layout of the decode kernel in experts_fp8.h).
constexpr int W_FP8_TILED = 2;
}  // namespace dma

// Which of a 1 KB e4m3 weight tile's 16 channel rows lane l of a producer takes (it takes the 16
// codes at k 16 (l % 4) of that row; four lanes a row, so the loads of a wave still cover the tile
// as 16 whole 64-byte rows).  The rows are dealt so that the wave's LDS stores are free of bank
// conflicts: a store instruction is served eight lanes at a time, and the two rows of eight lanes must
// differ in the swizzle key's lowest bit (rows r and r + 2), since both write the even (then the
// odd) chunks.  Lane order l / 4 put rows r and r + 1 (same key) there: 8.0 instead of 6.5 clocks
// per store instruction in a probe of all 720 assignments of lane bits to row and chunk bits.
__device__ __forceinline__ int fp8_tile_row(int lane) {
  return (((lane >> 2) & 1) << 1) | ((lane >> 3) & 1) | (((lane >> 4) & 3) << 2);
}

// The order in which a block walks its tiles: its light tiles spread evenly among its heavy ones,
// the pattern rotated by the block's XCD.  Light tiles of small experts stream their weights from
// HBM and leave the matrix pipe half idle; heavy tiles mostly hit L2 and are bound by the matrix
// pipe.  Walking the list front to back would make every CU stream from HBM at the same time at the
// end; this way the XCDs do so at different times, while the 32 blocks of one XCD stay on
// neighbouring tiles of the list (same round of the deal) and keep sharing their operands in L2.
// next() returns the index, in list order, of the block's next tile.  Every wave of a block
// steps its own copy; the sequence depends on the constructor arguments only.
struct TileOrder {
  int heavy, light, n, u, h_done, l_done;
  __device__ TileOrder(int heavy_, int light_, int xcd)
      : heavy(heavy_), light(light_), n(heavy_ + light_), u(xcd * (heavy_ + light_) / 8),
        h_done(0), l_done(0) {}
  __device__ int next() {
    // position u of the pattern is light iff floor((u + 1) light / n) > floor(u light / n)
    bool is_light = ((u + 1) * light) / n != (u * light) / n;
    if (is_light && l_done == light) is_light = false;
    if (!is_light && h_done == heavy) is_light = true;
    u = u + 1 == n ? 0 : u + 1;
    return is_light ? heavy + l_done++ : h_done++;
  }
};

// row_map (may be null): activation row r is read from A[row_map[r]] instead of A[r]; C rows are
// never mapped.
// BLAYOUT: FS2MOE_W_IN_OUT -- weights (Kdim, N) with N contiguous (the grouped experts), or
// FS2MOE_W_OUT_IN -- weights (N, Kdim) with Kdim contiguous (nn.Linear: the shared expert).  In the
// second case a unit's weights are, like its activations, 256 rows (channels) of 128 bytes: same
// pieces, same swizzle, same plain 16-byte fragment reads.  dma::W_FP8_TILED -- e4m3 codes (B0, B1
// point at bytes) with scales S0, S1 [E, N]: a unit's weights are 16 tiles of 1 KB, half the bytes
// of bf16; the producers turn the codes into bf16 in registers (exact) on the way to LDS and lay
// them out as in the second case, so the consumers' main loop is the same, and the scales multiply
// the f32 accumulators in the epilogue.
// KEEP_GU (with DUAL, bf16 weights): the epilogue also stores the two products themselves, rounded
// to bf16 and laid out like C, for a backward pass that would otherwise compute them again.  Their
// destinations arrive in S0 and S1, which bf16 weights leave unused: two more arguments cost every
// other variant of the kernel registers in its main loop (1-2.5 % of the layer, measured).
// TWO_SRC (single matrix, (out, in) bf16 weights): C = A @ B0_e^T + A2 @ B1_e^T, the second pair
// walked after the first into the same accumulators (Kdim is one pair's).  A2 arrives in S0, for the
// reason given above.
template <bool DUAL, int BLAYOUT, bool KEEP_GU = false, bool TWO_SRC = false>
__global__ __launch_bounds__(dma::NWAVES * 64) void glu_gemm_bf16_dma_kernel(
    const uint16_t* __restrict__ A, const int32_t* __restrict__ row_map, int lda,
    const uint16_t* __restrict__ B0, const uint16_t* __restrict__ B1,
    const float* __restrict__ S0, const float* __restrict__ S1, uint16_t* __restrict__ C, int ldc,
    int Kdim, int N, Groups g, int n_tiles) {
  using namespace dma;
  constexpr bool FP8 = BLAYOUT == W_FP8_TILED;
  static_assert(!KEEP_GU || (DUAL && !FP8), "the products are kept by the bf16 gate/up kernel only");
  static_assert(!TWO_SRC || (!DUAL && BLAYOUT == FS2MOE_W_OUT_IN), "two sources: one (out, in) matrix each");
  constexpr int BN = DUAL ? 128 : 256;    // real channels per tile
  constexpr int BROW = DUAL ? 256 : 512;  // bytes per LDS row of a weight sub-tile (in x out)
  constexpr bool KN = BLAYOUT == FS2MOE_W_IN_OUT;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  int32_t* s_hstart = reinterpret_cast<int32_t*>(smem_raw + RING_BYTES);  // [E + 1]
  int32_t* s_lstart = s_hstart + FS2MOE_MAX_EXPERTS + 4;                  // [E + 1]
  int32_t* s_counts = s_lstart + FS2MOE_MAX_EXPERTS + 4;
  int32_t* s_offsets = s_counts + FS2MOE_MAX_EXPERTS;
  float* s_scale = reinterpret_cast<float*>(smem_raw + RING_BYTES + TABLE_INTS * 4);  // [2][BNV]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: lives in a scalar register
  // Consumers w, w + 4 share a SIMD; rows go to w >> 1 so that a tile of up to 128 rows keeps one
  // wave per SIMD busy instead of two waves on half of the SIMDs.
  const int wm = (wave >> 1) & 3, wn = wave & 1;
  const int lr = lane & 31, lk = lane >> 5;

  // ---- tile tables (once per block) ------------------------------------------------------------
  const bool dense = g.counts == nullptr;
  const int E = dense ? 1 : g.E;
  // An expert's tiles are "heavy" (256 rows, or a last tile of more than LIGHT_ROWS rows) or "light"
  // (a last tile of at most LIGHT_ROWS rows, which keeps one consumer wave per SIMD busy instead of
  // two and so takes about half the time).  Tiles are listed heavy first (expert-major, n-tile
  // minor), then light, and dealt out round-robin: tile i goes to slot i % gridDim.x, where slots
  // 32 c .. 32 c + 31 are the blocks of XCD c (block b runs on XCD b % 8, each XCD has its own L2).
  // Every block then gets the same number of heavy tiles to within one, the light tiles fill up the
  // blocks that got one heavy tile fewer, and the 32 tiles in flight on an XCD are neighbours in the
  // list, which share activation rows (same rows, next channels) and weights (same expert).
  {
    __shared__ int s_wave_tot[2][NWAVES];
    const int cnt = dense ? (tid == 0 ? g.dense_rows : 0) : (tid < E ? g.counts[tid] : 0);
    const int rem = cnt % BM;
    const int heavy = cnt / BM + (rem > LIGHT_ROWS ? 1 : 0);
    const int light = (rem > 0 && rem <= LIGHT_ROWS) ? 1 : 0;
    int hincl = heavy, lincl = light;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const int hv = __shfl_up(hincl, off, kWave), lv = __shfl_up(lincl, off, kWave);
      if (lane >= off) {
        hincl += hv;
        lincl += lv;
      }
    }
    if (lane == 63) {
      s_wave_tot[0][wave] = hincl;
      s_wave_tot[1][wave] = lincl;
    }
    __syncthreads();
    int hbase = 0, lbase = 0;
    for (int w = 0; w < wave; ++w) {
      hbase += s_wave_tot[0][w];
      lbase += s_wave_tot[1][w];
    }
    if (tid < E) {
      s_hstart[tid] = hbase + hincl - heavy;
      s_lstart[tid] = lbase + lincl - light;
      s_counts[tid] = cnt;
      s_offsets[tid] = dense ? 0 : g.offsets[tid];
    }
    if (tid == E - 1) {
      s_hstart[E] = hbase + hincl;
      s_lstart[E] = lbase + lincl;
    }
    __syncthreads();
  }
  // The host guarantees that the number of tiles fits 31 bits.
  const int total_heavy = s_hstart[E];
  const int slot = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int grid = (int)gridDim.x;
  // The heavy tiles that do not fill a round of the deal (one tile per block) would hold their
  // blocks for a whole tile's time while the others idle.  When both halves of each of them and all
  // light tiles fit ONE round, they are dealt as halves of 128 rows (rows 0..127 and 128..255 of the
  // tile, each a light tile's work): the last round then takes a light tile's time.  Every output
  // element is still the same sum in the same order.
  const int all_heavy = total_heavy * n_tiles;
  const int lights = s_lstart[E] * n_tiles;
  const int rest = all_heavy % grid;
  const int split = 2 * rest + lights <= grid ? rest : 0;
  // list order: heavy tiles [0, heavy_end), halves [heavy_end, halves_end), light tiles after that
  const int heavy_end = all_heavy - split;
  const int halves_end = heavy_end + 2 * split;
  const int real = halves_end + lights;
  const int my_tiles = slot < real ? (real - slot + grid - 1) / grid : 0;
  if (my_tiles == 0) return;
  // of which heavy: the block's j-th tile (in list order) is heavy for j < my_heavy
  const int my_heavy = slot < heavy_end ? (heavy_end - slot + grid - 1) / grid : 0;

  // units per tile; the host guarantees Kdim % 64 == 0
  const int nu = (TWO_SRC ? 2 : 1) * (Kdim / (2 * BK));
  const int total_units = my_tiles * nu;

  // Wave-uniform parameters of a tile: expert, first row, end row, first channel.
  struct Tile {
    int e, row0, row_end, n0;
  };
  auto locate = [&](int j) {
    const int listed = slot + j * grid;
    const bool is_light = listed >= halves_end;
    // a half names its heavy tile: the halves of heavy tile heavy_end + i are listed at
    // heavy_end + 2 i and + 2 i + 1
    const int half = (listed >= heavy_end && !is_light) ? ((listed - heavy_end) & 1) : -1;
    const int logical = half >= 0 ? heavy_end + ((listed - heavy_end) >> 1) : listed;
    const int in_kind = is_light ? listed - halves_end : logical;
    int mt = in_kind / n_tiles;  // m-tile in list order: which expert
    const int32_t* start = is_light ? s_lstart : s_hstart;
    int found = 0;
    for (int e0 = 0; e0 < E; e0 += 64) {
      const int e = e0 + lane;
      const bool hit = e < E && start[e] <= mt && mt < start[e + 1];
      const unsigned long long m = __ballot(hit);
      if (m) found = e0 + (int)__builtin_ctzll(m);
    }
    found = __builtin_amdgcn_readfirstlane(found);
    const int off = s_offsets[found], cnt = s_counts[found];
    int nt, first_row;
    if (is_light) {
      nt = in_kind - mt * n_tiles;
      first_row = cnt / BM * BM;
    } else {
      // Inside an expert the heavy tiles are numbered in bands of BAND row blocks, row block minor
      // within a band: the 32 neighbouring tiles an XCD works on at a time then cover BAND row blocks
      // x 32 / BAND channel blocks and find both operands in its L2 (8 + 4 slabs for 32 tiles).
      // Channel block minor, an XCD would hold one row block x 32 channel blocks, whose weight slabs
      // nobody else on the XCD reads: with wide layers every tile then streams its weights from
      // memory and the kernel is bound by that.
      const int h0 = s_hstart[found];
      const int l = logical - h0 * n_tiles;
      const int per_band = BAND * n_tiles;
      const int b = l / per_band, t = l - b * per_band;
      const int left = s_hstart[found + 1] - h0 - b * BAND;
      const int gm = left < BAND ? left : BAND;
      nt = t / gm;
      first_row = (b * BAND + t - nt * gm) * BM;
    }
    int last_row = cnt;
    if (half >= 0) {
      first_row += half * LIGHT_ROWS;
      last_row = last_row < first_row + LIGHT_ROWS ? last_row : first_row + LIGHT_ROWS;
    }
    Tile t;
    t.e = found;
    t.row0 = __builtin_amdgcn_readfirstlane(off + first_row);
    t.row_end = __builtin_amdgcn_readfirstlane(off + last_row);
    t.n0 = __builtin_amdgcn_readfirstlane(nt) * BN;
    return t;
  };

  const size_t wstride = (size_t)Kdim * N;

  if (wave >= CONSUMERS) {
    // ---- producer: the load stream ----------------------------------------------------------------
    // An activation block is 32 pieces of 1 KB (8 rows x 128 B), a weight sub-stage 16 pieces;
    // producer q moves pieces q, q+4, q+8, ... of a unit: 16 loads of 16 bytes per lane into 16
    // different registers (loads into ONE register would be serialised by the hardware, two in flight
    // at most), later 16 LDS writes of a contiguous 1 KB each.  Every weight piece reads one matrix
    // only: with DUAL a sub-stage holds a gate sub-tile (pieces 0..7) followed by an up sub-tile
    // (pieces 8..15).  The registers are the third stage of the pipeline: unit u+2 is on its way from
    // memory while unit u+1 sits in LDS and unit u is being multiplied.
    const int q = wave - CONSUMERS;
    uint32_t pa[8], pb[(KN || FP8) ? 4 : 8];
    int a_pieces = 0;  // how many of this producer's 8 activation pieces hold rows of the tile
    const uint16_t* ld_bg = B0;
    const uint16_t* ld_bu = B0;
    // e4m3 weights: the scale of virtual channel 64 q + lane of the tile set up last, and which of
    // the two LDS slots it goes to (tiles alternate)
    float ld_scale = 0.f;
    int ld_tiles = 0;
    // The tile after the one set up last, looked up a tile ahead: which tile it is, and (fused
    // gather) the tokens its rows are read from.  Those come out of row_map, a load that the tile's
    // own loads depend on; asked for when the tile before it is set up, they have long arrived when
    // the tile's turn comes, and its first unit goes out without a round trip to memory in front.
    Tile pre_t = {0, 0, 0, 0};
    int pre_rows[8];
    auto lookup_ahead = [&](int j) {
      pre_t = locate(j);
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const int row = 8 * (q + 4 * jj) + (lane >> 3);
        int grow = pre_t.row0 + row;
        grow = grow < pre_t.row_end ? grow : pre_t.row_end - 1;  // clamped rows are never stored
        // fused gather: logical row r of the activations is row row_map[r] of A (rows below row_end
        // are real pairs, so their map entries are tokens, never the -1 of padding)
        pre_rows[jj] = row_map != nullptr ? row_map[grow] : grow;
      }
    };
    auto setup_loads = [&]() {
      const Tile t = pre_t;
      if constexpr (FP8) {
        // wstride counts codes = bytes here; the pointers stay typed as 16-bit
        ld_bg = reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(B0) +
                                                  (size_t)t.e * wstride);
        ld_bu = DUAL ? reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(B1) +
                                                         (size_t)t.e * wstride)
                     : ld_bg;
        const int v = 64 * q + lane;  // virtual channel of the tile: gate 0..127, up 128..255
        const bool up = DUAL && v >= 128;
        int ch = t.n0 + (up ? v - 128 : v);
        ch = ch < N ? ch : N - 1;  // clamped channels are never stored
        ld_scale = (up ? S1 : S0)[(size_t)t.e * N + ch];
        ++ld_tiles;
      } else {
        ld_bg = B0 + (size_t)t.e * wstride;
        ld_bu = (DUAL || TWO_SRC) ? B1 + (size_t)t.e * wstride : ld_bg;
      }
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const int p = q + 4 * jj;
        const int row = 8 * p + (lane >> 3), slot = lane & 7;
        const int kc = slot ^ ((row >> 1) & 7);
        pa[jj] = (uint32_t)(((size_t)pre_rows[jj] * lda + kc * 8) * 2);
      }
      // piece p holds rows 8p .. 8p+7; pieces past the tile's last row are not loaded (the consumer
      // waves that would read them are idle)
      const int rows = t.row_end - t.row0;
      a_pieces = rows >= BM ? 8 : (rows - 8 * q + 31) / 32;
      a_pieces = a_pieces < 0 ? 0 : a_pieces;
      if constexpr (FP8) {
        // a unit's weights are the 16 tiles (channel group gi = q + 4 jj of the 256 virtual channels,
        // k block ku); with DUAL groups 0..7 are gate channels and 8..15 the same up channels
        const int nkb = Kdim / (2 * BK);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int gi = q + 4 * jj;
          int group = t.n0 / 16 + (DUAL ? (gi & 7) : gi);
          group = group < N / 16 ? group : N / 16 - 1;  // clamped channels are never stored
          pb[jj] = (uint32_t)(((size_t)group * nkb) * 1024 + fp8_tile_row(lane) * 64 + (lane & 3) * 16);
        }
      } else if constexpr (KN) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          // piece r of a sub-tile = 1024 / BROW consecutive k rows
          constexpr int ROWS = 1024 / BROW, CHUNKS = BROW / 16;
          const int p = q + 4 * jj;
          const int r = DUAL ? (p & 7) : p;
          const int k = ROWS * r + lane / CHUNKS, slot = lane % CHUNKS;
          int col = t.n0 + (slot ^ ((k & 3) << 2)) * 8;
          col = col < N ? col : N - 8;  // clamped channels are never stored
          pb[jj] = (uint32_t)(((size_t)k * N + col) * 2);
        }
      } else {
        // 32 pieces of 8 channel rows x 128 B; with DUAL rows 0..127 are gate channels and rows
        // 128..255 the same up channels, so pieces 0..15 read one matrix and 16..31 the other
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          const int p = q + 4 * jj;
          const int row = 8 * p + (lane >> 3), slot = lane & 7;
          const int kc = slot ^ ((row >> 1) & 7);
          int ch = t.n0 + (DUAL ? (row & 127) : row);
          ch = ch < N ? ch : N - 1;  // clamped channels are never stored
          pb[jj] = (uint32_t)(((size_t)ch * Kdim + kc * 8) * 2);
        }
      }
    };
    u32x4 stage[FP8 ? 12 : 16];
    int stage_pieces = 0;  // a_pieces of the unit held in `stage`
    int stage_scale_slot = -1;  // e4m3: the unit in `stage` is the first of a tile with this slot
    float stage_scale = 0.f;
    // Unit ku of the tile set up last -> registers.
    auto load_unit = [&](int ku) {
      // with two sources the second half of a tile's units comes from the second pair
      const bool second = TWO_SRC && ku >= nu / 2;
      if constexpr (TWO_SRC) ku = second ? ku - nu / 2 : ku;
      const uint16_t* a_src = second ? reinterpret_cast<const uint16_t*>(S0) : A;
      const uint8_t* abase = reinterpret_cast<const uint8_t*>(a_src + (size_t)ku * (2 * BK));
#pragma unroll
      for (int jj = 0; jj < 8; ++jj)
        if (jj < a_pieces) stage[jj] = *reinterpret_cast<const u32x4*>(abase + pa[jj]);
      if constexpr (FP8) {
        const uint8_t* bg = reinterpret_cast<const uint8_t*>(ld_bg) + (size_t)ku * 1024;
        const uint8_t* bu = reinterpret_cast<const uint8_t*>(ld_bu) + (size_t)ku * 1024;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
          stage[8 + jj] = *reinterpret_cast<const u32x4*>((jj < 2 ? bg : bu) + pb[jj]);
        stage_scale_slot = ku == 0 ? ((ld_tiles - 1) & 1) : -1;
        stage_scale = ld_scale;
      } else if constexpr (KN) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const size_t k0 = ((size_t)ku * 2 + h) * BK * N;
          const uint8_t* bg = reinterpret_cast<const uint8_t*>(ld_bg + k0);
          const uint8_t* bu = reinterpret_cast<const uint8_t*>(ld_bu + k0);
          // pieces q, q+4 (gate when DUAL) and q+8, q+12 (up when DUAL)
          stage[8 + 4 * h + 0] = *reinterpret_cast<const u32x4*>(bg + pb[0]);
          stage[8 + 4 * h + 1] = *reinterpret_cast<const u32x4*>(bg + pb[1]);
          stage[8 + 4 * h + 2] = *reinterpret_cast<const u32x4*>(bu + pb[2]);
          stage[8 + 4 * h + 3] = *reinterpret_cast<const u32x4*>(bu + pb[3]);
        }
      } else {
        const uint8_t* bg =
            reinterpret_cast<const uint8_t*>((second ? ld_bu : ld_bg) + (size_t)ku * (2 * BK));
        const uint8_t* bu =
            TWO_SRC ? bg : reinterpret_cast<const uint8_t*>(ld_bu + (size_t)ku * (2 * BK));
        // pieces q + 4 jj: jj < 4 lie in rows 0..127 (gate when DUAL), the rest in rows 128..255
#pragma unroll
        for (int jj = 0; jj < 8; ++jj)
          stage[8 + jj] = *reinterpret_cast<const u32x4*>((jj < 4 ? bg : bu) + pb[jj]);
      }
      stage_pieces = a_pieces;
    };
    // Registers -> ring half `half`: lane i's 16 bytes of piece p go to p * 1024 + 16 i.
    auto write_unit = [&](int half) {
      uint8_t* dst = smem_raw + half * UNIT_BYTES + q * 1024 + lane * 16;
#pragma unroll
      for (int jj = 0; jj < 8; ++jj)
        if (jj < stage_pieces) *reinterpret_cast<u32x4*>(dst + jj * 4096) = stage[jj];
      if constexpr (FP8) {
        // Tile gi = q + 4 jj holds channel rows 16 gi .. 16 gi + 15 of the weight block; the lane's 16
        // codes are k 16 (lane % 4) .. +15 of row 16 gi + fp8_tile_row(lane), i.e. chunks 2 (lane % 4)
        // and the next one of that 128-byte row, stored where the fragment reads expect them (chunk
        // kc of row r in slot kc ^ ((r >> 1) & 7); 16 gi does not change the key).
        const int r = fp8_tile_row(lane), kc = 2 * (lane & 3), key = (r >> 1) & 7;
        uint8_t* wdst = smem_raw + half * UNIT_BYTES + A_BYTES + (16 * q + r) * 128;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const u32x4 c = stage[8 + jj];
          *reinterpret_cast<bf16x8*>(wdst + jj * 8192 + ((kc ^ key) << 4)) =
              fp8x8_to_bf16x8(c[0], c[1]);
          *reinterpret_cast<bf16x8*>(wdst + jj * 8192 + (((kc + 1) ^ key) << 4)) =
              fp8x8_to_bf16x8(c[2], c[3]);
        }
        if (stage_scale_slot >= 0) s_scale[stage_scale_slot * BNV + 64 * q + lane] = stage_scale;
      } else {
        // weights: in x out -- sub-stage h, pieces q + 4 j; out x in -- pieces q + 4 jj of the 32 KB
        // block.  Either way stage[8 + i] goes to byte offset i * 4096 of the weight area.
#pragma unroll
        for (int i = 0; i < 8; ++i)
          *reinterpret_cast<u32x4*>(dst + A_BYTES + i * 4096) = stage[8 + i];
      }
    };
    TileOrder order(my_heavy, my_tiles - my_heavy, (int)(blockIdx.x & 7));
    int ld_ku = -1;  // unit (within its tile) loaded last
    int looked_up = 1;  // tiles looked up so far
    lookup_ahead(order.next());
    auto load_next = [&]() {
      if (ld_ku < 0 || ld_ku + 1 == nu) {
        setup_loads();
        if (looked_up < my_tiles) {
          lookup_ahead(order.next());
          ++looked_up;
        }
        ld_ku = 0;
      } else {
        ++ld_ku;
      }
      load_unit(ld_ku);
    };
    // bf16 weights: write_unit and load_next in one pass, register by register -- the store of a
    // register into the ring, then the load of the next unit's piece into that register.  A wave
    // issues in order, and its LDS stores and its loads each take their turn at a unit of the CU that
    // it shares with the other producers (16 stores of 1 KB: about 1250 clocks next to the
    // consumers' reads; 16 loads: about 630): as two phases one after the other they add up,
    // interleaved the two units work at the same time.
    auto write_and_load = [&](int half) {
      if (ld_ku < 0 || ld_ku + 1 == nu) {
        setup_loads();
        if (looked_up < my_tiles) {
          lookup_ahead(order.next());
          ++looked_up;
        }
        ld_ku = 0;
      } else {
        ++ld_ku;
      }
      if constexpr (!FP8) {
        int ku = ld_ku;
        const bool second = TWO_SRC && ku >= nu / 2;
        if constexpr (TWO_SRC) ku = second ? ku - nu / 2 : ku;
        const uint16_t* a_src = second ? reinterpret_cast<const uint16_t*>(S0) : A;
        const uint8_t* abase = reinterpret_cast<const uint8_t*>(a_src + (size_t)ku * (2 * BK));
        uint8_t* dst = smem_raw + half * UNIT_BYTES + q * 1024 + lane * 16;
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
          if (jj < stage_pieces) *reinterpret_cast<u32x4*>(dst + jj * 4096) = stage[jj];
          if (jj < a_pieces) stage[jj] = *reinterpret_cast<const u32x4*>(abase + pa[jj]);
        }
        if constexpr (KN) {
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const size_t k0 = ((size_t)ku * 2 + h) * BK * N;
            const uint8_t* bg = reinterpret_cast<const uint8_t*>(ld_bg + k0);
            const uint8_t* bu = reinterpret_cast<const uint8_t*>(ld_bu + k0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              *reinterpret_cast<u32x4*>(dst + A_BYTES + (4 * h + i) * 4096) = stage[8 + 4 * h + i];
              stage[8 + 4 * h + i] = *reinterpret_cast<const u32x4*>((i < 2 ? bg : bu) + pb[i]);
            }
          }
        } else {
          const uint8_t* bg =
              reinterpret_cast<const uint8_t*>((second ? ld_bu : ld_bg) + (size_t)ku * (2 * BK));
          const uint8_t* bu =
              TWO_SRC ? bg : reinterpret_cast<const uint8_t*>(ld_bu + (size_t)ku * (2 * BK));
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            *reinterpret_cast<u32x4*>(dst + A_BYTES + jj * 4096) = stage[8 + jj];
            stage[8 + jj] = *reinterpret_cast<const u32x4*>((jj < 4 ? bg : bu) + pb[jj]);
          }
        }
        stage_pieces = a_pieces;
      }
    };
    load_next();
    write_unit(0);
    if (1 < total_units) load_next();
    int ku = 0;
    for (int gu = 0; gu < total_units; ++gu) {
      __syncthreads();  // unit gu is in LDS; the consumers are done with unit gu - 1
      if constexpr (FP8) {
        if (gu + 1 < total_units) write_unit((gu + 1) & 1);
        if (gu + 2 < total_units) load_next();
      } else {
        if (gu + 2 < total_units)
          write_and_load((gu + 1) & 1);
        else if (gu + 1 < total_units)
          write_unit((gu + 1) & 1);
      }
      if (++ku == nu) {
        ku = 0;
        __syncthreads();  // the consumers' barrier ahead of their epilogue
      }
    }
    return;
  }

  // ---- consumers ------------------------------------------------------------------------------------
  // ---- fragment addresses (bytes, from the start of a ring half) ------------------------------------
  //   activations: row r = wm*64 + fm*32 + lr of the block, chunk kc = 4*h + 2*ks + lk (h = weight
  //                sub-stage, ks = k-slice of 16) in slot kc ^ ((r >> 1) & 7);
  //                (r >> 1) & 7 == (lr >> 1) & 7, so fm only adds 32 rows.
  //   weights: k = 16*ks + 8*lk + (s >> 2) (+4 for the upper half) and k & 3 == (s >> 2) & 3, so ks
  //            adds 16 rows and the upper half 4 rows of BROW bytes: compile-time immediates.
  const int xrow = (wm * 64 + lr) * 128;
  const int xr3 = (lr >> 1) & 7;
  int wb[4];
  {
    const int s = lane & 15, half = (lane >> 4) & 1;
#pragma unroll
    for (int fn = 0; fn < 4; ++fn) {
      // sub-tile (matrix) and first channel of fragment fn inside it
      const int mat = DUAL ? (fn >> 1) : 0;
      const int cbase = DUAL ? (wn * 64 + (fn & 1) * 32) : (wn * 128 + fn * 32);
      if constexpr (KN) {
        const int k = lk * 8 + (s >> 2);
        const int col = cbase + half * 16 + (s & 3) * 4;
        wb[fn] = A_BYTES + mat * (B_BYTES / 2) + k * BROW + (((col >> 3) ^ ((k & 3) << 2)) * 16) +
                 (col & 7) * 2;
      } else {
        // row (channel) mat * 128 + cbase + lr of the weight block; its swizzle key is xr3 again
        wb[fn] = A_BYTES + (mat * 128 + cbase + lr) * 128;
      }
    }
  }

  f32x16 acc[4][2];  // [fn][fm]
  auto compute_unit = [&](int gu) {
    const uint8_t* su = smem_raw + (gu & 1) * UNIT_BYTES;
    const uint8_t* sa = su + xrow;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const uint8_t* sb = su + h * B_BYTES;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        bf16x8 xf[2], wf[4];
        const int xo = ((4 * h + 2 * ks + lk) ^ xr3) * 16;
#pragma unroll
        for (int fm = 0; fm < 2; ++fm)
          xf[fm] = lds_read_frag(reinterpret_cast<const uint16_t*>(sa + xo + fm * 4096));
#pragma unroll
        for (int fn = 0; fn < 4; ++fn) {
          if constexpr (KN)
            wf[fn] = lds_read_frag_tr(
                reinterpret_cast<const uint16_t*>(sb + wb[fn] + ks * 16 * BROW),
                reinterpret_cast<const uint16_t*>(sb + wb[fn] + ks * 16 * BROW + 4 * BROW));
          else
            wf[fn] = lds_read_frag(reinterpret_cast<const uint16_t*>(su + wb[fn] + xo));
        }
#pragma unroll
        for (int fn = 0; fn < 4; ++fn)
#pragma unroll
          for (int fm = 0; fm < 2; ++fm)
            acc[fn][fm] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[fn], xf[fm], acc[fn][fm], 0, 0, 0);
      }
    }
  };
  // Epilogue.  A lane holds, for row lr of each 32-row fragment, channels 8q + 4*lk + {0..3} of each
  // 32-channel fragment: stored directly, every store instruction would touch 32 different cache
  // lines with 16 bytes each, and the address unit spends its time per line, not per byte (the
  // direct epilogue cost as much as half the MFMA work of a tile).  So the wave first transposes its
  // tile through LDS, 32 rows at a time: the ring half that the tile's last unit was read from is
  // free until the producers pass the next barrier, and each consumer owns 8 KB of it.  Rows go in
  // as 8-byte writes and come back as 16-byte reads with consecutive lanes along a row, so a store
  // instruction writes whole 128-byte lines (4 rows x 256 B, or 8 rows x 128 B when DUAL).
  // The 16-byte chunk index is XOR-swizzled with the row so that neither side has bank conflicts
  // beyond two-way.
  // Chunk c of row r sits at r * ROWB + ((c ^ key(r)) << 4), key(r) = (r >> 1) & 7 when DUAL (rows are
  // 128 B: two rows span the banks) and r & 15 otherwise.  With r and c split into a per-lane part and
  // a compile-time part, every address below is one per-lane base XOR / plus constants.
  auto store_tile = [&](const Tile& t, int gu, int scale_slot) {
    constexpr int ROWB = DUAL ? 128 : 256;  // bytes per row of the wave's output tile
    constexpr int CH = ROWB / 16;           // 16-byte chunks per row
    constexpr int RPI = 64 / CH;            // rows per store instruction
    uint8_t* buf = smem_raw + (gu & 1) * UNIT_BYTES + wave * 8192;
    // Everything below is cheap to derive from the lane number but loop-invariant: computed ahead of
    // the main loop it would sit in registers that loop needs, or in scratch (three dwords reloaded
    // at the start of every tile's epilogue, as the compiler had it).  An opaque copy of the lane
    // number keeps the arithmetic here.
    int lane_l = lane;
    asm volatile("" : "+v"(lane_l));
    const int lane = lane_l, lr = lane & 31, lk = lane >> 5;
    // write side: row lr, chunk 4 fn + q, half lk
    const int wkey = DUAL ? ((lr >> 1) & 7) : (lr & 15);
    const uint32_t wbase = (uint32_t)(lr * ROWB + (wkey << 4) + lk * 8);
    // read side: row it * RPI + lane / CH, chunk lane % CH; the row's key is
    // (lane >> 4) | (it's low bits << 2), so the per-lane part is
    const uint32_t rbase =
        (uint32_t)((lane / CH) * ROWB + (((lane % CH) ^ (lane >> 4)) << 4));
    // store side: a uniform row base per store plus one per-lane byte offset
    const int n = t.n0 + (DUAL ? wn * 64 : wn * 128) + (lane % CH) * 8;
    const int m_wave = t.row0 + wm * 64;  // first row of the wave's tile
    const int r_lane = lane / CH;
    const uint32_t lane_off = (uint32_t)((r_lane * ldc + n) * 2);
    const bool col_ok = n < N;
    const uint32_t wbase_l = wbase, rbase_l = rbase, lane_off_l = lane_off;
#pragma unroll
    for (int fm = 0; fm < 2; ++fm) {
#pragma unroll
      for (int fn = 0; fn < (DUAL ? 2 : 4); ++fn) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float v[4];
          if constexpr (FP8) {
            // the lane's four channels 8 q + 4 lk + {0..3} of fragment fn: virtual channel c of the
            // tile (and 128 + c for the up half)
            const int c = (DUAL ? wn * 64 : wn * 128) + fn * 32 + 8 * q + 4 * lk;
            const float* sc = s_scale + scale_slot * BNV + c;
            const f32x4 sg = *reinterpret_cast<const f32x4*>(sc);
            if constexpr (DUAL) {
              const f32x4 su = *reinterpret_cast<const f32x4*>(sc + 128);
#pragma unroll
              for (int j = 0; j < 4; ++j)
                v[j] = silu_f32(acc[fn][fm][4 * q + j] * sg[j]) * (acc[fn + 2][fm][4 * q + j] * su[j]);
            } else {
#pragma unroll
              for (int j = 0; j < 4; ++j) v[j] = acc[fn][fm][4 * q + j] * sg[j];
            }
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if (DUAL)
                v[j] = silu_f32(acc[fn][fm][4 * q + j]) * acc[fn + 2][fm][4 * q + j];
              else
                v[j] = acc[fn][fm][4 * q + j];
            }
          }
          u32x2 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
          *reinterpret_cast<u32x2*>(buf + (wbase_l ^ (uint32_t)((4 * fn + q) << 4))) = o;
        }
      }
      constexpr int KEYMASK = DUAL ? 1 : 3;
#pragma unroll
      for (int it = 0; it < 32 / RPI; ++it) {
        const u32x4 val = *reinterpret_cast<const u32x4*>(
            buf + (rbase_l ^ (uint32_t)((it & KEYMASK) << 6)) + it * RPI * ROWB);
        const int r = m_wave + fm * 32 + it * RPI;  // uniform
        uint8_t* row_base = reinterpret_cast<uint8_t*>(C + (size_t)r * ldc);
        if (col_ok && r + r_lane < t.row_end)
          // streaming store: the tile is not read again by this kernel
          __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(row_base + lane_off_l));
      }
    }
  };
  // KEEP_GU: the same walk twice more, for the gate and the up product (a function of its own so
  // that the other variants' epilogue compiles to what it was).
  auto store_products = [&](const Tile& t, int gu) {
    constexpr int ROWB = 128, CH = 8, RPI = 8;
    uint8_t* buf = smem_raw + (gu & 1) * UNIT_BYTES + wave * 8192;
    int lane_l = lane;  // (as in store_tile)
    asm volatile("" : "+v"(lane_l));
    const int lane = lane_l, lr = lane & 31, lk = lane >> 5;
    const uint32_t wbase = (uint32_t)(lr * ROWB + (((lr >> 1) & 7) << 4) + lk * 8);
    const uint32_t rbase = (uint32_t)((lane / CH) * ROWB + (((lane % CH) ^ (lane >> 4)) << 4));
    const int n = t.n0 + wn * 64 + (lane % CH) * 8;
    const int m_wave = t.row0 + wm * 64;
    const int r_lane = lane / CH;
    const uint32_t lane_off = (uint32_t)((r_lane * ldc + n) * 2);
    const bool col_ok = n < N;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      uint16_t* out = reinterpret_cast<uint16_t*>(const_cast<float*>(which == 0 ? S0 : S1));
#pragma unroll
      for (int fm = 0; fm < 2; ++fm) {
#pragma unroll
        for (int fn = 0; fn < 2; ++fn)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const f32x16& a = acc[fn + 2 * which][fm];
            u32x2 o = {pack_bf16x2(a[4 * q], a[4 * q + 1]), pack_bf16x2(a[4 * q + 2], a[4 * q + 3])};
            *reinterpret_cast<u32x2*>(buf + (wbase ^ (uint32_t)((4 * fn + q) << 4))) = o;
          }
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
          const u32x4 val = *reinterpret_cast<const u32x4*>(
              buf + (rbase ^ (uint32_t)((it & 1) << 6)) + it * RPI * ROWB);
          const int r = m_wave + fm * 32 + it * RPI;  // uniform
          uint8_t* row_base = reinterpret_cast<uint8_t*>(out + (size_t)r * ldc);
          if (col_ok && r + r_lane < t.row_end)
            __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(row_base + lane_off));
        }
      }
    }
  };

  // ---- main stream -----------------------------------------------------------------------------------
  TileOrder order(my_heavy, my_tiles - my_heavy, (int)(blockIdx.x & 7));
  Tile cur = locate(order.next());
  bool wave_active = cur.row0 + wm * 64 < cur.row_end;
  int ku = 0, tiles_left = my_tiles - 1, tiles_done = 0;
  for (int gu = 0; gu < total_units; ++gu) {
    __syncthreads();  // the producers have seen unit gu land
    if (ku == 0) {
#pragma unroll
      for (int fn = 0; fn < 4; ++fn)
#pragma unroll
        for (int fm = 0; fm < 2; ++fm)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[fn][fm][i] = 0.f;
    }
    if (wave_active) compute_unit(gu);
    if (++ku == nu) {
      __syncthreads();  // every consumer is done with the ring half the epilogue borrows
      if (wave_active) store_tile(cur, gu, tiles_done & 1);
      if constexpr (KEEP_GU)
        if (wave_active) store_products(cur, gu);
      ++tiles_done;
      ku = 0;
      if (tiles_left-- > 0) {
        cur = locate(order.next());
        wave_active = cur.row0 + wm * 64 < cur.row_end;
      }
    }
  }
}

}  // namespace fs2moe

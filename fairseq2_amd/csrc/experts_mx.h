// Grouped GEMM on the fp8 matrix pipe (W8A8): e4m3 weights with one f32 scale per output channel,
// e4m3 activations with one power-of-two scale per row and 32 consecutive features (the block
// scaling that v_mfma_scale_f32_32x32x64_f8f6f4 applies in hardware).
//
// Same organisation as the bf16 throughput kernel (experts_dma.h): persistent blocks, 256 x 256
// tiles, eight consumer waves of 64 x 128 and four producer waves, a two-unit LDS ring with one
// barrier per unit.  A unit is 128 k here, so its bytes are those of a bf16 unit of 64 k (256 rows
// of 128 bytes per operand, the same pieces, the same swizzle) while its MFMAs do twice the flops
// in the same number of cycles.
//
// Operand order of the instruction, found by a probe: of a lane's 32 operand bytes the first 16
// are k 16 g .. 16 g + 15 and the last 16 are k 32 + 16 g .. 32 + 16 g + 15 (g = lane / 32); the
// scale held by lanes 0..31 applies to k 0..31 and the scale held by lanes 32..63 to k 32..63,
// whichever lane's registers the bytes sit in.  So for the k-step s of a unit, lane group g reads
// chunks 4 s + g and 4 s + 2 + g of its row and carries the scale of block 2 s + g.
//
// Weights arrive in the tiles of experts_fp8.h ([expert][channel / 16][k / 64][16][64], 1 KB each),
// so one packed copy serves the decode stream, the W8A16 path and this one.
//
// DUAL (gate/up): the epilogue applies the channel scales, the SiLU gate, and quantises the result
// the same way (block of 32 channels of a row -> power-of-two scale + e4m3 codes), which is what
// the down projection reads.  Single matrix: bf16 rows out.
#pragma once

#include "common.h"
#include "experts_dma.h"
#include "tile_map.h"

namespace fs2moe {
namespace mx {
constexpr int BM = 256, BNV = 256, UK = 128;  // rows, virtual channels, k per unit
constexpr int CONSUMERS = 8, PRODUCERS = 4, NWAVES = CONSUMERS + PRODUCERS;
constexpr int A_BYTES = BM * UK;   // 32 KB
constexpr int W_BYTES = BNV * UK;  // 32 KB
constexpr int UNIT_BYTES = A_BYTES + W_BYTES;
constexpr int RING_BYTES = 2 * UNIT_BYTES;
constexpr int LIGHT_ROWS = 128;
constexpr int TABLE_INTS = 4 * FS2MOE_MAX_EXPERTS + 8;
constexpr int WSCALE_BYTES = 2 * BNV * 4;  // channel scales of two tiles
constexpr int ASCALE_BYTES = 2 * BM * 4;   // four block scales per row, of two units
constexpr int SMEM_BYTES = RING_BYTES + TABLE_INTS * 4 + WSCALE_BYTES + ASCALE_BYTES;
constexpr int BAND = 8;

typedef __attribute__((ext_vector_type(8))) int i32x8;

// The shared exponent of a block: the smallest X with amax / 2^X <= 448 (the largest e4m3 value),
// from amax's bits alone: amax = m 2^e with m in [1, 2) needs X = e - 8 when m <= 1.75 and e - 7
// otherwise.  Clamped to what a scale byte can say; zero (and denormal) blocks get the smallest.
__device__ __forceinline__ int block_exponent(float amax) {
  const uint32_t u = __float_as_uint(amax) & 0x7fffffffu;
  const int be = (int)(u >> 23);
  int x = be - 127 - 8 + ((u & 0x7fffffu) > 0x600000u ? 1 : 0);
  if (be == 0) x = -127;
  return x < -127 ? -127 : (x > 127 ? 127 : x);
}
// Four floats times 2^-X -> four e4m3 codes in a dword (round to nearest even).
__device__ __forceinline__ uint32_t to_e4m3x4(float a, float b, float c, float d, float inv) {
  int r = 0;
  r = __builtin_amdgcn_cvt_pk_fp8_f32(a * inv, b * inv, r, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c * inv, d * inv, r, true);
  return (uint32_t)r;
}
}  // namespace mx

// Which of a 1 KB weight tile's 16 channel rows lane l of a producer takes (with the 16 codes at
// k 16 (l % 4) of it).  As fp8_tile_row in experts_dma.h, for this kernel's stores: a lane writes one
// 16-byte chunk, four lanes the 64-byte half of a 128-byte LDS row, and the two rows served together
// (eight lanes) must land in different halves: rows r and r + 8, whose swizzle keys differ by 4
// (6.5 against 8.0 clocks per store instruction in the probe).
__device__ __forceinline__ int mx_tile_row(int lane) {
  return (((lane >> 2) & 1) << 3) | ((lane >> 3) & 7);
}

// A [a_rows, Kdim] e4m3 codes with scale bytes As, both read through row_map when it is given; B0 / B1
// tiled e4m3 weights with channel scales S0 / S1 [E, N].
// DUAL: C = e4m3 codes [c_rows, N] (ldc bytes per row) and their scale bytes Cs; else C = bf16.
// Scale bytes lie k-group major: [K / 128][rows][4], the four blocks of 128 features of a row as
// one dword.  A unit needs exactly that dword of each of its 256 rows; row major ([rows][K / 32])
// the 64 lanes of the load touched 32 to 64 cache lines for their 256 bytes, and that one gathered
// load per unit made the producers' unit a quarter longer (1.38 against 1.09 us with the consumers'
// work removed).  This way consecutive rows are consecutive dwords: expert-major rows (the gated
// product) always are, and token rows read through the permutation mostly are for the experts
// that take most tokens, whose rows are dense runs of token numbers.
template <bool DUAL>
__global__ __launch_bounds__(mx::NWAVES * 64) void glu_gemm_mx_kernel(
    const uint8_t* __restrict__ A, const uint8_t* __restrict__ As,
    const int32_t* __restrict__ row_map, const uint8_t* __restrict__ B0,
    const uint8_t* __restrict__ B1, const float* __restrict__ S0, const float* __restrict__ S1,
    void* __restrict__ Cv, uint8_t* __restrict__ Cs, int ldc, int Kdim, int N, Groups g,
    int n_tiles, int a_rows, int c_rows) {
  using namespace mx;
  constexpr int BN = DUAL ? 128 : 256;  // real channels per tile
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_raw[];
  int32_t* s_hstart = reinterpret_cast<int32_t*>(smem_raw + RING_BYTES);  // [E + 1]
  int32_t* s_lstart = s_hstart + FS2MOE_MAX_EXPERTS + 4;                  // [E + 1]
  int32_t* s_counts = s_lstart + FS2MOE_MAX_EXPERTS + 4;
  int32_t* s_offsets = s_counts + FS2MOE_MAX_EXPERTS;
  float* s_wscale = reinterpret_cast<float*>(smem_raw + RING_BYTES + TABLE_INTS * 4);  // [2][BNV]
  uint32_t* s_ascale = reinterpret_cast<uint32_t*>(smem_raw + RING_BYTES + TABLE_INTS * 4 + WSCALE_BYTES);  // [2][BM]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) & 3, wn = wave & 1;
  const int lr = lane & 31, lk = lane >> 5;

  // ---- tile tables: heavy tiles (256 rows, or a last tile of more than 128) first, then light ones,
  // dealt round-robin over slots ordered by XCD (as in experts_dma.h)
  const bool dense = g.counts == nullptr;
  const int E = dense ? 1 : g.E;
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
  const int total_heavy = s_hstart[E];
  const int slot = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
  const int grid = (int)gridDim.x;
  // the heavy tiles left over by the whole rounds of the deal go out as halves of 128 rows when
  // those and the light tiles fit one round (as in the bf16 kernel: same sums, a shorter last round)
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
  const int my_heavy = slot < heavy_end ? (heavy_end - slot + grid - 1) / grid : 0;
  const int nu = Kdim / UK;  // the host guarantees Kdim % 128 == 0
  const int total_units = my_tiles * nu;

  struct Tile {
    int e, row0, row_end, n0;
  };
  auto locate = [&](int j) {
    const int listed = slot + j * grid;
    const bool is_light = listed >= halves_end;
    const int half = (listed >= heavy_end && !is_light) ? ((listed - heavy_end) & 1) : -1;
    const int logical = half >= 0 ? heavy_end + ((listed - heavy_end) >> 1) : listed;
    const int in_kind = is_light ? listed - halves_end : logical;
    int mt = in_kind / n_tiles;
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
      // heavy tiles of an expert in bands of BAND row blocks, row block minor within a band
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

  const size_t wstride = (size_t)Kdim * N;  // codes of one expert's matrix
  const int nkb = Kdim / 64;                // weight tiles along k

  if (wave >= CONSUMERS) {
    // ---- producers ----------------------------------------------------------------------------------
    // Producer q moves pieces q, q + 4, ... of both operands, 8 rows x 128 B each, straight from
    // global memory into LDS (buffer_load ... lds: lane i's 16 bytes land at 16 i of the piece, i.e.
    // row i / 8, slot i % 8, and the lane fetches the chunk that the swizzle puts there): no staging
    // registers and no LDS store instructions.  An activation piece is 8 rows of the (gathered)
    // operand; a weight piece is 8 channel rows of a 16-channel group, each row made of 64 bytes of
    // the group's two 1 KB tiles (16 channels x 64 k) of this unit.  Plus the unit's four scale bytes
    // of rows 64 q .. 64 q + 63 (a dword per lane, the same way) and, with a tile's first unit, its
    // channel scales.  The loads of unit u + 1 go out when the consumers are done with unit u - 1 (the
    // barrier of unit u) and must have landed by the next barrier: one unit of lead, so nothing may
    // stand between that barrier and the loads.  A tile's addresses are therefore worked out a tile
    // ahead (which tile, the tokens of its rows, its channel scale: lookup_ahead).
    // Against producers that stage through registers and store to LDS (same box, rocprofv3, Qwen3
    // prefill layer): gate/up 247.3 -> 241.5 us, down 164.0 -> 163.2 us; harness, random codes:
    // Mixtral's counts 2723 -> 2635 us, Scout's 1242 -> 1220, Qwen3's 470 -> 458.  (Without the
    // look-ahead the same producers were slower in the layer: 241 -> 247 and 158 -> 170 us.)
    const int q = wave - CONSUMERS;
    typedef __attribute__((address_space(3))) void* lds_ptr;
    uint32_t pa[8], pb[8], ps = 0;
    int a_pieces = 0;
    const uint8_t* ld_b[2] = {B0, B0};
    float ld_scale = 0.f;
    int ld_tiles = 0;
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(A), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t as_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(As), 0, -1, 0x00020000);
    // The tile after the one set up last, looked up a tile ahead: which tile it is, the tokens its
    // rows are read from (row_map: loads that the tile's own loads depend on) and its channel scale.
    Tile pre_t = {0, 0, 0, 0};
    int pre_rows[8], pre_srow = 0;
    float pre_scale = 0.f;
    auto lookup_ahead = [&](int j) {
      pre_t = locate(j);
      {
        const int v = 64 * q + lane;  // virtual channel: gate 0..127, up 128..255
        const bool up = DUAL && v >= 128;
        int ch = pre_t.n0 + (up ? v - 128 : v);
        ch = ch < N ? ch : N - 1;  // clamped channels are never stored
        pre_scale = (up ? S1 : S0)[(size_t)pre_t.e * N + ch];
      }
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        int grow = pre_t.row0 + 8 * (q + 4 * jj) + (lane >> 3);
        grow = grow < pre_t.row_end ? grow : pre_t.row_end - 1;  // clamped rows are never stored
        pre_rows[jj] = row_map != nullptr ? row_map[grow] : grow;
      }
      int grow = pre_t.row0 + 64 * q + lane;
      grow = grow < pre_t.row_end ? grow : pre_t.row_end - 1;
      pre_srow = row_map != nullptr ? row_map[grow] : grow;
    };
    auto setup_loads = [&]() {
      const Tile t = pre_t;
      ld_b[0] = B0 + (size_t)t.e * wstride;
      ld_b[1] = DUAL ? B1 + (size_t)t.e * wstride : ld_b[0];
      ld_scale = pre_scale;
      ++ld_tiles;
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const int row = 8 * (q + 4 * jj) + (lane >> 3), slot16 = lane & 7;
        const int kc = slot16 ^ ((row >> 1) & 7);
        pa[jj] = (uint32_t)((size_t)pre_rows[jj] * Kdim + kc * 16);
      }
      ps = (uint32_t)pre_srow * 4u;
      const int rows = t.row_end - t.row0;
      a_pieces = rows >= BM ? 8 : (rows - 8 * q + 31) / 32;
      a_pieces = a_pieces < 0 ? 0 : a_pieces;
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        const int P = q + 4 * jj;
        const int gi = P >> 1, r16 = 8 * (P & 1) + (lane >> 3);
        const int row = 8 * P + (lane >> 3);
        const int c = (lane & 7) ^ ((row >> 1) & 7);
        int group = t.n0 / 16 + (DUAL ? (gi & 7) : gi);
        group = group < N / 16 ? group : N / 16 - 1;  // clamped channels are never stored
        pb[jj] = (uint32_t)(((size_t)group * nkb + (c >> 2)) * 1024 + r16 * 64 + (c & 3) * 16);
      }
    };
    auto issue_unit = [&](int ku, int half) {
      uint8_t* base = smem_raw + half * UNIT_BYTES;
      const uint32_t koff_a = (uint32_t)ku * UK;
#pragma unroll
      for (int jj = 0; jj < 8; ++jj)
        if (jj < a_pieces)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (lds_ptr)(base + (q + 4 * jj) * 1024), 16, pa[jj], koff_a, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(as_rsrc, (lds_ptr)(&s_ascale[half * BM + 64 * q]), 4, ps,
                                               (uint32_t)ku * (uint32_t)a_rows * 4u, 0, 0);
      const __amdgpu_buffer_rsrc_t bg = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ld_b[0]), 0, -1, 0x00020000);
      const __amdgpu_buffer_rsrc_t bu = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(ld_b[1]), 0, -1, 0x00020000);
      const uint32_t koff_w = (uint32_t)ku * 2048u;  // two tiles along k per unit
#pragma unroll
      for (int jj = 0; jj < 8; ++jj) {
        if (DUAL && jj >= 4)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(bu, (lds_ptr)(base + A_BYTES + (q + 4 * jj) * 1024), 16, pb[jj], koff_w, 0, 0);
        else
          __builtin_amdgcn_raw_ptr_buffer_load_lds(bg, (lds_ptr)(base + A_BYTES + (q + 4 * jj) * 1024), 16, pb[jj], koff_w, 0, 0);
      }
      if (ku == 0) s_wscale[((ld_tiles - 1) & 1) * BNV + 64 * q + lane] = ld_scale;
    };
    TileOrder order(my_heavy, my_tiles - my_heavy, (int)(blockIdx.x & 7));
    int ld_ku = -1, looked_up = 1;
    lookup_ahead(order.next());
    auto issue_next = [&](int half) {
      const bool first = ld_ku < 0 || ld_ku + 1 == nu;
      if (first) {
        setup_loads();
        ld_ku = 0;
      } else {
        ++ld_ku;
      }
      issue_unit(ld_ku, half);
      if (first && looked_up < my_tiles) {  // (after the unit's loads have gone out)
        lookup_ahead(order.next());
        ++looked_up;
      }
    };
    issue_next(0);
    int ku = 0;
    for (int gu = 0; gu < total_units; ++gu) {
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of unit gu has landed
      __syncthreads();  // unit gu is in LDS; the consumers are done with unit gu - 1
      if (gu + 1 < total_units) issue_next((gu + 1) & 1);
      if (++ku == nu) {
        ku = 0;
        __syncthreads();  // the consumers' barrier ahead of their epilogue
      }
    }
    return;
  }

  // ---- consumers ------------------------------------------------------------------------------------
  // Row r of either operand block is 128 bytes; chunk c sits in slot c ^ ((r >> 1) & 7).  The wave's
  // rows are wm * 64 + fm * 32 + lr (activations) and mat * 128 + cbase + lr (weights): the key is
  // (lr >> 1) & 7 for all of them, and the weight rows of the fragments lie a compile-time number
  // of rows after those of fragment 0.
  constexpr int WFRAG[4] = {0, 32 * 128, DUAL ? 128 * 128 : 64 * 128, DUAL ? 160 * 128 : 96 * 128};

  f32x16 acc[4][2];  // [fn][fm]
  auto compute_unit = [&](int gu) {
    // 128 accumulators leave 40 registers: the fragments of a k-step take 24 of them, so every
    // address below is derived here, once per unit, from an opaque copy of the lane number instead
    // of living in registers (or scratch) across the units.
    int l = tid;
    asm volatile("" : "+v"(l));
    const int lr_ = l & 31, lk_ = (l >> 5) & 1;
    const uint32_t half = (uint32_t)(gu & 1) * UNIT_BYTES;
    const uint8_t* xa = smem_raw + half + (wm * 64 + lr_) * 128;
    const uint8_t* wa = smem_raw + half + A_BYTES + ((DUAL ? wn * 64 : wn * 128) + lr_) * 128;
    const uint32_t kx = (uint32_t)((lk_ ^ ((lr_ >> 1) & 7)) << 4);
    // the four block scales of rows (fm): byte 2 s + lk belongs to this lane group in step s, so
    // after a shift by 8 lk it is byte 0 in step 0 and byte 2 in step 1
    uint32_t sc[2];
#pragma unroll
    for (int fm = 0; fm < 2; ++fm)
      sc[fm] = s_ascale[(gu & 1) * BM + wm * 64 + fm * 32 + lr_] >> (8 * lk_);
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      // chunks 4 s + lk and 4 s + 2 + lk, swizzled
      const uint32_t o0 = kx ^ (uint32_t)((4 * s) << 4), o1 = kx ^ (uint32_t)((4 * s + 2) << 4);
      auto read32 = [&](const uint8_t* row) {
        const u32x4 lo = *reinterpret_cast<const u32x4*>(row + o0);
        const u32x4 hi = *reinterpret_cast<const u32x4*>(row + o1);
        const i32x8 v = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3],
                         (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        return v;
      };
      i32x8 xf[2];
#pragma unroll
      for (int fm = 0; fm < 2; ++fm) xf[fm] = read32(xa + fm * 4096);
#pragma unroll
      for (int fn = 0; fn < 4; ++fn) {
        const i32x8 wf = read32(wa + WFRAG[fn]);
#pragma unroll
        for (int fm = 0; fm < 2; ++fm) {
          // operand a = weights (scale 1 = exponent byte 127), operand b = activations
          if (s == 0)
            acc[fn][fm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                wf, xf[fm], acc[fn][fm], 0, 0, 0, 0x7f7f7f7f, 0, (int)sc[fm]);
          else
            acc[fn][fm] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                wf, xf[fm], acc[fn][fm], 0, 0, 0, 0x7f7f7f7f, 2, (int)sc[fm]);
        }
      }
    }
  };

  // Epilogue.  A lane holds, for row lr of each 32-row fragment, channels 8 q + 4 lk + {0..3} of each
  // 32-channel fragment.  The wave transposes 32 rows at a time through the ring half the tile's
  // last unit was read from (8 KB per consumer), so that store instructions write whole row pieces.
  auto store_tile = [&](const Tile& t, int gu, int scale_slot) {
    // Everything below is cheap to derive from the lane number but loop-invariant: computed ahead of
    // the main loop it would sit in registers that loop needs (or in scratch, reloaded per unit).
    // An opaque copy of the lane number keeps the address arithmetic here.
    int lane_l = tid;
    asm volatile("" : "+v"(lane_l));
    const int lane = lane_l & 63, lr = lane & 31, lk = lane >> 5;
    uint8_t* buf = smem_raw + (gu & 1) * UNIT_BYTES + wave * 8192;
    const float* wsc = s_wscale + scale_slot * BNV;
    const int m_wave = t.row0 + wm * 64;
    if constexpr (DUAL) {
      // e4m3 codes out: the wave's 64 channels are 64 bytes of a row; a block of 32 channels (one
      // fragment) is held by lanes lr and lr + 32
      uint8_t* C = static_cast<uint8_t*>(Cv);
      const int n = t.n0 + wn * 64;  // first real channel of the wave
      const bool col_ok = n < N;     // N is a multiple of 64
#pragma unroll
      for (int fm = 0; fm < 2; ++fm) {
        uint32_t sbytes = 0;
#pragma unroll
        for (int fn = 0; fn < 2; ++fn) {
          float v[16];
          float amax = 0.f;
#pragma unroll
          for (int qq = 0; qq < 4; ++qq) {
            const int c = wn * 64 + fn * 32 + 8 * qq + 4 * lk;
            const f32x4 sg = *reinterpret_cast<const f32x4*>(wsc + c);
            const f32x4 sup = *reinterpret_cast<const f32x4*>(wsc + 128 + c);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float x = silu_f32(acc[fn][fm][4 * qq + j] * sg[j]) * (acc[fn + 2][fm][4 * qq + j] * sup[j]);
              v[4 * qq + j] = x;
              amax = fmaxf(amax, fabsf(x));
            }
          }
          // the other half of the block sits in lane ^ 32
          amax = fmaxf(amax, __int_as_float(__builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __float_as_int(amax))));
          const int X = block_exponent(amax);
          const float inv = __builtin_ldexpf(1.0f, -X);
          sbytes |= (uint32_t)(X + 127) << (8 * fn);
          // (rows of 64 bytes: the 16-byte chunk index is XOR-ed with bits 2..3 of the row, or the 32
          // lanes of a store, 64 bytes apart, would share four banks)
#pragma unroll
          for (int qq = 0; qq < 4; ++qq) {
            const int dw = 8 * fn + 2 * qq + lk;  // dword of the row: chunk dw / 4
            *reinterpret_cast<uint32_t*>(buf + lr * 64 + ((((dw >> 2) ^ (lr >> 2)) & 3) << 4) + (dw & 3) * 4) =
                to_e4m3x4(v[4 * qq], v[4 * qq + 1], v[4 * qq + 2], v[4 * qq + 3], inv);
          }
        }
        const int r0 = m_wave + fm * 32;
#pragma unroll
        for (int it = 0; it < 2; ++it) {
          const int rl = it * 16 + (lane >> 2);
          const u32x4 val =
              *reinterpret_cast<const u32x4*>(buf + rl * 64 + ((((lane & 3) ^ (rl >> 2)) & 3) << 4));
          if (col_ok && r0 + rl < t.row_end)
            __builtin_nontemporal_store(
                val, reinterpret_cast<u32x4*>(C + (size_t)(r0 + rl) * ldc + n + (lane & 3) * 16));
        }
        if (lk == 0 && col_ok && r0 + lr < t.row_end)
          *reinterpret_cast<uint16_t*>(Cs + ((size_t)(n >> 7) * c_rows + r0 + lr) * 4 + ((n >> 5) & 3)) =
              (uint16_t)sbytes;
      }
    } else {
      // bf16 out, as the bf16 kernel stores it: rows of 256 bytes per wave, chunk c of row r at
      // r * 256 + ((c ^ (r & 15)) << 4)
      uint16_t* C = static_cast<uint16_t*>(Cv);
      constexpr int ROWB = 256, CH = 16, RPI = 4;
      const uint32_t wbase = (uint32_t)(lr * ROWB + ((lr & 15) << 4) + lk * 8);
      const uint32_t rbase = (uint32_t)((lane / CH) * ROWB + (((lane % CH) ^ (lane >> 4)) << 4));
      const int n = t.n0 + wn * 128 + (lane % CH) * 8;
      const int r_lane = lane / CH;
      const bool col_ok = n < N;
#pragma unroll
      for (int fm = 0; fm < 2; ++fm) {
#pragma unroll
        for (int fn = 0; fn < 4; ++fn) {
#pragma unroll
          for (int qq = 0; qq < 4; ++qq) {
            const int c = wn * 128 + fn * 32 + 8 * qq + 4 * lk;
            const f32x4 sg = *reinterpret_cast<const f32x4*>(wsc + c);
            u32x2 o = {pack_bf16x2(acc[fn][fm][4 * qq] * sg[0], acc[fn][fm][4 * qq + 1] * sg[1]),
                       pack_bf16x2(acc[fn][fm][4 * qq + 2] * sg[2], acc[fn][fm][4 * qq + 3] * sg[3])};
            *reinterpret_cast<u32x2*>(buf + (wbase ^ (uint32_t)((4 * fn + qq) << 4))) = o;
          }
        }
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
          const u32x4 val = *reinterpret_cast<const u32x4*>(
              buf + (rbase ^ (uint32_t)((it & 3) << 6)) + it * RPI * ROWB);
          const int r = m_wave + fm * 32 + it * RPI;
          if (col_ok && r + r_lane < t.row_end)
            __builtin_nontemporal_store(
                val, reinterpret_cast<u32x4*>(C + (size_t)(r + r_lane) * ldc + n));
        }
      }
    }
  };

  TileOrder order(my_heavy, my_tiles - my_heavy, (int)(blockIdx.x & 7));
  Tile cur = locate(order.next());
  bool wave_active = cur.row0 + wm * 64 < cur.row_end;
  int ku = 0, tiles_left = my_tiles - 1, tiles_done = 0;
  for (int gu = 0; gu < total_units; ++gu) {
    __syncthreads();
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
      __syncthreads();
      if (wave_active) store_tile(cur, gu, tiles_done & 1);
      ++tiles_done;
      ku = 0;
      if (tiles_left-- > 0) {
        cur = locate(order.next());
        wave_active = cur.row0 + wm * 64 < cur.row_end;
      }
    }
  }
}

// x [T, D] bf16 -> e4m3 codes [T, D] and one scale byte per row and 32 features, k-group major:
// [D / 128][T][4].  A lane owns a block of 32 features (64 bytes in, 32 bytes out); consecutive
// lanes take consecutive blocks of a row, so four lanes fill a scale dword.
__global__ __launch_bounds__(256) void mx_quantize_kernel(const uint16_t* __restrict__ x, int64_t T,
                                                          int D, uint8_t* __restrict__ xq,
                                                          uint8_t* __restrict__ xs) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int nb = D / 32;
  const int64_t blocks = T * nb;
  for (int64_t b = wave * 64 + lane; b < blocks; b += (int64_t)gridDim.x * 256) {
    const uint16_t* src = x + b * 32;
    u32x4 in[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) in[j] = *reinterpret_cast<const u32x4*>(src + 8 * j);
    float v[32];
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[8 * j + 2 * i] = __uint_as_float(in[j][i] << 16);
        v[8 * j + 2 * i + 1] = __uint_as_float(in[j][i] & 0xffff0000u);
        amax = fmaxf(amax, fmaxf(fabsf(v[8 * j + 2 * i]), fabsf(v[8 * j + 2 * i + 1])));
      }
    const int X = mx::block_exponent(amax);
    const float inv = __builtin_ldexpf(1.0f, -X);
    u32x4 out[2];
#pragma unroll
    for (int j = 0; j < 8; ++j)
      out[j >> 2][j & 3] = mx::to_e4m3x4(v[4 * j], v[4 * j + 1], v[4 * j + 2], v[4 * j + 3], inv);
    *reinterpret_cast<u32x4*>(xq + b * 32) = out[0];
    *reinterpret_cast<u32x4*>(xq + b * 32 + 16) = out[1];
    const int64_t row = b / nb;
    const int kb = (int)(b - row * nb);
    xs[((int64_t)(kb >> 2) * T + row) * 4 + (kb & 3)] = (uint8_t)(X + 127);
  }
}

}  // namespace fs2moe

// W8A8 expert path: block-scaled e4m3 activations against e4m3 weights on the fp8 matrix pipe.
// Host side of experts_mx.h.  No counterpart in the reference (its experts run in the parameters'
// dtype, experts.py:102-112); an opt-in of this library.
#include "experts_mx.h"

using namespace fs2moe;

static int mx_cu_count() {
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

extern "C" int fs2moe_mx_quantize(const void* x, int64_t rows, int32_t D, void* codes, void* scales,
                                  void* stream) {
  FS2_REQUIRE(x && codes && scales, "mx_quantize: null pointer");
  FS2_REQUIRE(rows >= 0 && D > 0 && D % 128 == 0, "mx_quantize: rows=%lld, D=%d (a multiple of 128)",
              (long long)rows, D);
  FS2_REQUIRE(aligned16(x) && aligned16(codes), "mx_quantize: buffers must be 16-byte aligned");
  if (rows == 0) return FS2MOE_OK;
  const int64_t blocks32 = rows * (D / 32);
  int64_t grid = (blocks32 + 255) / 256;
  if (grid > 8192) grid = 8192;
  hipLaunchKernelGGL(mx_quantize_kernel, dim3((unsigned)grid), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint16_t*>(x), rows, D,
                     static_cast<uint8_t*>(codes), static_cast<uint8_t*>(scales));
  return check_launch("mx_quantize");
}

extern "C" int fs2moe_grouped_swiglu_w8a8_supported(int32_t D, int32_t F, int64_t max_rows) {
  const int64_t wide = D > F ? D : F;
  return (D > 0 && F > 0 && D % mx::UK == 0 && F % mx::UK == 0 && max_rows >= 0 &&
          max_rows * wide <= 0xffffffffll && (int64_t)D * F <= 0xffffffffll)
             ? 1
             : 0;
}

extern "C" int fs2moe_grouped_swiglu_w8a8(const void* xq, const void* xs, const int32_t* row_map,
                                          const int32_t* counts, const int32_t* offsets,
                                          const void* w_gate, const void* w_up, const void* w_down,
                                          const float* s_gate, const float* s_up,
                                          const float* s_down, int32_t E, int32_t D, int32_t F,
                                          int64_t x_rows, int64_t max_rows, void* hq, void* hs,
                                          void* ye, void* stream) {
  using namespace mx;
  FS2_REQUIRE(xq && xs && counts && offsets && w_gate && w_up && w_down && s_gate && s_up && s_down &&
                  hq && hs && ye,
              "grouped_swiglu_w8a8: null pointer");
  FS2_REQUIRE(E >= 1 && E <= FS2MOE_MAX_EXPERTS, "grouped_swiglu_w8a8: E=%d outside [1, %d]", E,
              FS2MOE_MAX_EXPERTS);
  FS2_REQUIRE(max_rows >= 0 && max_rows < (1ll << 31), "grouped_swiglu_w8a8: max_rows=%lld",
              (long long)max_rows);
  // x_rows: the rows of xq / xs (their number places a k-group's scales): the token count with a
  // row map, else max_rows
  FS2_REQUIRE(x_rows >= 1 && x_rows < (1ll << 31) && (row_map != nullptr || x_rows == max_rows),
              "grouped_swiglu_w8a8: x_rows=%lld", (long long)x_rows);
  FS2_REQUIRE(fs2moe_grouped_swiglu_w8a8_supported(D, F, max_rows),
              "grouped_swiglu_w8a8: D=%d and F=%d must be multiples of %d, and the operands "
              "addressable with 32-bit byte offsets",
              D, F, UK);
  FS2_REQUIRE(aligned16(xq) && aligned16(w_gate) && aligned16(w_up) && aligned16(w_down) &&
                  aligned16(hq) && aligned16(ye) && aligned16(s_gate) && aligned16(s_up) &&
                  aligned16(s_down) && (reinterpret_cast<uintptr_t>(xs) & 3u) == 0 &&
                  (reinterpret_cast<uintptr_t>(hs) & 3u) == 0,
              "grouped_swiglu_w8a8: buffers must be 16-byte aligned (scale bytes: 4)");
  if (max_rows == 0) return FS2MOE_OK;
  FS2_REQUIRE(x_rows * (int64_t)D <= 0xffffffffll, "grouped_swiglu_w8a8: xq is addressed with 32-bit byte offsets");
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto k1 = glu_gemm_mx_kernel<true>;
  auto k2 = glu_gemm_mx_kernel<false>;
  static bool attr_set = false;  // benign race: setting the attribute is idempotent
  if (!attr_set) {
    const void* ks[2] = {reinterpret_cast<const void*>(k1), reinterpret_cast<const void*>(k2)};
    for (const void* k : ks) {
      hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, SMEM_BYTES);
      if (e != hipSuccess) {
        set_error("grouped_swiglu_w8a8: cannot reserve %d bytes of LDS: %s", SMEM_BYTES,
                  hipGetErrorString(e));
        return FS2MOE_ERR_LAUNCH;
      }
    }
    attr_set = true;
  }
  const int num_blocks = mx_cu_count();
  if (num_blocks == 0) {
    set_error("grouped_swiglu_w8a8: cannot query the compute-unit count");
    return FS2MOE_ERR_LAUNCH;
  }
  const int nt1 = (F + 127) / 128, nt2 = (D + 255) / 256;
  {
    const int64_t m_tiles = max_rows / BM + E + 1;
    if (m_tiles * nt1 > 0x7fffffffll || m_tiles * nt2 > 0x7fffffffll) {
      set_error("grouped_swiglu_w8a8: too many tiles");
      return FS2MOE_ERR_UNSUPPORTED;
    }
  }
  Groups g{counts, offsets, E, 0};
  hipLaunchKernelGGL(k1, dim3((unsigned)num_blocks), dim3(NWAVES * 64), SMEM_BYTES, st,
                     static_cast<const uint8_t*>(xq), static_cast<const uint8_t*>(xs), row_map,
                     static_cast<const uint8_t*>(w_gate), static_cast<const uint8_t*>(w_up), s_gate,
                     s_up, hq, static_cast<uint8_t*>(hs), F, D, F, g, nt1, (int)x_rows, (int)max_rows);
  if (int rc = check_launch("glu_gemm_mx<gate,up>")) return rc;
  hipLaunchKernelGGL(k2, dim3((unsigned)num_blocks), dim3(NWAVES * 64), SMEM_BYTES, st,
                     static_cast<const uint8_t*>(hq), static_cast<const uint8_t*>(hs),
                     static_cast<const int32_t*>(nullptr), static_cast<const uint8_t*>(w_down),
                     static_cast<const uint8_t*>(nullptr), s_down, static_cast<const float*>(nullptr),
                     ye, static_cast<uint8_t*>(nullptr), D, F, D, g, nt2, (int)max_rows, 0);
  return check_launch("glu_gemm_mx<down>");
}

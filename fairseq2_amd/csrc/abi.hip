// Library-wide pieces of the C ABI: version, thread-local error text, launch checking.
#include <cstdarg>
#include <cstdio>
#include <mutex>

#include "common.h"

namespace fs2moe {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    set_error("%s: launch failed: %s", what, hipGetErrorString(e));
    return FS2MOE_ERR_LAUNCH;
  }
  return FS2MOE_OK;
}

}  // namespace fs2moe

extern "C" int fs2moe_abi_version(void) { return FS2MOE_ABI_VERSION; }

extern "C" const char* fs2moe_last_error(void) { return fs2moe::g_error; }

// ---- the whole layer ----------------------------------------------------------------------------
namespace {

// Carves 256-byte aligned pieces out of the caller's workspace (or only adds up their sizes).
struct Carver {
  uint8_t* base;
  int64_t used = 0;
  void* take(int64_t bytes) {
    void* p = base ? base + used : nullptr;
    used += (bytes + 255) / 256 * 256;
    return p;
  }
};

struct ForwardBuffers {
  int32_t *topk_idx, *counts, *offsets, *perm, *inv_perm;
  float* topk_w;
  void *disp_ws, *router_ws, *xn, *xe, *h, *ye, *shared_h;
  // W8A8: the token rows as block-scaled e4m3 (in the place of xe) and the gated product likewise
  // (in the place of h)
  void *xq, *xs, *hq, *hs;
  // a weight per expert row (in the place of xe) where the expert kernels scale the rows themselves
  float* row_w;
  int64_t max_rows, disp_ws_bytes, router_ws_bytes, total;
};

ForwardBuffers carve_forward(void* workspace, int32_t T, int32_t D, int32_t E, int32_t K, int32_t F,
                             int32_t F_shared, int32_t tile_m, int32_t act_dtype, bool need_xe,
                             bool need_xn, bool act_q = false, bool need_row_w = false) {
  const int64_t esz = fs2moe::elem_size(act_dtype);
  ForwardBuffers b;
  b.max_rows = FS2MOE_MAX_ROWS(T, K, E, tile_m);
  b.disp_ws_bytes = fs2moe_dispatch_workspace_bytes(T, K, E);
  Carver c{static_cast<uint8_t*>(workspace)};
  b.topk_idx = static_cast<int32_t*>(c.take((int64_t)T * K * 4));
  b.topk_w = static_cast<float*>(c.take((int64_t)T * K * 4));
  b.counts = static_cast<int32_t*>(c.take((int64_t)E * 4));
  b.offsets = static_cast<int32_t*>(c.take((int64_t)(E + 1) * 4));
  b.perm = static_cast<int32_t*>(c.take(b.max_rows * 4));
  b.inv_perm = static_cast<int32_t*>(c.take((int64_t)T * K * 4));
  b.disp_ws = c.take(b.disp_ws_bytes);
  b.router_ws_bytes = fs2moe_router_workspace_bytes(T, D, E, act_dtype);
  b.router_ws = b.router_ws_bytes > 0 ? c.take(b.router_ws_bytes) : nullptr;
  b.xn = need_xn ? c.take((int64_t)T * D * esz) : nullptr;
  b.xe = need_xe ? c.take(b.max_rows * D * esz) : nullptr;
  // (4 bytes a row where the copy would have taken D elements: the workspace sized with the copy holds it)
  b.row_w = need_row_w ? static_cast<float*>(c.take(b.max_rows * 4)) : nullptr;
  b.xq = b.xs = b.hq = b.hs = nullptr;
  if (act_q) {
    // T rows of D codes and D / 32 scale bytes each: less than the row copy that is not made, so a
    // workspace of fs2moe_forward_workspace_bytes (sized with the copy) holds them
    b.xq = c.take((int64_t)T * D);
    b.xs = c.take((int64_t)T * (D / 32));
  }
  b.h = c.take(b.max_rows * F * esz);
  if (act_q) {
    // max_rows x (F codes + F / 32 scale bytes) inside the bf16 product's place
    b.hq = b.h;
    b.hs = static_cast<uint8_t*>(b.h) + (b.max_rows * F + 255) / 256 * 256;
  }
  b.ye = c.take(b.max_rows * D * esz);
  b.shared_h = F_shared > 0 ? c.take((int64_t)T * F_shared * esz) : nullptr;
  b.total = c.used;
  return b;
}

}  // namespace

extern "C" int64_t fs2moe_forward_workspace_bytes(int32_t T, int32_t D, int32_t E, int32_t K,
                                                  int32_t F, int32_t F_shared, int32_t tile_m,
                                                  int32_t act_dtype) {
  if (T < 0 || D < 1 || E < 1 || K < 1 || F < 1 || F_shared < 0 || tile_m < 1) return -1;
  // sized for the path that copies the rows: which path runs depends on the mode and the types
  return carve_forward(nullptr, T, D, E, K, F, F_shared, tile_m, act_dtype, true, false).total;
}

extern "C" int64_t fs2moe_forward_norm_workspace_bytes(int32_t T, int32_t D, int32_t E, int32_t K,
                                                       int32_t F, int32_t F_shared, int32_t tile_m,
                                                       int32_t act_dtype) {
  if (T < 0 || D < 1 || E < 1 || K < 1 || F < 1 || F_shared < 0 || tile_m < 1) return -1;
  return carve_forward(nullptr, T, D, E, K, F, F_shared, tile_m, act_dtype, true, true).total;
}

namespace {

// A stream of the library's own per device, for the shared expert of a decode step.  The shared
// expert depends on the rows only, and with a handful of tokens the routed path (the router's two
// small kernels, the dispatch, one or a few experts' weight streams) leaves most of the chip idle
// while it runs: the shared expert's two kernels go onto this stream, forked from the caller's
// stream by an event and joined back by another before the combine, so a caller sees one stream's
// worth of ordering (and a capturing stream captures both branches).  Default priority, created
// on the first use on a device and kept; the events are reused, which is why the record-and-wait
// pairs are taken under a lock: between one thread's record and its wait another thread's
// record of the same event would replace what is waited for.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  bool tried = false;
};
constexpr int kSideDevices = 64;
SideStream g_side[kSideDevices];
std::mutex g_side_mu;

// null: no such stream on this device (creation failed once); the caller then runs everything on
// its own stream.
SideStream* side_stream() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kSideDevices) return nullptr;
  std::lock_guard<std::mutex> lock(g_side_mu);
  SideStream& s = g_side[dev];
  if (!s.tried) {
    s.tried = true;
    if (hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&s.join, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();  // the failure is handled here: nothing for the next call to find
      s.stream = nullptr;
    }
  }
  return s.stream != nullptr ? &s : nullptr;
}

// normed: the rows are RMS-normalised on the way into the router (norm_weight may be null), and
// every stage reads the normalised copy in the workspace.
// may_fork: the shared expert of a few tokens may run on the library's side stream (not for the
// entry point that must create nothing).
int forward_impl(bool may_fork, bool normed, const void* x_in, const void* norm_weight, float norm_eps,
                 const void* residual, const void* router, const float* router_bias,
                 const void* w_gate, const void* w_up, const void* w_down, const float* s_gate,
                 const float* s_up, const float* s_down, const void* shared_gate,
                 const void* shared_up, const void* shared_down, int32_t T, int32_t D, int32_t E,
                 int32_t K, int32_t F, int32_t F_shared, int32_t tile_m, int32_t act_dtype,
                 int32_t w_dtype, int32_t score_fn, int32_t renormalize, int32_t scale_input,
                 void* workspace, int64_t workspace_bytes, void* out, void* stream) {
  const void* x = x_in;
  const bool act_q = (w_dtype & FS2MOE_ACT_MXFP8) != 0;
  w_dtype &= ~FS2MOE_ACT_MXFP8;
  FS2_REQUIRE(x && router && w_gate && w_up && w_down && out, "forward: null pointer");
  FS2_REQUIRE(T >= 0 && D >= 1 && E >= 1 && K >= 1 && F >= 1 && F_shared >= 0 && tile_m >= 1,
              "forward: bad sizes T=%d D=%d E=%d K=%d F=%d F_shared=%d tile_m=%d", T, D, E, K, F,
              F_shared, tile_m);
  const bool shared = shared_gate || shared_up || shared_down;
  FS2_REQUIRE(!shared || (shared_gate && shared_up && shared_down && F_shared > 0),
              "forward: the shared expert needs its three matrices and F_shared > 0");
  // the raw rows are read by the router only when they are normalised there
  FS2_REQUIRE(normed || x != out, "forward: out must not alias x");
  // the shared expert's output passes through `out` before the residual is read
  FS2_REQUIRE(!(shared && residual == out),
              "forward: with a shared expert out must not alias residual");
  const int64_t need = carve_forward(nullptr, T, D, E, K, F, shared ? F_shared : 0, tile_m,
                                     act_dtype, true, normed).total;
  FS2_REQUIRE(workspace && workspace_bytes >= need,
              "forward: workspace of %lld bytes is smaller than the %lld needed",
              (long long)workspace_bytes, (long long)need);
  FS2_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 255u) == 0,
              "forward: workspace must be 256-byte aligned");
  if (T == 0) return FS2MOE_OK;

  // rows are read through the permutation where the expert kernels can (see fs2moe_grouped_swiglu)
  const int64_t widest = (int64_t)FS2MOE_MAX_ROWS(T, K, E, tile_m) * (D > F ? D : F) * 2;
  const bool fused = !scale_input && fs2moe_grouped_swiglu_fuses_gather(D, F, act_dtype, w_dtype) &&
                     (w_dtype == FS2MOE_FP8_E4M3 || widest <= 0xffffffffll);
  if (act_q) {
    FS2_REQUIRE(w_dtype == FS2MOE_FP8_E4M3 && act_dtype == FS2MOE_BF16 && s_gate && s_up && s_down,
                "forward: FS2MOE_ACT_MXFP8 goes with e4m3 weights, their scales and bf16 rows");
    FS2_REQUIRE(!scale_input, "forward: FS2MOE_ACT_MXFP8 with scale_input is not built into this "
                              "call; use the stage calls");
    FS2_REQUIRE(fs2moe_grouped_swiglu_w8a8_supported(D, F, FS2MOE_MAX_ROWS(T, K, E, tile_m)),
                "forward: FS2MOE_ACT_MXFP8 with D=%d, F=%d: sizes the W8A8 kernels do not take "
                "(fs2moe_grouped_swiglu_w8a8_supported)", D, F);
  }
  // The reference's routing mode multiplies each row by its routing weight on the way in, which
  // dispatch does as it copies the rows.  With at most 16 bf16 tokens (a decode step) the expert
  // kernels stage a few rows in LDS and stream the weights past them: they take the row from x
  // through perm and scale it there, so that no copy is made and dispatch can run inside the router's
  // second kernel as in the other mode.
  const bool scaled_stream = scale_input && !act_q && T <= 16 && D * 2 >= 4 &&
                             fs2moe::swiglu_streams_rows(act_dtype, w_dtype, D, F, E, T);
  const ForwardBuffers b = carve_forward(workspace, T, D, E, K, F, shared ? F_shared : 0, tile_m,
                                         act_dtype, !fused && !act_q && !scaled_stream, normed, act_q,
                                         scaled_stream);
  FS2_REQUIRE(b.total <= need, "forward: internal: the buffers do not fit the workspace");
  // The shared expert's output is the row the routed outputs are added onto (moe.py:143-150).  With
  // at most 16 tokens it runs beside the routed path (see SideStream): from the start when it
  // reads the caller's rows, after the router when it reads the rows the router normalises.
  // (forking and joining cost the host four calls, about as long as a whole step of a small layer
  // takes it to launch: D 2048 / F 4096, 16 experts, one token 53 -> 100 us with them, where D 4096 /
  // F 8192 goes 137 -> 129 and Scout's D 5120 / F 8192 173 -> 156; so only where the shared expert
  // streams at least 192 MB of weights)
  const bool big_shared = (int64_t)3 * D * F_shared * fs2moe::elem_size(act_dtype) >= (192ll << 20);
  SideStream* side = (shared && may_fork && T <= 16 && big_shared) ? side_stream() : nullptr;
  const bool beside = side != nullptr && side->stream != static_cast<hipStream_t>(stream);
  auto shared_on = [&](void* s, const void* rows) {
    return fs2moe_dense_swiglu(rows, shared_gate, shared_up, shared_down, T, D, F_shared, act_dtype,
                               b.shared_h, out, s);
  };
  auto shared_beside = [&]() -> int {
    hipStream_t main = static_cast<hipStream_t>(stream);
    {
      std::lock_guard<std::mutex> lock(g_side_mu);
      if (hipEventRecord(side->fork, main) != hipSuccess ||
          hipStreamWaitEvent(side->stream, side->fork, 0) != hipSuccess) {
        fs2moe::set_error("forward: cannot fork the shared expert's stream: %s",
                          hipGetErrorString(hipGetLastError()));
        return FS2MOE_ERR_LAUNCH;
      }
    }
    return shared_on(side->stream, normed ? b.xn : x_in);
  };
  // the caller's stream goes on only when the side stream has come this far (called once the
  // routed experts are on their way, in front of the combine; and on every way out after a fork,
  // so that the side stream never stays forked from a capturing stream)
  auto shared_joins = [&]() -> int {
    std::lock_guard<std::mutex> lock(g_side_mu);
    if (hipEventRecord(side->join, side->stream) != hipSuccess ||
        hipStreamWaitEvent(static_cast<hipStream_t>(stream), side->join, 0) != hipSuccess) {
      fs2moe::set_error("forward: cannot join the shared expert's stream: %s",
                        hipGetErrorString(hipGetLastError()));
      return FS2MOE_ERR_LAUNCH;
    }
    return FS2MOE_OK;
  };
  bool forked = false;
  // router, dispatch and the routed experts, with the shared expert forked off on the way
  auto routed_path = [&]() -> int {
    if (beside && !normed) {
      forked = true;
      if (int rc = shared_beside()) return rc;
    }
    // (with a few tokens and no rows to copy the router's kernel dispatches as well)
    fs2moe::DispatchAfterRouter disp = {tile_m,     b.max_rows, b.counts,        b.offsets, b.perm,
                                        b.inv_perm, b.disp_ws,  b.disp_ws_bytes, b.row_w,   false};
    if (int rc = fs2moe::router_then_dispatch(
            x, normed ? norm_weight : nullptr, normed ? norm_eps : 0.f, normed ? b.xn : nullptr, router,
            router_bias, T, D, E, K, act_dtype, score_fn, renormalize, b.topk_idx, b.topk_w, b.router_ws,
            b.router_ws_bytes, b.xe == nullptr ? &disp : nullptr, stream))
      return rc;
    if (normed) x = b.xn;
    if (beside && normed) {
      forked = true;
      if (int rc = shared_beside()) return rc;
    }
    if (!disp.done) {
      if (scaled_stream) {
        if (int rc = fs2moe::dispatch_with_row_weights(b.topk_idx, b.topk_w, T, K, E, tile_m,
                                                       b.max_rows, b.counts, b.offsets, b.perm,
                                                       b.inv_perm, b.row_w, stream))
          return rc;
      } else if (int rc = fs2moe_dispatch(b.topk_idx, b.topk_w, x, T, K, E, D, tile_m, act_dtype,
                                          scale_input, b.max_rows, b.counts, b.offsets, b.perm,
                                          b.inv_perm, b.xe, b.disp_ws, b.disp_ws_bytes, stream)) {
        return rc;
      }
    }
    if (act_q) {
      // the token rows to block-scaled e4m3 once; both products read codes (the first through perm)
      if (int rc = fs2moe_mx_quantize(x, T, D, b.xq, b.xs, stream)) return rc;
      return fs2moe_grouped_swiglu_w8a8(b.xq, b.xs, b.perm, b.counts, b.offsets, w_gate, w_up, w_down,
                                        s_gate, s_up, s_down, E, D, F, T, b.max_rows, b.hq, b.hs, b.ye,
                                        stream);
    }
    if (scaled_stream)
      return fs2moe::grouped_swiglu_scaled_rows(x, b.perm, b.row_w, b.counts, b.offsets, w_gate, w_up,
                                                w_down, E, D, F, b.max_rows, b.h, b.ye, T, stream);
    // (a token takes an expert at most once: with up to 16 tokens no expert has more rows than that)
    return fs2moe_grouped_swiglu_rows(fused ? x : b.xe, fused ? b.perm : nullptr, b.counts, b.offsets,
                                      w_gate, w_up, w_down, s_gate, s_up, s_down, E, D, F, b.max_rows,
                                      act_dtype, w_dtype, b.h, b.ye, T <= 16 ? T : 0, stream);
  };
  int rc_routed = routed_path();
  if (forked) {
    const int rc_join = shared_joins();
    if (rc_routed == FS2MOE_OK) rc_routed = rc_join;
  }
  if (rc_routed != FS2MOE_OK) return rc_routed;
  const void* base = nullptr;
  if (shared) {
    if (!beside)
      if (int rc = shared_on(stream, x)) return rc;
    base = out;
  }
  if (residual != nullptr)
    return fs2moe_combine_residual(b.ye, b.inv_perm, b.topk_idx, b.topk_w, base, residual, T, K, D,
                                   act_dtype, scale_input ? 0 : 1, out, stream);
  return fs2moe_combine(b.ye, b.inv_perm, b.topk_idx, b.topk_w, base, T, K, D, act_dtype,
                        scale_input ? 0 : 1, out, stream);
}

}  // namespace

extern "C" int fs2moe_forward(const void* x, const void* residual, const void* router,
                              const float* router_bias,
                              const void* w_gate, const void* w_up, const void* w_down,
                              const float* s_gate, const float* s_up, const float* s_down,
                              const void* shared_gate, const void* shared_up,
                              const void* shared_down, int32_t T, int32_t D, int32_t E, int32_t K,
                              int32_t F, int32_t F_shared, int32_t tile_m, int32_t act_dtype,
                              int32_t w_dtype, int32_t score_fn, int32_t renormalize,
                              int32_t scale_input, void* workspace, int64_t workspace_bytes,
                              void* out, void* stream) {
  return forward_impl(true, false, x, nullptr, 0.f, residual, router, router_bias, w_gate, w_up, w_down,
                      s_gate, s_up, s_down, shared_gate, shared_up, shared_down, T, D, E, K, F,
                      F_shared, tile_m, act_dtype, w_dtype, score_fn, renormalize, scale_input,
                      workspace, workspace_bytes, out, stream);
}

extern "C" int fs2moe_forward_norm(const void* x, const void* norm_weight, float norm_eps,
                                   const void* residual, const void* router,
                                   const float* router_bias,
                                   const void* w_gate, const void* w_up, const void* w_down,
                                   const float* s_gate, const float* s_up, const float* s_down,
                                   const void* shared_gate, const void* shared_up,
                                   const void* shared_down, int32_t T, int32_t D, int32_t E,
                                   int32_t K, int32_t F, int32_t F_shared, int32_t tile_m,
                                   int32_t act_dtype, int32_t w_dtype, int32_t score_fn,
                                   int32_t renormalize, int32_t scale_input, void* workspace,
                                   int64_t workspace_bytes, void* out, void* stream) {
  return forward_impl(true, true, x, norm_weight, norm_eps, residual, router, router_bias, w_gate, w_up,
                      w_down, s_gate, s_up, s_down, shared_gate, shared_up, shared_down, T, D, E, K,
                      F, F_shared, tile_m, act_dtype, w_dtype, score_fn, renormalize, scale_input,
                      workspace, workspace_bytes, out, stream);
}

// ---- the whole layer for callers that cannot allocate ----------------------------------------------
// Every intermediate of fs2moe_forward lives in one array inside the library's own device image, so
// the call needs no workspace from the caller and never touches an allocator.  Every device the
// library runs on holds its own copy of the array, at its own address, until the process ends.
namespace {

static __device__ __align__(256) unsigned char scratch[FS2MOE_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
// Device address of `scratch` on each device, looked up once per device with that device current.
// Plain word-sized stores of the same value: a race between two first calls is benign.
void* g_scratch_ptr[kMaxDevices] = {};

// The address of this device's copy of the array (the array's name is only a host-side handle and
// must never reach a kernel), or null with the error text set.
void* static_scratch() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fs2moe::set_error("forward_static: cannot identify the current device (%s, device %d)",
                      hipGetErrorString(e), dev);
    return nullptr;
  }
  void* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (p != nullptr) return p;
  e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
  if (e != hipSuccess || p == nullptr) {
    fs2moe::set_error("forward_static: hipGetSymbolAddress failed on device %d: %s", dev,
                      hipGetErrorString(e));
    return nullptr;
  }
  __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);
  return p;
}

}  // namespace

extern "C" int64_t fs2moe_forward_static_capacity(void) { return FS2MOE_STATIC_SCRATCH_BYTES; }

extern "C" int fs2moe_forward_static(const void* x, const void* residual, const void* router,
                                     const float* router_bias, const void* w_gate,
                                     const void* w_up, const void* w_down, const float* s_gate,
                                     const float* s_up, const float* s_down,
                                     const void* shared_gate, const void* shared_up,
                                     const void* shared_down, int32_t T, int32_t D, int32_t E,
                                     int32_t K, int32_t F, int32_t F_shared, int32_t tile_m,
                                     int32_t act_dtype, int32_t w_dtype, int32_t score_fn,
                                     int32_t renormalize, int32_t scale_input, void* out,
                                     void* stream) {
  const int64_t need = fs2moe_forward_workspace_bytes(T, D, E, K, F, F_shared, tile_m, act_dtype);
  FS2_REQUIRE(need >= 0, "forward_static: bad sizes T=%d D=%d E=%d K=%d F=%d F_shared=%d tile_m=%d",
              T, D, E, K, F, F_shared, tile_m);
  FS2_REQUIRE(need <= (int64_t)FS2MOE_STATIC_SCRATCH_BYTES,
              "forward_static: these sizes need %lld bytes of scratch, the built-in array holds "
              "%lld; use fs2moe_forward with a workspace of the caller's",
              (long long)need, (long long)FS2MOE_STATIC_SCRATCH_BYTES);
  void* ws = static_scratch();
  if (ws == nullptr) return FS2MOE_ERR_LAUNCH;
  // Every stage writes what it later reads (nothing in the workspace has to start at zero), so the
  // previous call's contents need no clearing.
  // (everything on the caller's stream: this entry point creates nothing, streams included)
  return forward_impl(false, false, x, nullptr, 0.f, residual, router, router_bias, w_gate, w_up,
                      w_down, s_gate, s_up, s_down, shared_gate, shared_up, shared_down, T, D, E, K,
                      F, F_shared, tile_m, act_dtype, w_dtype, score_fn, renormalize, scale_input, ws,
                      FS2MOE_STATIC_SCRATCH_BYTES, out, stream);
}

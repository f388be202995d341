/*
 * fs2moe — C ABI of the MI355X (gfx950) mixture-of-experts feed-forward forward path.
 *
 * The reference (fairseq2) has no foreign-function boundary on this path: its MoE layer is a
 * sequence of stock torch operators.  Each entry point below therefore replaces one group of those
 * operator calls, cited as file:line relative to the fairseq2 source tree, and a host binding
 * (Python/ctypes in this repository) strings them together behind the reference module's
 * constructor and forward(seqs) interface.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; the library never allocates, frees or
 *     synchronises, and launches all work on the given stream (a hipStream_t passed as void*);
 *   - tensors are dense and row-major, last dimension contiguous, 16-byte aligned;
 *   - return value 0 = success, negative = error (see fs2moe_last_error, thread-local text);
 *   - T tokens, D model dim, E experts, K experts per token, F expert inner dim;
 *   - "rows" are the (expert, token) pairs in expert-major, token-ascending order, each expert's
 *     block rounded up to tile_m rows.  FS2MOE_MAX_ROWS(T,K,E,tile_m) bounds their number, so the
 *     caller can size buffers without reading anything back from the device.
 */
#ifndef FS2MOE_H_
#define FS2MOE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FS2MOE_ABI_VERSION 15

/* element types */
#define FS2MOE_F32 0
#define FS2MOE_BF16 1
#define FS2MOE_FP8_E4M3 2 /* OCP e4m3fn codes, weights only, with per-output-channel f32 scales */
/* May be OR-ed into the w_dtype argument of the whole-layer calls next to FS2MOE_FP8_E4M3: the expert
 * products then run on the fp8 matrix pipe (W8A8), the rows rounded to block-scaled e4m3 on the way
 * (fs2moe_mx_quantize, fs2moe_grouped_swiglu_w8a8 inside the call; an opt-in with no counterpart in
 * the reference).  Accepted for bf16 activations, scale_input 0 and sizes for which
 * fs2moe_grouped_swiglu_w8a8_supported(D, F, FS2MOE_MAX_ROWS(T, K, E, tile_m)) returns 1. */
#define FS2MOE_ACT_MXFP8 0x100

/* router score functions */
#define FS2MOE_SCORE_SIGMOID 0 /* reference: sigmoid of the selected raw logit (moe.py:113,127) */
#define FS2MOE_SCORE_SOFTMAX 1 /* extension: softmax over all experts */
/* May be OR-ed into a score_fn argument: `router` then points at an (E, D) matrix (each expert's
 * weights contiguous: the transpose of the reference's parameter, e.g. a copy the caller keeps and
 * refreshes when the parameter changes) instead of (D, E).  Read that way the router's bf16 kernel
 * needs no transposing reads.  Accepted only where fs2moe_router_takes_out_in returns 1. */
#define FS2MOE_ROUTER_OUT_IN 0x100

/* weight orientation of a GLU network */
#define FS2MOE_W_IN_OUT 0 /* (E*in, out), out contiguous: grouped experts (experts.py:53-82) */
#define FS2MOE_W_OUT_IN 1 /* (out, in), in contiguous: nn.Linear, the shared expert (ffn.py:302-347) */

/* limits */
#define FS2MOE_MAX_EXPERTS 512
#define FS2MOE_MAX_TOP_K 32

/* bytes of the library's built-in scratch array (fs2moe_forward_static) */
#define FS2MOE_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)

/* error codes */
#define FS2MOE_OK 0
#define FS2MOE_ERR_ARG (-1)     /* null pointer, size or enum out of range, misalignment */
#define FS2MOE_ERR_UNSUPPORTED (-2) /* valid request this build has no kernel for */
#define FS2MOE_ERR_LAUNCH (-3)  /* the HIP runtime refused a launch */

/* upper bound on the number of tile-padded rows */
#define FS2MOE_MAX_ROWS(T, K, E, tile_m) \
  ((int64_t)(T) * (K) + (int64_t)(E) * ((tile_m) - 1))

int fs2moe_abi_version(void);
const char* fs2moe_last_error(void);

/*
 * Router: logits = x @ router (+ bias); per token the K largest logits (descending; ties to the
 * lower expert id; NaN ranks highest) and their combine weights.
 * Replaces moe.py:104-127 (matmul, torch.topk, dense score matrix, sigmoid).
 *   x        [T, D]  act_dtype           router [D, E] act_dtype      bias [E] f32 or NULL
 *   topk_idx [T, K]  int32 (out)         topk_w [T, K] f32 (out)      logits [T, E] f32 (out) or NULL
 * score_fn SIGMOID: w = sigmoid(logit) (divided by the selected sum if renormalize).
 * score_fn SOFTMAX: w = softmax over all E, or over the K selected logits if renormalize.
 * workspace: optional device scratch of fs2moe_router_workspace_bytes(...) bytes, 16-byte aligned.
 *   With few tokens (up to 4096, bf16) several blocks then share a token tile, each summing a range
 *   of D into the workspace, and a second kernel adds the ranges and selects; without it (NULL, or
 *   fewer bytes) one block per 32 tokens walks all of D.  The logits of the two ways differ by f32
 *   summation order only.
 */
int64_t fs2moe_router_workspace_bytes(int32_t T, int32_t D, int32_t E, int32_t act_dtype);
/* 1 if the router of this size reads an (E, D) matrix when FS2MOE_ROUTER_OUT_IN is set (bf16, D a
 * multiple of 128, E a multiple of 8 up to 256, enough tokens that every token tile of 32 has a block
 * of its own: more than 4096, or a narrow model), else 0: then pass (D, E).
 * No counterpart in the reference (its router parameter is (D, E): llama4/moe.py:75-77). */
int32_t fs2moe_router_takes_out_in(int32_t T, int32_t D, int32_t E, int32_t act_dtype);
int fs2moe_router_topk(const void* x, const void* router, const float* bias, int32_t T, int32_t D,
                       int32_t E, int32_t K, int32_t act_dtype, int32_t score_fn,
                       int32_t renormalize, int32_t* topk_idx, float* topk_w, float* logits,
                       void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Router with the RMS normalisation of the calling pre-norm decoder layer in front of it: every row
 * of x is normalised into xn on the way, and xn is what is routed (and what the later stages must
 * be given as their activations).
 * Replaces the ffn_layer_norm call of models/transformer_lm/decoder_layer.py:187-191 (RMSNorm,
 * nn/normalization.py:234-236, i.e. torch.nn.functional.rms_norm) together with moe.py:104-127.
 *   xn = round(x * rsqrt(mean(x^2) + eps) * weight): mean and both products in f32, one rounding
 *   to act_dtype.
 *   x [T, D] act_dtype   norm_weight [D] act_dtype or NULL (no elementwise weight)
 *   xn [T, D] act_dtype (out; must not alias x)       the rest as for fs2moe_router_topk
 */
int fs2moe_router_topk_norm(const void* x, const void* norm_weight, float norm_eps, void* xn,
                            const void* router, const float* bias, int32_t T, int32_t D, int32_t E,
                            int32_t K, int32_t act_dtype, int32_t score_fn, int32_t renormalize,
                            int32_t* topk_idx, float* topk_w, float* logits, void* workspace,
                            int64_t workspace_bytes, void* stream);

/*
 * Host mirror of the router's selection: from a token's logits (HOST memory, bias included, e.g. the
 * `logits` output of fs2moe_router_topk copied back) the K experts and their weights, by the rule the
 * device applies (descending; ties to the lower expert id; NaN highest; -0 = +0).  The indices equal
 * the device's bit for bit, near-ties included; the weights agree to float rounding.  Runs on the
 * CPU and touches no GPU: it is what lets a test or an integrator verify the routing exactly where
 * two logits are closer than the accumulation error of any reference matmul.
 * Replaces torch.topk and the score function of moe.py:113-127 on given logits.
 *   logits [T, E] f32 (host)     topk_idx [T, K] int32 (host, out)     topk_w [T, K] f32 (host, out)
 */
int fs2moe_cpu_router_select(const float* logits, int32_t T, int32_t E, int32_t K, int32_t score_fn,
                             int32_t renormalize, int32_t* topk_idx, float* topk_w);

/*
 * Bytes of device scratch fs2moe_dispatch needs (per-block histograms and ranks; the whole-layer
 * calls use the same bytes for the histograms their router kernel writes per 32 tokens).
 */
int64_t fs2moe_dispatch_workspace_bytes(int32_t T, int32_t K, int32_t E);

/*
 * Dispatch: per-expert histogram, tile-padded exclusive scan, stable permutation, row gather.
 * Replaces moe.py:115-134 (the (E,T) score matrix, the tiled arange, gather and input scaling) with
 * the sparse equivalent: only the T*K selected pairs are materialised.
 *   counts   [E]     int32 (out)   tokens per expert
 *   offsets  [E+1]   int32 (out)   first row of each expert; offsets[E] = number of padded rows
 *   perm     [max_rows] int32 (out) token of each row, -1 on padding rows and beyond offsets[E]
 *   inv_perm [T, K]  int32 (out)   row of pair (t, slot)
 *   xe       [max_rows, D] act_dtype (out) x[perm[row]] (times its weight if scale_input), zeros on
 *            padding rows; may be NULL to skip the gather
 *   max_rows must be >= FS2MOE_MAX_ROWS(T,K,E,tile_m).
 */
int fs2moe_dispatch(const int32_t* topk_idx, const float* topk_w, const void* x, int32_t T,
                    int32_t K, int32_t E, int32_t D, int32_t tile_m, int32_t act_dtype,
                    int32_t scale_input, int64_t max_rows, int32_t* counts, int32_t* offsets,
                    int32_t* perm, int32_t* inv_perm, void* xe, void* workspace,
                    int64_t workspace_bytes, void* stream);

/*
 * Grouped SwiGLU experts: for every expert e and each of its rows,
 *   ye[row] = (SiLU(xe[row] @ Wg_e) * (xe[row] @ Wu_e)) @ Wd_e.
 * Replaces experts.py:90-114 (three torch.bmm and the SiLU gate) on the routed rows only.
 *   xe [max_rows, D] act_dtype     counts [E], offsets [E+1] as written by fs2moe_dispatch
 *   row_map [max_rows] int32 or NULL.  When given, xe is the token matrix x [T, D] itself and row r
 *     of the experts' input is x[row_map[r]] (pass fs2moe_dispatch's perm): the gather of moe.py:131
 *     is fused into the first GEMM's loads and fs2moe_dispatch can be called with xe = NULL.  Only
 *     where fs2moe_grouped_swiglu_fuses_gather says so, only for unscaled rows (scale_input = 0),
 *     and, with weights in the activation dtype, only while max_rows * max(D, F) * 2 bytes stay
 *     below 4 GB (FS2MOE_ERR_UNSUPPORTED otherwise: gather the rows with fs2moe_dispatch instead).
 *   w_gate, w_up [E*D, F], w_down [E*F, D] in w_dtype, orientation FS2MOE_W_IN_OUT;
 *     for FS2MOE_FP8_E4M3 (bf16 activations, D and F multiples of 64) the codes are tiled
 *     [E][out/16][in/64][16][64] -- 1 KB tiles of 16 output channels x 64 input features, i.e.
 *     gate/up [E][F/16][D/64][16][64], down [E][D/16][F/64][16][64] -- and s_gate, s_up [E, F],
 *     s_down [E, D] are the per-output-channel f32 scales (NULL otherwise)
 *   h  [max_rows, F] act_dtype (scratch, out)     ye [max_rows, D] act_dtype (out)
 */
int fs2moe_grouped_swiglu(const void* xe, const int32_t* row_map, const int32_t* counts,
                          const int32_t* offsets, const void* w_gate, const void* w_up,
                          const void* w_down, const float* s_gate, const float* s_up,
                          const float* s_down, int32_t E, int32_t D, int32_t F, int64_t max_rows,
                          int32_t act_dtype, int32_t w_dtype, void* h, void* ye, void* stream);

/*
 * fs2moe_grouped_swiglu for a caller that knows an upper bound on the rows of any one expert
 * (rows_per_expert; 0: no bound known, then this is fs2moe_grouped_swiglu).  The number of tokens is
 * such a bound (torch.topk of moe.py:113 gives a token an expert at most once), which is what a
 * decode step of a few sequences (generation/: one token per sequence and step) has to offer: with
 * a bound of 1..16 and bf16 weights the two products run as streams over the active experts' weights
 * (no LDS tiles; up to 4 rows on the vector ALUs, 5..16 on the matrix pipe) instead of as GEMM tiles
 * (larger bounds: as 0).  Same arguments and
 * results (to the order of f32 additions) otherwise; a count above the bound is still computed
 * correctly, only slowly.
 */
int fs2moe_grouped_swiglu_rows(const void* xe, const int32_t* row_map, const int32_t* counts,
                               const int32_t* offsets, const void* w_gate, const void* w_up,
                               const void* w_down, const float* s_gate, const float* s_up,
                               const float* s_down, int32_t E, int32_t D, int32_t F,
                               int64_t max_rows, int32_t act_dtype, int32_t w_dtype, void* h,
                               void* ye, int32_t rows_per_expert, void* stream);

/* 1 if fs2moe_grouped_swiglu accepts a row_map for these sizes and types, else 0. */
int fs2moe_grouped_swiglu_fuses_gather(int32_t D, int32_t F, int32_t act_dtype, int32_t w_dtype);

/*
 * Dense SwiGLU network on all T tokens (the shared expert):
 *   y = (SiLU(x @ Wg^T) * (x @ Wu^T)) @ Wd^T  with nn.Linear-oriented weights.
 * Replaces moe.py:143-145 -> ffn.py:374-395 (three F.linear and the SiLU gate).
 *   x [T, D]   w_gate, w_up [F, D]   w_down [D, F]   h [T, F] scratch   y [T, D] (out)
 * Up to 16 bf16 rows (a decode step) run as a stream over the three matrices instead of as GEMM
 * tiles; the results differ from the tiles' only in the order of the f32 additions.
 */
int fs2moe_dense_swiglu(const void* x, const void* w_gate, const void* w_up, const void* w_down,
                        int32_t T, int32_t D, int32_t F, int32_t act_dtype, void* h, void* y,
                        void* stream);

/*
 * Combine: out[t] = base[t] + sum over the token's K experts, in ascending expert id, of
 * ye[inv_perm[t, slot]] (times topk_w[t, slot] if weight_output), accumulated in f32.
 * Replaces moe.py:147-150 (zeros_like / shared output and scatter_add_).
 *   base [T, D] act_dtype or NULL (zeros)     out [T, D] act_dtype (may alias base)
 */
int fs2moe_combine(const void* ye, const int32_t* inv_perm, const int32_t* topk_idx,
                   const float* topk_w, const void* base, int32_t T, int32_t K, int32_t D,
                   int32_t act_dtype, int32_t weight_output, void* out, void* stream);

/*
 * Combine with the residual connection of the calling decoder layer folded in:
 *   out[t] = residual[t] + base[t] + sum ...  (one f32 accumulation, one rounding).
 * Replaces moe.py:147-150 together with the addition that follows the feed-forward network in
 * models/transformer_lm/decoder_layer.py:188-204 (AdditiveResidualConnect, nn/residual.py:42-47).
 *   residual [T, D] act_dtype; out may alias base or residual.
 */
int fs2moe_combine_residual(const void* ye, const int32_t* inv_perm, const int32_t* topk_idx,
                            const float* topk_w, const void* base, const void* residual, int32_t T,
                            int32_t K, int32_t D, int32_t act_dtype, int32_t weight_output,
                            void* out, void* stream);

/*
 * The whole layer in one call: router, dispatch, grouped experts, shared expert (if its weights are
 * given) and combine, on the given stream, with every intermediate in the caller's workspace.
 * Replaces MoE.forward (moe.py:94-157) for a host that does not want to string the stages together
 * itself; the result is what the five calls above give, bit for bit (they are what it calls).
 *   x [T, D] act_dtype            router [D, E] act_dtype          router_bias [E] f32 or NULL
 *   residual [T, D] act_dtype or NULL: added to the output as in fs2moe_combine_residual
 *   w_gate, w_up, w_down, s_*     as for fs2moe_grouped_swiglu; w_dtype FS2MOE_FP8_E4M3 | FS2MOE_ACT_MXFP8
 *               runs the experts as fs2moe_grouped_swiglu_w8a8 does (the quantised rows take the
 *               place of the row copy in the workspace, whose size does not change)
 *   shared_gate, shared_up [F_shared, D], shared_down [D, F_shared] act_dtype, or all NULL
 *   scale_input 1: combine weights multiply the experts' input rows (the reference, moe.py:132-134);
 *               0: they multiply the experts' output rows
 *   workspace   at least fs2moe_forward_workspace_bytes(...) bytes, 256-byte aligned
 *   out [T, D] act_dtype (out; must not alias x; may alias residual unless there is a shared expert)
 * With a large shared expert (192 MB of weights or more) and at most 16 tokens its kernels run on a stream of the
 * library's own, forked from `stream` and joined back to it inside the call (events; under stream
 * capture both branches are captured): to the caller the call is ordered on `stream` as before.
 */
int64_t fs2moe_forward_workspace_bytes(int32_t T, int32_t D, int32_t E, int32_t K, int32_t F,
                                       int32_t F_shared, int32_t tile_m, int32_t act_dtype);
int fs2moe_forward(const void* x, const void* residual, const void* router,
                   const float* router_bias, const void* w_gate,
                   const void* w_up, const void* w_down, const float* s_gate, const float* s_up,
                   const float* s_down, const void* shared_gate, const void* shared_up,
                   const void* shared_down, int32_t T, int32_t D, int32_t E, int32_t K, int32_t F,
                   int32_t F_shared, int32_t tile_m, int32_t act_dtype, int32_t w_dtype,
                   int32_t score_fn, int32_t renormalize, int32_t scale_input, void* workspace,
                   int64_t workspace_bytes, void* out, void* stream);

/*
 * The whole layer preceded by the RMS normalisation of a pre-norm decoder layer:
 *   out = [residual +] MoE(RMSNorm(x))
 * i.e. with residual = x the whole feed-forward step of
 * models/transformer_lm/decoder_layer.py:187-204 in one call.  The router normalises the rows on
 * the way (fs2moe_router_topk_norm) into the workspace and all later stages read that copy.
 *   norm_weight [D] act_dtype or NULL     norm_eps >= 0     everything else as for fs2moe_forward
 *   workspace   at least fs2moe_forward_norm_workspace_bytes(...) bytes, 256-byte aligned
 *   out may alias x (the raw rows are read by the router only) and residual, but with a shared
 *   expert it must not alias residual.
 */
int64_t fs2moe_forward_norm_workspace_bytes(int32_t T, int32_t D, int32_t E, int32_t K, int32_t F,
                                            int32_t F_shared, int32_t tile_m, int32_t act_dtype);
int fs2moe_forward_norm(const void* x, const void* norm_weight, float norm_eps,
                        const void* residual, const void* router, const float* router_bias,
                        const void* w_gate, const void* w_up, const void* w_down,
                        const float* s_gate, const float* s_up, const float* s_down,
                        const void* shared_gate, const void* shared_up, const void* shared_down,
                        int32_t T, int32_t D, int32_t E, int32_t K, int32_t F, int32_t F_shared,
                        int32_t tile_m, int32_t act_dtype, int32_t w_dtype, int32_t score_fn,
                        int32_t renormalize, int32_t scale_input, void* workspace,
                        int64_t workspace_bytes, void* out, void* stream);

/*
 * W8A8: the experts on the fp8 matrix pipe, an opt-in of this library with no counterpart in the
 * reference (its experts run in the parameters' dtype, models/transformer/experts.py:102-112).
 * Weights are the e4m3 codes and per-output-channel scales of fs2moe_grouped_swiglu (w_dtype
 * FS2MOE_FP8_E4M3); activations are e4m3 codes with one power-of-two scale per row and block of 32
 * consecutive features, stored as the exponent byte X + 127:
 *     X = the smallest integer with max|block| / 2^X <= 448   (-127 for a zero block)
 *     code = e4m3(value / 2^X), round to nearest even         value ~ code * 2^X
 *
 * Scale bytes are stored k-group major, [features / 128][rows][4]: the four blocks of 128
 * consecutive features of a row form one dword, and the dwords of consecutive rows are consecutive
 * (what a kernel reads per step is exactly that dword of each of its rows).
 *
 * fs2moe_mx_quantize: x [rows, D] bf16 -> codes [rows, D] (1 byte each) and scales [D / 128][rows][4];
 *   D a multiple of 128.
 * fs2moe_grouped_swiglu_w8a8: the grouped SwiGLU network of fs2moe_grouped_swiglu on such rows.
 *   xq [x_rows, D] codes, xs [D / 128][x_rows][4] scales, both read through row_map [max_rows] when it
 *   is given (the gather of moe.py:131 fused into the first product; x_rows = T), else expert-major
 *   (x_rows = max_rows);
 *   hq [max_rows, F] / hs [F / 128][max_rows][4]: the gated product, quantised the same way by the
 *   first kernel's epilogue (from its f32 values) and read by the second; ye [max_rows, D] bf16.
 *   D and F multiples of 128 (fs2moe_grouped_swiglu_w8a8_supported says whether sizes qualify).
 */
int fs2moe_mx_quantize(const void* x, int64_t rows, int32_t D, void* codes, void* scales,
                       void* stream);
int fs2moe_grouped_swiglu_w8a8_supported(int32_t D, int32_t F, int64_t max_rows);
int fs2moe_grouped_swiglu_w8a8(const void* xq, const void* xs, const int32_t* row_map,
                               const int32_t* counts, const int32_t* offsets, const void* w_gate,
                               const void* w_up, const void* w_down, const float* s_gate,
                               const float* s_up, const float* s_down, int32_t E, int32_t D,
                               int32_t F, int64_t x_rows, int64_t max_rows, void* hq, void* hs,
                               void* ye, void* stream);

/*
 * The whole layer without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  Same computation and result as fs2moe_forward, bit for bit; the
 * intermediates live in a FS2MOE_STATIC_SCRATCH_BYTES array inside the library's device image (one
 * copy per GPU, held until the process ends), and the call makes no allocation of any kind.
 *   Sizes whose fs2moe_forward_workspace_bytes(...) exceed fs2moe_forward_static_capacity() are
 *   rejected with FS2MOE_ERR_ARG (decode-sized batches fit; prefill-sized ones do not).
 *   All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 *   streams or threads) race and must be serialised by the caller.
 *   The first call on a device looks up the array's address and sets kernel attributes (host-side
 *   work, no allocation): make it once outside any stream capture before capturing later calls.
 */
int64_t fs2moe_forward_static_capacity(void);
int fs2moe_forward_static(const void* x, const void* residual, const void* router,
                          const float* router_bias, const void* w_gate, const void* w_up,
                          const void* w_down, const float* s_gate, const float* s_up,
                          const float* s_down, const void* shared_gate, const void* shared_up,
                          const void* shared_down, int32_t T, int32_t D, int32_t E, int32_t K,
                          int32_t F, int32_t F_shared, int32_t tile_m, int32_t act_dtype,
                          int32_t w_dtype, int32_t score_fn, int32_t renormalize,
                          int32_t scale_input, void* out, void* stream);

/*
 * ---- Backward pass ------------------------------------------------------------------------------
 * The reference layer is differentiated by torch.autograd (the trainer calls backward on the loss,
 * trainer.py:586-587); the entry points below, together with fs2moe_dispatch (the gather of output
 * gradients into expert order) and fs2moe_combine (the scatter of input gradients back to token
 * order), are what that derivation needs of the device.
 *
 * One grouped GEMM: c[r] = a[r] @ B_e for the rows r of every expert e.
 * Replaces one torch.bmm of experts.py:107-112, or its transpose in the backward pass (the input
 * gradient of x @ W is dy @ W^T: the same weights read in the other orientation), or one F.linear of
 * ffn.py:374-395.
 *   a [rows, K] dtype (through row_map as in fs2moe_grouped_swiglu, when given)
 *   b  FS2MOE_W_IN_OUT: [E*K, N], FS2MOE_W_OUT_IN: [E*N, K]          c [max_rows, N] dtype (out)
 *   counts/offsets NULL: one matrix (E = 1) and max_rows rows.  K and N multiples of 8.
 */
int fs2moe_grouped_gemm(const void* a, const int32_t* row_map, const int32_t* counts,
                        const int32_t* offsets, const void* b, int32_t b_layout, int32_t E, int32_t K,
                        int32_t N, int64_t max_rows, int32_t dtype, void* c, void* stream);

/*
 * Two grouped GEMMs into one result: c[r] = a1[r] @ B1_e^T + a2[r] @ B2_e^T for the rows r of every
 * expert e, accumulated in f32 and rounded once.  The input gradient of the gate/up pair of
 * experts.py:107-112 (x @ gate_proj and x @ inner_proj share x, so their input gradients add).
 *   a1, a2 [rows, K] bf16; b1, b2 [E*N, K] bf16 (FS2MOE_W_OUT_IN); c [max_rows, N] bf16 (out).
 *   bf16 only, K a multiple of 64, N of 8, matrices below 4 GB: fs2moe_grouped_gemm_sum_supported
 *   says 1; otherwise FS2MOE_ERR_UNSUPPORTED (two fs2moe_grouped_gemm calls and an addition do it).
 */
int fs2moe_grouped_gemm_sum_supported(int32_t K, int32_t N, int64_t max_rows, int32_t dtype);
int fs2moe_grouped_gemm_sum(const void* a1, const void* b1, const void* a2, const void* b2,
                            const int32_t* counts, const int32_t* offsets, int32_t E, int32_t K,
                            int32_t N, int64_t max_rows, int32_t dtype, void* c, void* stream);

/*
 * fs2moe_grouped_swiglu for the forward pass of a training step: also stores the two products
 * g = xe @ W_gate and u = xe @ W_up (rounded to the activation dtype), which autograd keeps for the
 * backward pass of ffn.py:374-395 / experts.py:107-112 (the inputs of SiLU and of the product).
 * The backward pass can compute them again with two fs2moe_grouped_gemm calls instead; keeping them
 * costs 2 * rows * F elements of memory and saves those two products.
 *   bf16 activations and weights (reference layout), D and F multiples of 64, activation matrices
 *   below 4 GB: fs2moe_grouped_swiglu_keeps says 1; otherwise FS2MOE_ERR_UNSUPPORTED.
 *   g, u [max_rows, F] (out); everything else as for fs2moe_grouped_swiglu.
 */
int fs2moe_grouped_swiglu_keeps(int32_t D, int32_t F, int64_t max_rows, int32_t act_dtype);
/* The same for the shared expert (fs2moe_dense_swiglu; max_rows = T in fs2moe_grouped_swiglu_keeps). */
int fs2moe_dense_swiglu_keep(const void* x, const void* w_gate, const void* w_up,
                             const void* w_down, int32_t T, int32_t D, int32_t F, int32_t act_dtype,
                             void* g, void* u, void* h, void* y, void* stream);
int fs2moe_grouped_swiglu_keep(const void* xe, const int32_t* row_map, const int32_t* counts,
                               const int32_t* offsets, const void* w_gate, const void* w_up,
                               const void* w_down, int32_t E, int32_t D, int32_t F,
                               int64_t max_rows, int32_t act_dtype, void* g, void* u, void* h,
                               void* ye, void* stream);

/*
 * Weight gradient: dw_e [M, N] = A_e^T @ B_e, the contraction running over the rows of expert e
 * (zero for an expert without rows).  What autograd derives for the weights of experts.py:107-112
 * (A = the experts' input rows or h, B = the gradient of the product) and of ffn.py:374-395.
 *   a [rows, M] dtype (row r read from a[a_row_map[r]] when a_row_map is given)   b [rows, N] dtype
 *   dw [E*M, N] dtype (out).  M and N multiples of 8 (bf16) or 4 (f32).
 *   workspace: optional device scratch of fs2moe_grouped_wgrad_workspace_bytes(grouped, ...) bytes,
 *   16-byte aligned (grouped = 0 when counts is NULL).  One group with few output tiles (the router's
 *   gradient) then has its rows cut into segments whose f32 partial sums a second kernel adds in
 *   order; without it (NULL, or fewer bytes) each tile walks all rows.
 */
int64_t fs2moe_grouped_wgrad_workspace_bytes(int32_t grouped, int32_t M, int32_t N,
                                             int64_t max_rows);
int fs2moe_grouped_wgrad(const void* a, const int32_t* a_row_map, const void* b,
                         const int32_t* counts, const int32_t* offsets, int32_t E, int32_t M,
                         int32_t N, int64_t max_rows, int32_t dtype, void* dw, void* workspace,
                         int64_t workspace_bytes, void* stream);

/*
 * SwiGLU backward, element-wise: h = SiLU(g) * u, dg = dh * u * SiLU'(g), du = dh * SiLU(g).
 * The derivative of experts.py:110-111 / ffn.py:384-391.  h, dg, du may alias g, u, dh element for
 * element.     all [rows, F] dtype
 */
int fs2moe_swiglu_backward(const void* g, const void* u, const void* dh, int64_t rows, int32_t F,
                           int32_t dtype, void* h, void* dg, void* du, void* stream);

/*
 * Gradient of the combine weights: out[t, k] = <a[a_rows[t, k]] (+ a2[a_rows[t, k]]), b[t]> in f32.
 * The derivative of the scaling of moe.py:132-134 (a = the gradient of the scaled rows, b = x) or,
 * when the weights scale the experts' output, of the weighted sum (a = ye, b = the output gradient).
 *   a, a2 [rows, D] dtype (a2 may be NULL)   a_rows [T, K] int32   b [T, D] dtype   out [T, K] f32
 */
int fs2moe_pair_dot(const void* a, const void* a2, const int32_t* a_rows, const void* b, int32_t T,
                    int32_t K, int32_t D, int32_t dtype, float* out, void* stream);

/*
 * Router backward: gradient of the K combine weights -> gradient of all E logits of each token
 * (zero where the score function does not reach).  The derivative of moe.py:113-127 with the score
 * functions of fs2moe_router_topk.
 *   logits [T, E] f32 (as written by fs2moe_router_topk)   topk_idx [T, K]   topk_w, d_w [T, K] f32
 *   dlogits [T, E] dtype (out)
 */
int fs2moe_router_backward(const float* logits, const int32_t* topk_idx, const float* topk_w,
                           const float* d_w, int32_t T, int32_t E, int32_t K, int32_t score_fn,
                           int32_t renormalize, int32_t dtype, void* dlogits, void* stream);

/*
 * Backward of the RMS normalisation that fs2moe_router_topk_norm / fs2moe_forward_norm put in front
 * of the layer: y = x * rsqrt(mean(x^2) + eps) * weight.  What autograd derives for
 * torch.nn.functional.rms_norm (nn/normalization.py:234-236), the ffn_layer_norm call of
 * models/transformer_lm/decoder_layer.py:187-191.
 *   dx[t] = r_t * (dy[t] * weight) - x[t] * r_t^3 * <dy[t] * weight, x[t]> / D
 *   dweight[j] = sum over t (ascending, in up to 256 slabs) of dy[t, j] * x[t, j] * r_t
 * all in f32 with one rounding per stored element.
 *   x, dy [T, D] dtype   weight [D] dtype or NULL   dx [T, D] dtype (out; must not alias x or dy)
 *   dweight [D] dtype (out) or NULL; when given, workspace must hold
 *   fs2moe_rms_norm_backward_workspace_bytes(T, D) bytes (16-byte aligned); otherwise it is unused.
 */
int64_t fs2moe_rms_norm_backward_workspace_bytes(int32_t T, int32_t D);
int fs2moe_rms_norm_backward(const void* x, const void* weight, float eps, const void* dy,
                             int32_t T, int32_t D, int32_t dtype, void* dx, void* dweight,
                             void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FS2MOE_H_ */

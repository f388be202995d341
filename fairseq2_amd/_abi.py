"""ctypes binding of ``libfs2moe.so`` (declared in ``include/fs2moe.h``).

The library is the only compute path.  If it cannot be loaded the functions
here raise; nothing falls back to torch operators.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int32, c_int64, c_void_p

import torch
from torch import Tensor

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libfs2moe.so")

ABI_VERSION = 15

F32, BF16, FP8_E4M3 = 0, 1, 2
SCORE_SIGMOID, SCORE_SOFTMAX = 0, 1
ROUTER_OUT_IN = 0x100
ACT_MXFP8 = 0x100  # OR-ed into a whole-layer call's w_dtype next to e4m3 weights: W8A8  # OR-ed into score_fn: the router argument is (E, D)
W_IN_OUT, W_OUT_IN = 0, 1
MAX_EXPERTS, MAX_TOP_K = 512, 32

# name -> (restype, argtypes); mirrors include/fs2moe.h one to one
_PROTOTYPES = {
    "fs2moe_abi_version": (c_int32, []),
    "fs2moe_last_error": (c_char_p, []),
    "fs2moe_router_workspace_bytes": (c_int64, [c_int32, c_int32, c_int32, c_int32]),
    "fs2moe_router_takes_out_in": (c_int32, [c_int32, c_int32, c_int32, c_int32]),
    "fs2moe_router_topk": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p],
    ),
    "fs2moe_router_topk_norm": (
        c_int32,
        [c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
         c_void_p],
    ),
    "fs2moe_cpu_router_select": (
        c_int32, [c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]
    ),
    "fs2moe_dispatch_workspace_bytes": (c_int64, [c_int32, c_int32, c_int32]),
    "fs2moe_dispatch": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
         c_void_p],
    ),
    "fs2moe_grouped_swiglu": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p,
         c_void_p],
    ),
    "fs2moe_grouped_swiglu_rows": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_void_p, c_void_p,
         c_int32, c_void_p],
    ),
    "fs2moe_grouped_swiglu_fuses_gather": (c_int32, [c_int32, c_int32, c_int32, c_int32]),
    "fs2moe_grouped_swiglu_keeps": (c_int32, [c_int32, c_int32, c_int64, c_int32]),
    "fs2moe_dense_swiglu_keep": (c_int32, [c_void_p] * 4 + [c_int32] * 4 + [c_void_p] * 5),
    "fs2moe_grouped_gemm_sum_supported": (c_int32, [c_int32, c_int32, c_int64, c_int32]),
    "fs2moe_grouped_gemm_sum": (
        c_int32, [c_void_p] * 6 + [c_int32] * 3 + [c_int64, c_int32, c_void_p, c_void_p],
    ),
    "fs2moe_grouped_swiglu_keep": (
        c_int32,
        [c_void_p] * 7 + [c_int32] * 3 + [c_int64, c_int32] + [c_void_p] * 5,
    ),
    "fs2moe_dense_swiglu": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p,
         c_void_p, c_void_p],
    ),
    "fs2moe_combine": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_void_p, c_void_p],
    ),
    "fs2moe_combine_residual": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int32, c_int32, c_void_p, c_void_p],
    ),
    "fs2moe_forward_workspace_bytes": (
        c_int64, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32]
    ),
    "fs2moe_forward": (
        c_int32,
        [c_void_p] * 13 + [c_int32] * 12 + [c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "fs2moe_forward_norm_workspace_bytes": (
        c_int64, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32]
    ),
    "fs2moe_forward_static_capacity": (c_int64, []),
    "fs2moe_forward_static": (
        c_int32,
        [c_void_p] * 13 + [c_int32] * 12 + [c_void_p, c_void_p],
    ),
    "fs2moe_grouped_gemm": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_void_p, c_void_p],
    ),
    "fs2moe_grouped_wgrad_workspace_bytes": (c_int64, [c_int32, c_int32, c_int32, c_int64]),
    "fs2moe_grouped_wgrad": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int64,
         c_int32, c_void_p, c_void_p, c_int64, c_void_p],
    ),
    "fs2moe_swiglu_backward": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p, c_void_p,
         c_void_p],
    ),
    "fs2moe_pair_dot": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p,
         c_void_p],
    ),
    "fs2moe_router_backward": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_void_p, c_void_p],
    ),
    "fs2moe_rms_norm_backward_workspace_bytes": (c_int64, [c_int32, c_int32]),
    "fs2moe_rms_norm_backward": (
        c_int32,
        [c_void_p, c_void_p, c_float, c_void_p, c_int32, c_int32, c_int32, c_void_p, c_void_p,
         c_void_p, c_int64, c_void_p],
    ),
    "fs2moe_mx_quantize": (c_int32, [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p]),
    "fs2moe_grouped_swiglu_w8a8_supported": (c_int32, [c_int32, c_int32, c_int64]),
    "fs2moe_grouped_swiglu_w8a8": (
        c_int32, [c_void_p] * 11 + [c_int32] * 3 + [c_int64] * 2 + [c_void_p] * 4,
    ),
    "fs2moe_forward_norm": (
        c_int32,
        [c_void_p, c_void_p, c_float] + [c_void_p] * 12 + [c_int32] * 12
        + [c_void_p, c_int64, c_void_p, c_void_p],
    ),
}

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)

_lib: ctypes.CDLL | None = None


class Fs2MoeError(RuntimeError):
    """An entry point of libfs2moe returned an error code."""


def load() -> ctypes.CDLL:
    """Loads the shared library, once.  Raises if it is missing or of another ABI version."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m fairseq2_amd.build` "
            "(there is no fallback implementation)"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in _PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.fs2moe_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libfs2moe ABI version {got}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().fs2moe_last_error().decode("utf-8", "replace")
        raise Fs2MoeError(f"{what} failed ({rc}): {msg}")


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return F32
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float8_e4m3fn:
        return FP8_E4M3
    raise TypeError(f"libfs2moe has no kernels for {dtype} (supported: float32, bfloat16)")


def _ptr(t: Tensor | None) -> int | None:
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("libfs2moe takes device tensors only")
    if not t.is_contiguous():
        raise ValueError("libfs2moe takes contiguous tensors only")
    return t.data_ptr()


def _same(name: str, t: Tensor, shape: tuple, dtype: torch.dtype, dev: torch.device) -> None:
    if tuple(t.shape) != tuple(shape) or t.dtype != dtype or t.device != dev or not t.is_contiguous():
        raise ValueError(
            f"{name} must be a contiguous {tuple(shape)} {dtype} tensor on {dev}, got {tuple(t.shape)} "
            f"{t.dtype} on {t.device}")


def _check_groups(counts: Tensor, offsets: Tensor, num_experts: int, dev: torch.device) -> None:
    _same("counts", counts, (num_experts,), torch.int32, dev)
    _same("offsets", offsets, (num_experts + 1,), torch.int32, dev)


def _check_selection(topk_idx: Tensor, topk_w: Tensor | None, dev: torch.device) -> tuple[int, int]:
    if topk_idx.dim() != 2:
        raise ValueError("topk_idx must be (T, K)")
    _same("topk_idx", topk_idx, topk_idx.shape, torch.int32, dev)
    if topk_w is not None:
        _same("topk_w", topk_w, topk_idx.shape, torch.float32, dev)
    return topk_idx.shape[0], topk_idx.shape[1]


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def max_rows(num_tokens: int, top_k: int, num_experts: int, tile_m: int) -> int:
    """Upper bound on the tile-padded number of rows (FS2MOE_MAX_ROWS)."""
    return num_tokens * top_k + num_experts * (tile_m - 1)


# ------------------------------------------------------------------------------------------------
def router_topk(
    x: Tensor,
    router: Tensor,
    bias: Tensor | None,
    top_k: int,
    score_fn: int = SCORE_SIGMOID,
    renormalize: bool = False,
    want_logits: bool = False,
    split: bool = True,
    router_t: Tensor | None = None,
) -> tuple[Tensor, Tensor, Tensor | None]:
    """``x`` (T, D), ``router`` (D, E) -> ``topk_idx`` int32 (T, K), ``topk_w`` f32 (T, K), logits.
    ``router_t``: optionally the same matrix expert-major, (E, D), used where the library reads it.

    ``split=False`` withholds the scratch buffer that lets several blocks share a token tile when
    there are few tokens (see ``fs2moe_router_topk``)."""
    lib = load()
    t, d = x.shape
    e = router.shape[1]
    if router.shape[0] != d or router.dtype != x.dtype:
        raise ValueError("router must be (D, E) in the dtype of x")
    idx = torch.empty((t, top_k), dtype=torch.int32, device=x.device)
    w = torch.empty((t, top_k), dtype=torch.float32, device=x.device)
    logits = torch.empty((t, e), dtype=torch.float32, device=x.device) if want_logits else None
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != e):
        raise ValueError("router bias must be f32 of E elements")
    mat, score_fn = router_operand(lib, x, router, router_t, score_fn)
    rc = lib.fs2moe_router_topk(
        _ptr(x), _ptr(mat), _ptr(bias), t, d, e, top_k, dtype_code(x.dtype), score_fn,
        int(renormalize), _ptr(idx), _ptr(w), _ptr(logits), *_router_workspace(lib, x, e, split), _stream(),
    )
    _check(rc, "fs2moe_router_topk")
    return idx, w, logits


def cpu_router_select(logits: Tensor, top_k: int, score_fn: int = SCORE_SIGMOID,
                      renormalize: bool = False) -> tuple[Tensor, Tensor]:
    """Host mirror of the device's selection (``fs2moe_cpu_router_select``): from f32 logits on the
    CPU, the experts (bit for bit what the device selects from the same logits) and their weights."""
    lib = load()
    logits = logits.detach().to("cpu", torch.float32).contiguous()
    t, e = logits.shape
    idx = torch.empty((t, top_k), dtype=torch.int32)
    w = torch.empty((t, top_k), dtype=torch.float32)
    rc = lib.fs2moe_cpu_router_select(logits.data_ptr(), t, e, top_k, score_fn, int(renormalize),
                                      idx.data_ptr(), w.data_ptr())
    _check(rc, "fs2moe_cpu_router_select")
    return idx, w


def router_expert_major(router: Tensor, holder=None) -> Tensor | None:
    """The bf16 router matrix expert-major, ``(E, D)``: a derived copy that the router kernel reads
    without transposing (``ROUTER_OUT_IN``).  It is kept on ``holder`` (the module that owns the
    parameter; by default the tensor object itself, which for a parameter lives as long as its
    module) and made again whenever the parameter has changed: in-place updates bump its version
    counter, a move or a new tensor changes its address.  None for other dtypes."""
    if router.dtype != torch.bfloat16 or not router.is_cuda:
        return None
    holder = router if holder is None else holder
    try:
        version = router._version
    except RuntimeError:
        # a tensor made under torch.inference_mode() has no version counter: nothing would say when
        # it has been written to, so no copy is kept and the router reads the matrix as it is
        return None
    key = (version, router.data_ptr(), tuple(router.shape))
    hit = getattr(holder, "_fs2moe_router_t", None)
    if hit is None or hit[0] != key:
        with torch.no_grad():
            hit = (key, router.detach().t().contiguous())
        try:
            object.__setattr__(holder, "_fs2moe_router_t", hit)
        except (AttributeError, TypeError):
            pass  # nowhere to keep it: made again on the next call
    return hit[1]


def router_operand(lib, x: Tensor, router: Tensor, router_t: Tensor | None, score_fn: int) -> tuple[Tensor, int]:
    """The router matrix to pass and the score_fn to pass with it: the expert-major copy ``router_t``
    ``(E, D)`` with ``ROUTER_OUT_IN`` set where the library reads that form at this size, else
    ``router`` ``(D, E)``."""
    if router_t is None:
        return router, score_fn
    d, e = router.shape
    if router_t.shape != (e, d) or router_t.dtype != router.dtype or not router_t.is_contiguous():
        raise ValueError("router_t must be the contiguous (E, D) transpose of router")
    if lib.fs2moe_router_takes_out_in(x.shape[0], d, e, dtype_code(x.dtype)):
        return router_t, score_fn | ROUTER_OUT_IN
    return router, score_fn


def _router_workspace(lib, x: Tensor, num_experts: int, split: bool) -> tuple[int | None, int]:
    """(pointer, bytes) of a fresh scratch buffer for the router, or (None, 0)."""
    need = lib.fs2moe_router_workspace_bytes(x.shape[0], x.shape[1], num_experts, dtype_code(x.dtype)) if split else 0
    if need <= 0:
        return None, 0
    ws = torch.empty(need, dtype=torch.uint8, device=x.device)  # stream-ordered: safe to drop after the call
    return _ptr(ws), need


def _check_norm_weight(weight: Tensor | None, x: Tensor) -> None:
    if weight is not None and (weight.dtype != x.dtype or weight.numel() != x.shape[1] or not weight.is_contiguous()):
        raise ValueError("the norm weight must be a contiguous (D,) tensor in the dtype of x")


def router_topk_norm(
    x: Tensor,
    norm_weight: Tensor | None,
    norm_eps: float,
    router: Tensor,
    bias: Tensor | None,
    top_k: int,
    score_fn: int = SCORE_SIGMOID,
    renormalize: bool = False,
    want_logits: bool = False,
    split: bool = True,
    router_t: Tensor | None = None,
) -> tuple[Tensor, Tensor, Tensor, Tensor | None]:
    """RMS-normalises the rows of ``x`` and routes the result: ``xn``, then as :func:`router_topk`."""
    lib = load()
    t, d = x.shape
    e = router.shape[1]
    if router.shape[0] != d or router.dtype != x.dtype:
        raise ValueError("router must be (D, E) in the dtype of x")
    _check_norm_weight(norm_weight, x)
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != e):
        raise ValueError("router bias must be f32 of E elements")
    xn = torch.empty_like(x)
    idx = torch.empty((t, top_k), dtype=torch.int32, device=x.device)
    w = torch.empty((t, top_k), dtype=torch.float32, device=x.device)
    logits = torch.empty((t, e), dtype=torch.float32, device=x.device) if want_logits else None
    mat, score_fn = router_operand(lib, x, router, router_t, score_fn)
    rc = lib.fs2moe_router_topk_norm(
        _ptr(x), _ptr(norm_weight), float(norm_eps), _ptr(xn), _ptr(mat), _ptr(bias), t, d, e,
        top_k, dtype_code(x.dtype), score_fn, int(renormalize), _ptr(idx), _ptr(w), _ptr(logits),
        *_router_workspace(lib, x, e, split), _stream(),
    )
    _check(rc, "fs2moe_router_topk_norm")
    return xn, idx, w, logits


class Dispatched:
    """Outputs of :func:`dispatch`."""

    __slots__ = ("counts", "offsets", "perm", "inv_perm", "xe", "max_rows", "tile_m")

    def __init__(self, counts, offsets, perm, inv_perm, xe, max_rows_, tile_m):
        self.counts, self.offsets, self.perm, self.inv_perm = counts, offsets, perm, inv_perm
        self.xe, self.max_rows, self.tile_m = xe, max_rows_, tile_m


def dispatch(
    topk_idx: Tensor,
    topk_w: Tensor | None,
    x: Tensor,
    num_experts: int,
    tile_m: int,
    scale_input: bool,
    gather: bool = True,
) -> Dispatched:
    lib = load()
    dev = x.device
    t, k = _check_selection(topk_idx, topk_w, dev)
    if x.dim() != 2 or x.shape[0] != t:
        raise ValueError("x must be (T, D) with one row per row of topk_idx")
    if scale_input and topk_w is None:
        raise ValueError("scaling the rows needs topk_w")
    d = x.shape[1]
    rows = max_rows(t, k, num_experts, tile_m)
    counts = torch.empty(num_experts, dtype=torch.int32, device=dev)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(rows, dtype=torch.int32, device=dev)
    inv_perm = torch.empty((t, k), dtype=torch.int32, device=dev)
    xe = torch.empty((rows, d), dtype=x.dtype, device=dev) if gather else None
    ws_bytes = lib.fs2moe_dispatch_workspace_bytes(t, k, num_experts)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = lib.fs2moe_dispatch(
        _ptr(topk_idx), _ptr(topk_w), _ptr(x), t, k, num_experts, d, tile_m, dtype_code(x.dtype),
        int(scale_input), rows, _ptr(counts), _ptr(offsets), _ptr(perm), _ptr(inv_perm), _ptr(xe),
        _ptr(ws), ws_bytes, _stream(),
    )
    _check(rc, "fs2moe_dispatch")
    return Dispatched(counts, offsets, perm, inv_perm, xe, rows, tile_m)


def pack_fp8_weights(q: Tensor, num_experts: int) -> Tensor:
    """Re-tiles e4m3 codes from the reference orientation ``(E*in, out)`` to the kernel's
    ``(E, out/16, in/64, 16, 64)``: 1 KB tiles of 16 output channels x 64 input features."""
    if q.dtype != torch.float8_e4m3fn or q.dim() != 2 or q.shape[0] % num_experts:
        raise ValueError("expected float8_e4m3fn codes of shape (E*in, out)")
    k, n = q.shape[0] // num_experts, q.shape[1]
    if k % 64 or n % 16:
        raise ValueError("fp8 weights need in-features % 64 == 0 and out-features % 16 == 0")
    b = q.view(torch.uint8).view(num_experts, k // 64, 64, n // 16, 16)
    return b.permute(0, 3, 1, 4, 2).contiguous().view(torch.float8_e4m3fn)


def unpack_fp8_weights(tiled: Tensor, num_experts: int) -> Tensor:
    """Inverse of :func:`pack_fp8_weights`: the kernel's ``(E, out/16, in/64, 16, 64)`` tiles back to
    the reference orientation ``(E*in, out)``."""
    if tiled.dtype != torch.float8_e4m3fn or tiled.dim() != 5 or tiled.shape[0] != num_experts:
        raise ValueError("expected float8_e4m3fn tiles of shape (E, out/16, in/64, 16, 64)")
    e, n16, k64 = tiled.shape[:3]
    b = tiled.view(torch.uint8).permute(0, 2, 4, 1, 3).contiguous()  # (E, in/64, 64, out/16, 16)
    return b.view(e * k64 * 64, n16 * 16).view(torch.float8_e4m3fn)


def grouped_swiglu(
    xe: Tensor,
    counts: Tensor,
    offsets: Tensor,
    w_gate: Tensor,
    w_up: Tensor,
    w_down: Tensor,
    num_experts: int,
    scales: tuple[Tensor, Tensor, Tensor] | None = None,
    row_map: Tensor | None = None,
    rows_per_expert: int = 0,
) -> tuple[Tensor, Tensor]:
    """Returns ``(ye, h)`` for the rows of ``xe`` (rows, D).

    ``rows_per_expert``: an upper bound on the rows of any one expert when the caller knows one
    (the number of tokens is one), else 0; with 1..16 and bf16 weights the products run as streams
    over the weights instead of as GEMM tiles (``fs2moe_grouped_swiglu_rows``).

    With ``row_map`` (int32, one entry per row: ``Dispatched.perm``) ``xe`` is the token matrix
    ``(T, D)`` and row ``r`` of the experts' input is ``xe[row_map[r]]``: the gather is fused into
    the first GEMM (see :func:`fuses_gather`).

    Without ``scales`` the weights are in the activation dtype and the reference layout
    (``(E*D, F)``, ``(E*D, F)``, ``(E*F, D)``).  With ``scales`` they are e4m3 codes tiled by
    :func:`pack_fp8_weights`, ``(E, F/16, D/64, 16, 64)`` twice and ``(E, D/16, F/64, 16, 64)``,
    with f32 scales ``(E, F)``, ``(E, F)``, ``(E, D)``.
    """
    lib = load()
    rows, d = xe.shape
    if row_map is not None:
        if row_map.dtype != torch.int32 or row_map.dim() != 1:
            raise ValueError("row_map must be a 1-d int32 tensor")
        rows = row_map.shape[0]
    _check_groups(counts, offsets, num_experts, xe.device)
    if scales is None:
        f = w_down.shape[0] // num_experts
        if w_gate.shape != (num_experts * d, f) or w_up.shape != w_gate.shape:
            raise ValueError("gate/up weights must be (E*D, F)")
        if w_down.shape != (num_experts * f, d):
            raise ValueError("down weights must be (E*F, D)")
        for name, w in (("w_gate", w_gate), ("w_up", w_up), ("w_down", w_down)):
            _same(name, w, w.shape, xe.dtype, xe.device)
    else:
        f = w_gate.shape[1] * 16
        if w_gate.shape != (num_experts, f // 16, d // 64, 16, 64) or w_up.shape != w_gate.shape:
            raise ValueError("fp8 gate/up codes must be tiled (E, F/16, D/64, 16, 64)")
        if w_down.shape != (num_experts, d // 16, f // 64, 16, 64):
            raise ValueError("fp8 down codes must be tiled (E, D/16, F/64, 16, 64)")
        want = [(num_experts, f), (num_experts, f), (num_experts, d)]
        if [tuple(s.shape) for s in scales] != want or any(s.dtype != torch.float32 for s in scales):
            raise ValueError("fp8 scales must be f32 (E, F), (E, F), (E, D)")
        for w in (w_gate, w_up, w_down):
            if w.dtype not in (torch.float8_e4m3fn, torch.uint8) or w.device != xe.device:
                raise ValueError("fp8 codes must be float8_e4m3fn (or their uint8 bytes) on the device of xe")
    h = torch.empty((rows, f), dtype=xe.dtype, device=xe.device)
    ye = torch.empty((rows, d), dtype=xe.dtype, device=xe.device)
    sg, su, sd = scales if scales is not None else (None, None, None)
    rc = lib.fs2moe_grouped_swiglu_rows(
        _ptr(xe), _ptr(row_map), _ptr(counts), _ptr(offsets), _ptr(w_gate), _ptr(w_up),
        _ptr(w_down), _ptr(sg), _ptr(su), _ptr(sd), num_experts, d, f, rows, dtype_code(xe.dtype),
        dtype_code(w_gate.dtype), _ptr(h), _ptr(ye), int(rows_per_expert), _stream(),
    )
    _check(rc, "fs2moe_grouped_swiglu_rows")
    return ye, h


def keeps_products(model_dim: int, inner_dim: int, rows: int, act_dtype: torch.dtype) -> bool:
    """Whether :func:`grouped_swiglu_keep` exists for these sizes and this type."""
    return bool(load().fs2moe_grouped_swiglu_keeps(model_dim, inner_dim, rows, dtype_code(act_dtype)))


def mx_quantize(x: Tensor) -> tuple[Tensor, Tensor]:
    """bf16 rows ``(rows, D)`` -> e4m3 codes ``(rows, D)`` (as uint8) and one exponent byte per row
    and 32 features in the library's k-group-major layout ``(D / 128, rows, 4)``
    (``fs2moe_mx_quantize``; :func:`mx_scales_row_major` gives ``(rows, D / 32)``)."""
    lib = load()
    if x.dim() != 2 or x.dtype != torch.bfloat16 or x.shape[1] % 128:
        raise ValueError("mx_quantize takes (rows, D) bf16 with D a multiple of 128")
    rows, d = x.shape
    codes = torch.empty((rows, d), dtype=torch.uint8, device=x.device)
    scales = torch.empty((d // 128, rows, 4), dtype=torch.uint8, device=x.device)
    rc = lib.fs2moe_mx_quantize(_ptr(x), rows, d, _ptr(codes), _ptr(scales), _stream())
    _check(rc, "fs2moe_mx_quantize")
    return codes, scales


def mx_scales_row_major(scales: Tensor) -> Tensor:
    """Scale bytes ``(K / 128, rows, 4)`` as the library stores them -> ``(rows, K / 32)``."""
    g, rows, four = scales.shape
    return scales.permute(1, 0, 2).reshape(rows, g * four).contiguous()


def mx_scales_k_major(scales: Tensor) -> Tensor:
    """Scale bytes ``(rows, K / 32)`` -> the library's ``(K / 128, rows, 4)``."""
    rows, nb = scales.shape
    return scales.reshape(rows, nb // 4, 4).permute(1, 0, 2).contiguous()


def w8a8_supported(model_dim: int, inner_dim: int, rows: int) -> bool:
    return bool(load().fs2moe_grouped_swiglu_w8a8_supported(model_dim, inner_dim, rows))


def grouped_swiglu_w8a8(
    xq: Tensor,
    xs: Tensor,
    counts: Tensor,
    offsets: Tensor,
    w_gate: Tensor,
    w_up: Tensor,
    w_down: Tensor,
    scales: tuple[Tensor, Tensor, Tensor],
    num_experts: int,
    row_map: Tensor | None = None,
) -> tuple[Tensor, Tensor, Tensor]:
    """The grouped SwiGLU network on the fp8 matrix pipe (``fs2moe_grouped_swiglu_w8a8``): block-scaled
    e4m3 rows (:func:`mx_quantize`) against tiled e4m3 weights with channel scales.  Returns
    ``(ye, hq, hs)``: bf16 output rows and the quantised gated product (scales k-group major)."""
    lib = load()
    rows, d = xq.shape
    x_rows = rows
    dev = xq.device
    _same("xq", xq, (rows, d), torch.uint8, dev)
    _same("xs", xs, (d // 128, rows, 4), torch.uint8, dev)
    if row_map is not None:
        if row_map.dtype != torch.int32 or row_map.dim() != 1:
            raise ValueError("row_map must be a 1-d int32 tensor")
        rows = row_map.shape[0]
    _check_groups(counts, offsets, num_experts, dev)
    f = w_gate.shape[1] * 16
    if w_gate.shape != (num_experts, f // 16, d // 64, 16, 64) or w_up.shape != w_gate.shape:
        raise ValueError("fp8 gate/up codes must be tiled (E, F/16, D/64, 16, 64)")
    if w_down.shape != (num_experts, d // 16, f // 64, 16, 64):
        raise ValueError("fp8 down codes must be tiled (E, D/16, F/64, 16, 64)")
    want = [(num_experts, f), (num_experts, f), (num_experts, d)]
    if [tuple(s.shape) for s in scales] != want or any(s.dtype != torch.float32 for s in scales):
        raise ValueError("fp8 scales must be f32 (E, F), (E, F), (E, D)")
    hq = torch.empty((rows, f), dtype=torch.uint8, device=dev)
    hs = torch.empty((f // 128, rows, 4), dtype=torch.uint8, device=dev)
    ye = torch.empty((rows, d), dtype=torch.bfloat16, device=dev)
    rc = lib.fs2moe_grouped_swiglu_w8a8(
        _ptr(xq), _ptr(xs), _ptr(row_map), _ptr(counts), _ptr(offsets), _ptr(w_gate), _ptr(w_up),
        _ptr(w_down), _ptr(scales[0]), _ptr(scales[1]), _ptr(scales[2]), num_experts, d, f, x_rows,
        rows, _ptr(hq), _ptr(hs), _ptr(ye), _stream(),
    )
    _check(rc, "fs2moe_grouped_swiglu_w8a8")
    return ye, hq, hs


def grouped_swiglu_keep(
    xe: Tensor,
    counts: Tensor,
    offsets: Tensor,
    w_gate: Tensor,
    w_up: Tensor,
    w_down: Tensor,
    num_experts: int,
    row_map: Tensor | None = None,
) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """:func:`grouped_swiglu` that also returns the gate and the up product: ``(ye, h, g, u)``."""
    lib = load()
    rows, d = xe.shape
    if row_map is not None:
        if row_map.dtype != torch.int32 or row_map.dim() != 1:
            raise ValueError("row_map must be a 1-d int32 tensor")
        rows = row_map.shape[0]
    _check_groups(counts, offsets, num_experts, xe.device)
    f = w_down.shape[0] // num_experts
    if w_gate.shape != (num_experts * d, f) or w_up.shape != w_gate.shape:
        raise ValueError("gate/up weights must be (E*D, F)")
    if w_down.shape != (num_experts * f, d):
        raise ValueError("down weights must be (E*F, D)")
    for name, w in (("w_gate", w_gate), ("w_up", w_up), ("w_down", w_down)):
        _same(name, w, w.shape, xe.dtype, xe.device)
    g, u, h = (torch.empty((rows, f), dtype=xe.dtype, device=xe.device) for _ in range(3))
    ye = torch.empty((rows, d), dtype=xe.dtype, device=xe.device)
    rc = lib.fs2moe_grouped_swiglu_keep(
        _ptr(xe), _ptr(row_map), _ptr(counts), _ptr(offsets), _ptr(w_gate), _ptr(w_up),
        _ptr(w_down), num_experts, d, f, rows, dtype_code(xe.dtype), _ptr(g), _ptr(u), _ptr(h),
        _ptr(ye), _stream(),
    )
    _check(rc, "fs2moe_grouped_swiglu_keep")
    return ye, h, g, u


def fuses_gather(model_dim: int, inner_dim: int, act_dtype: torch.dtype, w_dtype: torch.dtype) -> bool:
    """Whether :func:`grouped_swiglu` takes a ``row_map`` for these sizes and types."""
    return bool(
        load().fs2moe_grouped_swiglu_fuses_gather(
            model_dim, inner_dim, dtype_code(act_dtype), dtype_code(w_dtype)
        )
    )


def dense_swiglu(x: Tensor, w_gate: Tensor, w_up: Tensor, w_down: Tensor) -> Tensor:
    """``(SiLU(x Wg^T) * (x Wu^T)) Wd^T`` with nn.Linear-oriented weights."""
    lib = load()
    t, d = x.shape
    f = w_gate.shape[0]
    if w_gate.shape != (f, d) or w_up.shape != (f, d) or w_down.shape != (d, f):
        raise ValueError("shared-expert weights must be (F, D), (F, D), (D, F)")
    for name, w in (("w_gate", w_gate), ("w_up", w_up), ("w_down", w_down)):
        _same(name, w, w.shape, x.dtype, x.device)
    h = torch.empty((t, f), dtype=x.dtype, device=x.device)
    y = torch.empty((t, d), dtype=x.dtype, device=x.device)
    rc = lib.fs2moe_dense_swiglu(
        _ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(w_down), t, d, f, dtype_code(x.dtype), _ptr(h),
        _ptr(y), _stream(),
    )
    _check(rc, "fs2moe_dense_swiglu")
    return y


def dense_swiglu_keep(x: Tensor, w_gate: Tensor, w_up: Tensor, w_down: Tensor) -> tuple[Tensor, Tensor, Tensor]:
    """:func:`dense_swiglu` that also returns the gate and the up product: ``(y, g, u)``."""
    lib = load()
    t, d = x.shape
    f = w_gate.shape[0]
    if w_gate.shape != (f, d) or w_up.shape != (f, d) or w_down.shape != (d, f):
        raise ValueError("shared-expert weights must be (F, D), (F, D), (D, F)")
    for name, w in (("w_gate", w_gate), ("w_up", w_up), ("w_down", w_down)):
        _same(name, w, w.shape, x.dtype, x.device)
    g, u, h = (torch.empty((t, f), dtype=x.dtype, device=x.device) for _ in range(3))
    y = torch.empty((t, d), dtype=x.dtype, device=x.device)
    rc = lib.fs2moe_dense_swiglu_keep(
        _ptr(x), _ptr(w_gate), _ptr(w_up), _ptr(w_down), t, d, f, dtype_code(x.dtype), _ptr(g),
        _ptr(u), _ptr(h), _ptr(y), _stream(),
    )
    _check(rc, "fs2moe_dense_swiglu_keep")
    return y, g, u


def combine(
    ye: Tensor,
    inv_perm: Tensor,
    topk_idx: Tensor,
    topk_w: Tensor | None,
    base: Tensor | None,
    weight_output: bool,
    out: Tensor | None = None,
    residual: Tensor | None = None,
) -> Tensor:
    """``out[t] = (residual[t] +) base[t] + sum of the token's expert rows``; ``out`` may be
    ``base`` or ``residual`` itself."""
    lib = load()
    t, k = _check_selection(topk_idx, topk_w, ye.device)
    _same("inv_perm", inv_perm, (t, k), torch.int32, ye.device)
    if weight_output and topk_w is None:
        raise ValueError("weighting the output needs topk_w")
    d = ye.shape[1]
    if base is not None:
        _same("base", base, (t, d), ye.dtype, ye.device)
    if out is None:
        out = torch.empty((t, d), dtype=ye.dtype, device=ye.device)
    else:
        _same("out", out, (t, d), ye.dtype, ye.device)
    if residual is None:
        rc = lib.fs2moe_combine(
            _ptr(ye), _ptr(inv_perm), _ptr(topk_idx), _ptr(topk_w), _ptr(base), t, k, d,
            dtype_code(ye.dtype), int(weight_output), _ptr(out), _stream(),
        )
        _check(rc, "fs2moe_combine")
    else:
        _same("residual", residual, (t, d), ye.dtype, ye.device)
        rc = lib.fs2moe_combine_residual(
            _ptr(ye), _ptr(inv_perm), _ptr(topk_idx), _ptr(topk_w), _ptr(base), _ptr(residual), t, k,
            d, dtype_code(ye.dtype), int(weight_output), _ptr(out), _stream(),
        )
        _check(rc, "fs2moe_combine_residual")
    return out


# ---------------------------------------------------------------------------------- backward pass
def grouped_gemm(
    a: Tensor,
    b: Tensor,
    layout: int,
    counts: Tensor | None = None,
    offsets: Tensor | None = None,
    num_experts: int = 1,
    row_map: Tensor | None = None,
    rows: int | None = None,
) -> Tensor:
    """``c[r] = a[r] @ B_e`` for the rows ``r`` of every expert ``e`` (``fs2moe_grouped_gemm``).

    ``b`` holds one ``(K, N)`` matrix per expert, ``layout`` ``W_IN_OUT``: ``(E*K, N)``, or
    ``W_OUT_IN``: ``(E*N, K)`` -- i.e. the second form multiplies by the transpose of what the
    forward pass multiplied by in the first.  Without ``counts`` all rows belong to one matrix.  With
    ``row_map``, row ``r`` of the product is computed from ``a[row_map[r]]`` and ``rows`` is the
    number of rows of the result."""
    lib = load()
    e = num_experts
    k = a.shape[1]
    if b.dim() != 2 or b.dtype != a.dtype or b.device != a.device or not b.is_contiguous() or b.numel() % (e * k):
        raise ValueError("b must hold one (K, N) or (N, K) matrix per expert in the dtype of a")
    n = b.numel() // (e * k)
    _same("b", b, (e * k, n) if layout == W_IN_OUT else (e * n, k), a.dtype, a.device)
    if (counts is None) != (offsets is None):
        raise ValueError("counts and offsets come together")
    if counts is not None:
        _same("counts", counts, (e,), torch.int32, a.device)
        _same("offsets", offsets, (e + 1,), torch.int32, a.device)
    elif e != 1:
        raise ValueError("a dense product has one matrix")
    if row_map is not None:
        if rows is None:
            rows = row_map.shape[0]
        _same("row_map", row_map, (row_map.shape[0],), torch.int32, a.device)
        if row_map.shape[0] < rows:
            raise ValueError("row_map is shorter than the result")
    else:
        rows = a.shape[0]
    c = torch.empty((rows, n), dtype=a.dtype, device=a.device)
    rc = lib.fs2moe_grouped_gemm(
        _ptr(a), _ptr(row_map), _ptr(counts), _ptr(offsets), _ptr(b), layout, e, k, n, rows,
        dtype_code(a.dtype), _ptr(c), _stream(),
    )
    _check(rc, "fs2moe_grouped_gemm")
    return c


def grouped_gemm_sum_supported(k: int, n: int, rows: int, dtype: torch.dtype) -> bool:
    """Whether :func:`grouped_gemm_sum` exists for these sizes and this type."""
    return bool(load().fs2moe_grouped_gemm_sum_supported(k, n, rows, dtype_code(dtype)))


def grouped_gemm_sum(
    a1: Tensor, b1: Tensor, a2: Tensor, b2: Tensor,
    counts: Tensor | None = None, offsets: Tensor | None = None, num_experts: int = 1,
) -> Tensor:
    """``c[r] = a1[r] @ B1_e^T + a2[r] @ B2_e^T`` with ``(E*N, K)`` weights, one rounding
    (``fs2moe_grouped_gemm_sum``)."""
    lib = load()
    e = num_experts
    rows, k = a1.shape
    n = b1.shape[0] // e
    _same("a2", a2, (rows, k), a1.dtype, a1.device)
    _same("b1", b1, (e * n, k), a1.dtype, a1.device)
    _same("b2", b2, (e * n, k), a1.dtype, a1.device)
    if not a1.is_contiguous():
        raise ValueError("a1 must be contiguous")
    if (counts is None) != (offsets is None):
        raise ValueError("counts and offsets come together")
    if counts is not None:
        _same("counts", counts, (e,), torch.int32, a1.device)
        _same("offsets", offsets, (e + 1,), torch.int32, a1.device)
    elif e != 1:
        raise ValueError("a dense product has one matrix")
    c = torch.empty((rows, n), dtype=a1.dtype, device=a1.device)
    rc = lib.fs2moe_grouped_gemm_sum(
        _ptr(a1), _ptr(b1), _ptr(a2), _ptr(b2), _ptr(counts), _ptr(offsets), e, k, n, rows,
        dtype_code(a1.dtype), _ptr(c), _stream(),
    )
    _check(rc, "fs2moe_grouped_gemm_sum")
    return c


def grouped_wgrad(
    a: Tensor,
    b: Tensor,
    counts: Tensor | None = None,
    offsets: Tensor | None = None,
    num_experts: int = 1,
    a_row_map: Tensor | None = None,
) -> Tensor:
    """``dw_e = A_e^T @ B_e`` over the rows of each expert: ``(E*M, N)`` (``fs2moe_grouped_wgrad``).
    ``b`` has one row per row of the experts' buffer; ``a`` as well, or, with ``a_row_map``, row
    ``r`` of ``A`` is ``a[a_row_map[r]]``."""
    lib = load()
    e = num_experts
    rows, n = b.shape
    m = a.shape[1]
    if a.dtype != b.dtype or a.device != b.device or not a.is_contiguous() or not b.is_contiguous():
        raise ValueError("a and b must be contiguous tensors of one dtype on one device")
    if (counts is None) != (offsets is None):
        raise ValueError("counts and offsets come together")
    if counts is not None:
        _same("counts", counts, (e,), torch.int32, a.device)
        _same("offsets", offsets, (e + 1,), torch.int32, a.device)
    elif e != 1:
        raise ValueError("a dense product has one matrix")
    if a_row_map is not None:
        _same("a_row_map", a_row_map, (a_row_map.shape[0],), torch.int32, a.device)
        if a_row_map.shape[0] < rows:
            raise ValueError("a_row_map is shorter than b")
    elif a.shape[0] != rows:
        raise ValueError("a and b must have the same number of rows")
    dw = torch.empty((e * m, n), dtype=a.dtype, device=a.device)
    ws_bytes = lib.fs2moe_grouped_wgrad_workspace_bytes(int(counts is not None), m, n, rows)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes > 0 else None
    rc = lib.fs2moe_grouped_wgrad(
        _ptr(a), _ptr(a_row_map), _ptr(b), _ptr(counts), _ptr(offsets), e, m, n, rows,
        dtype_code(a.dtype), _ptr(dw), _ptr(ws), max(ws_bytes, 0), _stream(),
    )
    _check(rc, "fs2moe_grouped_wgrad")
    return dw


def swiglu_backward(g: Tensor, u: Tensor, dh: Tensor, in_place: bool = True) -> tuple[Tensor, Tensor, Tensor]:
    """``(h, dg, du)`` of ``h = SiLU(g) * u`` given ``dh``; ``dg`` and ``du`` overwrite ``g`` and
    ``u`` unless ``in_place`` is false."""
    lib = load()
    _same("u", u, g.shape, g.dtype, g.device)
    _same("dh", dh, g.shape, g.dtype, g.device)
    if not g.is_contiguous():
        raise ValueError("g must be contiguous")
    h = torch.empty_like(g)
    dg, du = (g, u) if in_place else (torch.empty_like(g), torch.empty_like(u))
    rc = lib.fs2moe_swiglu_backward(
        _ptr(g), _ptr(u), _ptr(dh), g.shape[0], g.shape[1], dtype_code(g.dtype), _ptr(h), _ptr(dg),
        _ptr(du), _stream(),
    )
    _check(rc, "fs2moe_swiglu_backward")
    return h, dg, du


def pair_dot(a: Tensor, a_rows: Tensor, b: Tensor, a2: Tensor | None = None) -> Tensor:
    """``out[t, k] = <a[a_rows[t, k]] (+ a2[a_rows[t, k]]), b[t]>`` in f32 (``fs2moe_pair_dot``)."""
    lib = load()
    t, k = a_rows.shape
    d = b.shape[1]
    _same("a_rows", a_rows, (t, k), torch.int32, b.device)
    _same("b", b, (t, d), a.dtype, a.device)
    _same("a", a, (a.shape[0], d), a.dtype, a.device)
    if a2 is not None:
        _same("a2", a2, a.shape, a.dtype, a.device)
    out = torch.empty((t, k), dtype=torch.float32, device=b.device)
    rc = lib.fs2moe_pair_dot(_ptr(a), _ptr(a2), _ptr(a_rows), _ptr(b), t, k, d, dtype_code(a.dtype),
                             _ptr(out), _stream())
    _check(rc, "fs2moe_pair_dot")
    return out


def router_backward(logits: Tensor, topk_idx: Tensor, topk_w: Tensor, d_w: Tensor, score_fn: int,
                    renormalize: bool, dtype: torch.dtype) -> Tensor:
    """Gradient of the combine weights -> gradient of the logits ``(T, E)`` in ``dtype``."""
    lib = load()
    t, e = logits.shape
    k = topk_idx.shape[1]
    dev = logits.device
    _same("logits", logits, (t, e), torch.float32, dev)
    _same("topk_idx", topk_idx, (t, k), torch.int32, dev)
    _same("topk_w", topk_w, (t, k), torch.float32, dev)
    _same("d_w", d_w, (t, k), torch.float32, dev)
    dl = torch.empty((t, e), dtype=dtype, device=dev)
    rc = lib.fs2moe_router_backward(_ptr(logits), _ptr(topk_idx), _ptr(topk_w), _ptr(d_w), t, e, k,
                                    score_fn, int(renormalize), dtype_code(dtype), _ptr(dl), _stream())
    _check(rc, "fs2moe_router_backward")
    return dl


def rms_norm_backward(x: Tensor, weight: Tensor | None, eps: float, dy: Tensor,
                      want_weight_grad: bool = True) -> tuple[Tensor, Tensor | None]:
    """``(dx, dweight)`` of ``y = rms_norm(x) * weight`` given ``dy`` (``fs2moe_rms_norm_backward``);
    ``dweight`` is None without a weight or when not asked for."""
    lib = load()
    t, d = x.shape
    _same("x", x, (t, d), x.dtype, x.device)
    _same("dy", dy, (t, d), x.dtype, x.device)
    if weight is not None:
        _same("weight", weight, (d,), x.dtype, x.device)
    dx = torch.empty_like(x)
    dw = ws = None
    ws_bytes = 0
    if weight is not None and want_weight_grad:
        dw = torch.empty_like(weight)
        ws_bytes = lib.fs2moe_rms_norm_backward_workspace_bytes(t, d)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    rc = lib.fs2moe_rms_norm_backward(
        _ptr(x), _ptr(weight), float(eps), _ptr(dy), t, d, dtype_code(x.dtype), _ptr(dx), _ptr(dw),
        _ptr(ws), ws_bytes, _stream(),
    )
    _check(rc, "fs2moe_rms_norm_backward")
    return dx, dw


def check_layer_arguments(x, router, router_bias, w_gate, w_up, w_down, num_experts, f, scales, shared) -> None:
    """Shapes, dtypes, devices and contiguity of everything ``fs2moe_forward`` takes as a raw pointer:
    a mismatched tensor would otherwise be read out of bounds or with the wrong layout on the GPU."""
    e = num_experts
    if x.dim() != 2 or not x.is_cuda or not x.is_contiguous():
        raise ValueError("x must be a contiguous (T, D) tensor on the GPU")
    t, d = x.shape
    dev = x.device

    def need(name, tensor, shape, dtype):
        if tensor is None:
            raise ValueError(f"{name} is missing")
        if tuple(tensor.shape) != tuple(shape) or tensor.dtype != dtype:
            raise ValueError(f"{name} must be {tuple(shape)} {dtype}, got {tuple(tensor.shape)} {tensor.dtype}")
        if tensor.device != dev or not tensor.is_contiguous():
            raise ValueError(f"{name} must be contiguous and on {dev}")

    need("router", router, (d, e), x.dtype)
    if router_bias is not None:
        need("router_bias", router_bias, (e,), torch.float32)
    if scales is None:
        need("gate weights", w_gate, (e * d, f), x.dtype)
        need("up weights", w_up, (e * d, f), x.dtype)
        need("down weights", w_down, (e * f, d), x.dtype)
    else:
        if x.dtype != torch.bfloat16 or d % 64 or f % 64:
            raise ValueError("fp8 weights need bf16 activations and D, F multiples of 64")
        need("gate codes", w_gate, (e, f // 16, d // 64, 16, 64), torch.float8_e4m3fn)
        need("up codes", w_up, (e, f // 16, d // 64, 16, 64), torch.float8_e4m3fn)
        need("down codes", w_down, (e, d // 16, f // 64, 16, 64), torch.float8_e4m3fn)
        need("gate scales", scales[0], (e, f), torch.float32)
        need("up scales", scales[1], (e, f), torch.float32)
        need("down scales", scales[2], (e, d), torch.float32)
    if shared is not None:
        fs = shared[0].shape[0]
        need("shared gate", shared[0], (fs, d), x.dtype)
        need("shared up", shared[1], (fs, d), x.dtype)
        need("shared down", shared[2], (d, fs), x.dtype)


def forward(
    x: Tensor,
    router: Tensor,
    router_bias: Tensor | None,
    w_gate: Tensor,
    w_up: Tensor,
    w_down: Tensor,
    num_experts: int,
    top_k: int,
    *,
    scales: tuple[Tensor, Tensor, Tensor] | None = None,
    shared: tuple[Tensor, Tensor, Tensor] | None = None,
    tile_m: int = 16,
    score_fn: int = SCORE_SIGMOID,
    renormalize: bool = False,
    scale_input: bool = True,
    workspace: Tensor | None = None,
    residual: Tensor | None = None,
    norm: tuple[Tensor | None, float] | None = None,
    router_t: Tensor | None = None,
    act_quant: bool = False,
) -> Tensor:
    """The whole layer through ``fs2moe_forward``: one call, intermediates in one workspace.
    ``router_t``: optionally the router matrix expert-major, (E, D), used where the library reads it.
    ``act_quant`` (with ``scales``, i.e. e4m3 weights): the expert products on the fp8 matrix pipe,
    the rows rounded to block-scaled e4m3 inside the call (``FS2MOE_ACT_MXFP8``).
    With ``residual`` ``(T, D)`` the result is ``residual + layer(x)`` from the same accumulation.
    With ``norm`` = (weight or None, eps) the rows are RMS-normalised on the way into the router
    (``fs2moe_forward_norm``): the result is ``[residual +] layer(rms_norm(x))``.

    ``x`` is ``(T, D)``; weights as for :func:`grouped_swiglu` (with ``scales`` they are tiled e4m3
    codes); ``shared`` holds the shared expert's ``(F_s, D)``, ``(F_s, D)``, ``(D, F_s)`` matrices.
    """
    lib = load()
    t, d = x.shape
    if act_quant and scales is None:
        raise ValueError("act_quant goes with e4m3 weights (scales)")
    if scales is None:
        f = w_down.shape[0] // num_experts
    else:
        f = w_gate.shape[1] * 16
    f_shared = shared[0].shape[0] if shared is not None else 0
    check_layer_arguments(x, router, router_bias, w_gate, w_up, w_down, num_experts, f, scales, shared)
    sizes = (t, d, num_experts, top_k, f, f_shared, tile_m, dtype_code(x.dtype))
    need = lib.fs2moe_forward_workspace_bytes(*sizes) if norm is None else lib.fs2moe_forward_norm_workspace_bytes(*sizes)
    if need < 0:
        raise ValueError("fs2moe_forward_workspace_bytes rejected the sizes")
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device)
    if residual is not None and (residual.shape != x.shape or residual.dtype != x.dtype or not residual.is_contiguous()):
        raise ValueError("residual must be a contiguous tensor of x's shape and dtype")
    out = torch.empty_like(x)
    sg, su, sd = scales if scales is not None else (None, None, None)
    hg, hu, hd = shared if shared is not None else (None, None, None)
    mat, score_fn = router_operand(lib, x, router, router_t, score_fn)
    tail = (
        _ptr(residual), _ptr(mat), _ptr(router_bias), _ptr(w_gate), _ptr(w_up), _ptr(w_down), _ptr(sg),
        _ptr(su), _ptr(sd), _ptr(hg), _ptr(hu), _ptr(hd), t, d, num_experts, top_k, f, f_shared,
        tile_m, dtype_code(x.dtype), dtype_code(w_gate.dtype) | (ACT_MXFP8 if act_quant else 0),
        score_fn, int(renormalize),
        int(scale_input), _ptr(workspace), workspace.numel(), _ptr(out), _stream(),
    )
    if norm is None:
        _check(lib.fs2moe_forward(_ptr(x), *tail), "fs2moe_forward")
    else:
        _check_norm_weight(norm[0], x)
        _check(lib.fs2moe_forward_norm(_ptr(x), _ptr(norm[0]), float(norm[1]), *tail), "fs2moe_forward_norm")
    return out

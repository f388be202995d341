"""CPU oracle for the mixture-of-experts feed-forward forward path.

THIS IS TEST INFRASTRUCTURE.  Only the test suite, the smoke check and the
CPU-baseline leg of the benchmark may import it; the product never does.

It restates, in stock torch CPU ops, what fairseq2 computes for this path:

* ``ref_dense_forward``   follows ``src/fairseq2/models/llama4/moe.py:102-157``
  op for op (dense score matrix, E-fold gather, three ``bmm``s of
  ``src/fairseq2/models/transformer/experts.py:102-112``, ``scatter_add_``),
  with the shared expert of ``src/fairseq2/models/transformer/ffn.py:374-395``.
  It is also the formulation timed as the CPU baseline.
* ``ref_sparse_forward``  evaluates the same mathematics one expert at a time
  on only the tokens routed to it, and returns every intermediate the device
  kernels are compared with.
* ``expert_inner_dim``    is the constructor's inner-dimension rule
  (``moe.py:52-65``).
* ``route``               gives the integer artefacts: the selected set per
  token, expert counts, the expert-major / token-ascending permutation implied
  by the reference's ``(E, T)`` score matrix (``moe.py:115-119``), tile-padded
  offsets and the inverse permutation.
* ``rms_norm``            is the normalisation a pre-norm decoder layer applies
  in front of the block (``src/fairseq2/nn/normalization.py:234-236`` as called
  from ``src/fairseq2/models/transformer_lm/decoder_layer.py:187-191``), which
  the device router can apply on the way.

The arithmetic itself lives in PyTorch, which the reference calls directly
(``@`` at ``moe.py:109``, ``torch.topk`` ``:113``, ``sigmoid`` ``:127``,
``gather`` ``:132``, ``scatter_add_`` ``:150``, ``torch.bmm`` and ``SiLU`` at
``experts.py:107-112``, ``F.linear`` via ``nn/projection.py:279-281,517-519``).
The reference holds no test, fixture or golden vector for this path, so the
functions here are pinned by what the mathematics fixes instead (see
``tests/test_oracle_pins.py``): pure-Python brute force on tiny layers, the
dense/sparse identity between two independently written formulations, the
E=1/K=1 reduction to a plain GLU network, K=E, closed forms for the
inner-dimension rule and the score functions, and invariants of the
permutation.  Every function below has such a check; none is "parity unpinned".

Tie rule.  ``torch.topk`` breaks exact ties arbitrarily, and the reference
throws the order away (it scatters into a dense matrix), so only the selected
set matters.  The rule used here and by the device router: descending logit,
ties to the lower expert id, NaN ranks above everything (as in torch).

Extensions beyond the reference (defaults reproduce it): a per-expert router
bias, ``score_fn="softmax"`` with optional renormalisation over the selected
experts, ``scale_on="output"`` (weight the expert output instead of the
expert input), and ``act_quant="mxfp8"``: the inputs of the two expert
products rounded to block-scaled e4m3 (``mx_quantize``; the cast itself is
PyTorch's ``float8_e4m3fn`` conversion, pinned against a brute-force nearest
search over all 256 codes in ``tests/test_oracle_pins.py``).
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch
import torch.nn.functional as F
from torch import Tensor


# --------------------------------------------------------------------------- a1
def expert_inner_dim(
    inner_dim: int,
    use_shared_expert: bool,
    capacity_factor: float,
    *,
    inner_dim_scale: float = 2 / 3,
    inner_dim_to_multiple: int = 1,
    auto_scale: bool = True,
) -> int:
    """Inner dimension of each expert, as derived by ``MoE.__init__`` (``moe.py:52-65``)."""
    if inner_dim_scale != 1.0:
        inner_dim = int(inner_dim * inner_dim_scale)
    if auto_scale:
        inner_dim = int(inner_dim / (capacity_factor + int(use_shared_expert)))
    if inner_dim_to_multiple != 1:
        inner_dim = inner_dim_to_multiple * (
            (inner_dim + inner_dim_to_multiple - 1) // inner_dim_to_multiple
        )
    return inner_dim


# ------------------------------------------------------- in front of the block
def rms_norm(x: Tensor, weight: Tensor | None, eps: float) -> Tensor:
    """RMS normalisation over the last dimension with the arithmetic of
    ``torch.nn.functional.rms_norm``, the routine ``RMSNorm.forward`` calls
    (``nn/normalization.py:234-236``): the mean of squares, ``x * rsqrt(mean + eps)`` and the
    product with the weight in single precision (double stays double), one cast back to the type
    of ``x``.  (The spelled-out path below it, ``:238-247``, used only with a torch that lacks
    the routine, casts before the weight as well: up to one rounding step apart in bf16.)
    ``decoder_layer.py:187-191`` applies the module to the rows before the feed-forward block."""
    xf = x if x.dtype == torch.float64 else x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * (weight if weight.dtype == torch.float64 else weight.float())
    return y.type_as(x)


# --------------------------------------------------------------------------- a2
def router_logits(x: Tensor, router: Tensor, bias: Tensor | None = None) -> Tensor:
    """``x.reshape(-1, D) @ router`` (``moe.py:109``), plus the optional bias."""
    logits = x.reshape(-1, x.shape[-1]) @ router
    if bias is not None:
        logits = logits + bias.to(logits.dtype)
    return logits


def topk_lowest_index(logits: Tensor, k: int) -> Tensor:
    """Indices of the k largest entries per row: descending value, ties to the
    lower index, NaN above +inf.  Returns int64 ``(T, k)`` in that order."""
    l = logits.detach().to(torch.float64)
    key = torch.where(torch.isnan(l), torch.full_like(l, float("inf")), l)
    is_nan = torch.isnan(l).to(torch.float64)
    # Stable sorts: first by descending value (equal values keep index order),
    # then NaNs to the front, again keeping relative order.
    idx = torch.argsort(-key, dim=1, stable=True)
    nan_sorted = torch.gather(is_nan, 1, idx)
    idx2 = torch.argsort(-nan_sorted, dim=1, stable=True)
    idx = torch.gather(idx, 1, idx2)
    return idx[:, :k].contiguous()


def combine_weights(
    logits: Tensor, topk_idx: Tensor, score_fn: str = "sigmoid", renormalize: bool = False
) -> Tensor:
    """Weights ``(T, K)`` of the selected experts.

    ``sigmoid``: ``sigmoid(logit)`` of each selected logit (``moe.py:113,127``).
    ``softmax``: softmax over all E logits, taken at the selected experts; with
    ``renormalize`` divided by their sum (equal to a softmax over the selected
    logits alone).
    """
    sel = torch.gather(logits, 1, topk_idx)
    if score_fn == "sigmoid":
        w = torch.sigmoid(sel)
        if renormalize:
            w = w / w.sum(dim=1, keepdim=True)
        return w
    if score_fn == "softmax":
        if renormalize:
            return torch.softmax(sel, dim=1)
        return torch.gather(torch.softmax(logits, dim=1), 1, topk_idx)
    raise ValueError(f"unknown score_fn {score_fn!r}")


# --------------------------------------------------------------------- a3 / a4
@dataclass
class Routing:
    """Integer routing artefacts (bit-exact contract with the device kernels)."""

    topk_idx: np.ndarray  # (T, K) int32, descending logit / lower id on ties
    counts: np.ndarray  # (E,) int32
    offsets: np.ndarray  # (E + 1,) int32, start row of each expert, tile padded
    perm: np.ndarray  # (M_pad,) int32, token of each row, -1 for padding rows
    inv_perm: np.ndarray  # (T, K) int32, row of pair (t, slot)
    num_rows: int  # M_pad == offsets[E]


def route(topk_idx: Tensor | np.ndarray, num_experts: int, tile_m: int = 1) -> Routing:
    """Counts, padded offsets and the canonical permutation.

    The canonical order is the row-major order of the non-zeros of the
    reference's ``(E, T)`` score matrix (``moe.py:115-119``): expert-major,
    token-ascending.  Each expert's row block is rounded up to ``tile_m`` rows;
    padding rows carry token ``-1``.
    """
    idx = np.asarray(topk_idx, dtype=np.int64)
    t, k = idx.shape
    counts = np.bincount(idx.reshape(-1), minlength=num_experts).astype(np.int32)
    padded = (counts.astype(np.int64) + tile_m - 1) // tile_m * tile_m
    offsets = np.zeros(num_experts + 1, dtype=np.int64)
    np.cumsum(padded, out=offsets[1:])
    m_pad = int(offsets[-1])

    flat_e = idx.reshape(-1)
    flat_t = np.repeat(np.arange(t, dtype=np.int64), k)
    # Expert-major, token-ascending: a stable sort by expert of pairs already in token order.
    order = np.argsort(flat_e, kind="stable")
    starts = np.zeros(num_experts + 1, dtype=np.int64)
    np.cumsum(counts, out=starts[1:])
    e_sorted = flat_e[order]
    rank = np.arange(t * k, dtype=np.int64) - starts[e_sorted]
    rows = offsets[e_sorted] + rank

    perm = np.full(m_pad, -1, dtype=np.int32)
    perm[rows] = flat_t[order].astype(np.int32)
    inv = np.empty(t * k, dtype=np.int32)
    inv[order] = rows.astype(np.int32)
    return Routing(
        idx.astype(np.int32), counts, offsets.astype(np.int32), perm, inv.reshape(t, k), m_pad
    )


# --------------------------------------------------------------------------- a6
# ------------------------------------------------------------ block-scaled e4m3
MX_BLOCK = 32
E4M3_MAX = 448.0


def mx_block_exponent(amax: Tensor) -> Tensor:
    """The shared exponent X of blocks with the given largest magnitudes: the smallest integer with
    ``amax / 2**X <= 448``, i.e. for ``amax = m 2**e`` with ``m`` in [1, 2): ``e - 8`` when
    ``m <= 1.75``, else ``e - 7``.  Zero blocks (and magnitudes below the smallest normal float32)
    get -127; the result is clamped to [-127, 127] (what one byte, X + 127, can say)."""
    a = amax.detach().to(torch.float32)
    m, e = torch.frexp(a)  # a = m 2**e with m in [0.5, 1)
    x = e.to(torch.int32) - 1 - 8 + (m > 0.875).to(torch.int32)
    x = torch.where(a < 2.0 ** -126, torch.full_like(x, -127), x)
    return x.clamp(-127, 127)


def mx_quantize(x: Tensor) -> tuple[Tensor, Tensor]:
    """Rows ``(*, D)`` -> e4m3 codes ``(*, D)`` (``torch.float8_e4m3fn``) and exponent bytes
    ``(*, D / 32)`` (uint8, X + 127): every block of 32 consecutive features is divided by
    ``2**X`` (exact) and rounded to e4m3, to nearest, ties to even."""
    d = x.shape[-1]
    assert d % MX_BLOCK == 0
    v = x.detach().to(torch.float32).reshape(*x.shape[:-1], d // MX_BLOCK, MX_BLOCK)
    xexp = mx_block_exponent(v.abs().amax(dim=-1))
    scaled = torch.ldexp(v, -xexp.unsqueeze(-1))
    codes = scaled.to(torch.float8_e4m3fn).reshape(x.shape)
    return codes, (xexp + 127).to(torch.uint8)


def mx_dequantize(codes: Tensor, scale_bytes: Tensor, dtype: torch.dtype = torch.float32) -> Tensor:
    d = codes.shape[-1]
    v = codes.to(torch.float32).reshape(*codes.shape[:-1], d // MX_BLOCK, MX_BLOCK)
    x = scale_bytes.to(torch.int32) - 127
    return torch.ldexp(v, x.unsqueeze(-1)).reshape(codes.shape).to(dtype)


def mx_round(x: Tensor) -> Tensor:
    """``x`` as the fp8 matrix pipe sees it: quantised and de-quantised, in ``x``'s dtype."""
    return mx_dequantize(*mx_quantize(x), dtype=x.dtype)


def glu_expert(u: Tensor, wg: Tensor, wu: Tensor, wd: Tensor) -> Tensor:
    """One expert: ``(SiLU(u @ Wg) * (u @ Wu)) @ Wd`` (``experts.py:107-112``)."""
    return (F.silu(u @ wg) * (u @ wu)) @ wd


def shared_glu(x: Tensor, gate_w: Tensor, up_w: Tensor, down_w: Tensor) -> Tensor:
    """Shared expert with ``nn.Linear``-oriented weights (``ffn.py:374-395``):
    ``output_proj(inner_proj(x) * silu(gate_proj(x)))``."""
    return F.linear(F.linear(x, up_w) * F.silu(F.linear(x, gate_w)), down_w)


# ------------------------------------------------------------------ whole layer
def ref_dense_forward(
    seqs: Tensor,
    router: Tensor,
    gate: Tensor,
    up: Tensor,
    down: Tensor,
    top_k: int,
    *,
    shared: tuple[Tensor, Tensor, Tensor] | None = None,
    router_bias: Tensor | None = None,
    score_fn: str = "sigmoid",
    renormalize: bool = False,
    scale_on: str = "input",
    activation=F.silu,
) -> Tensor:
    """The reference's dense formulation, op for op (``moe.py:102-157``).  ``activation`` is the
    routed experts' gate activation (``experts.py:84-87``: any module, SiLU by default).

    Every expert runs over all T tokens; unselected pairs get a zero input
    (reference mode) or a zero weight (output-weighted extension).
    """
    x = seqs
    dim = x.shape[-1]
    num_experts = router.shape[1]

    logits = x.reshape(-1, dim) @ router
    if router_bias is not None:
        logits = logits + router_bias.to(logits.dtype)
    num_tokens = logits.shape[0]

    if score_fn == "sigmoid" and not renormalize:
        scores, token_indices = torch.topk(logits, top_k, dim=1)
        scores = (
            torch.full_like(logits, float("-inf")).scatter_(1, token_indices, scores).transpose(0, 1)
        )
        top_scores = torch.sigmoid(scores)
    else:
        idx = topk_lowest_index(logits, top_k)
        w = combine_weights(logits, idx, score_fn, renormalize)
        top_scores = torch.zeros_like(logits).scatter_(1, idx, w).transpose(0, 1)

    token_indices = torch.arange(num_tokens).view(1, -1).expand(num_experts, -1)
    token_indices = token_indices.reshape(-1, 1).expand(-1, dim)

    routed_input = torch.gather(x.reshape(-1, dim), dim=0, index=token_indices)
    if scale_on == "input":
        routed_input = routed_input * top_scores.reshape(-1, 1)
    routed_input = routed_input.reshape(num_experts, -1, dim)

    wg = gate.view(num_experts, -1, gate.shape[-1])
    wu = up.view(num_experts, -1, up.shape[-1])
    wd = down.view(num_experts, -1, down.shape[-1])
    h = activation(torch.bmm(routed_input, wg))
    h = h * torch.bmm(routed_input, wu)
    routed_output = torch.bmm(h, wd).reshape(-1, dim)
    if scale_on == "output":
        routed_output = routed_output * top_scores.reshape(-1, 1)

    if shared is not None:
        out = shared_glu(x, *shared).reshape(-1, dim).clone()
    else:
        out = torch.zeros_like(x.reshape(-1, dim))
    out.scatter_add_(dim=0, index=token_indices, src=routed_output)
    return out.reshape(seqs.shape)


@dataclass
class SparseResult:
    logits: Tensor  # (T, E)
    topk_idx: Tensor  # (T, K) int64
    topk_w: Tensor  # (T, K)
    routing: Routing
    xe: Tensor  # (M_pad, D) expert inputs in permuted order (zeros on padding rows)
    h: Tensor  # (M_pad, F)
    ye: Tensor  # (M_pad, D)
    base: Tensor  # (T, D) shared-expert output or zeros
    out: Tensor  # seqs.shape


def ref_sparse_forward(
    seqs: Tensor,
    router: Tensor,
    gate: Tensor,
    up: Tensor,
    down: Tensor,
    top_k: int,
    *,
    shared: tuple[Tensor, Tensor, Tensor] | None = None,
    router_bias: Tensor | None = None,
    score_fn: str = "sigmoid",
    renormalize: bool = False,
    scale_on: str = "input",
    tile_m: int = 1,
    topk_idx: Tensor | None = None,
    tokens: Tensor | None = None,
    act_quant: str | None = None,
) -> SparseResult:
    """Per-expert evaluation of the layer on only the routed tokens.

    ``act_quant="mxfp8"``: the rows entering the gate/up products and the gated product entering
    the down projection are rounded to block-scaled e4m3 first (``mx_round``); the router, the
    shared expert and the combination see the unrounded rows.

    ``topk_idx`` may be supplied to evaluate with a given selection.  ``tokens``
    restricts the expert evaluation to a subset of token ids (the output rows of
    all other tokens are left at the base value); routing artefacts always cover
    every token.
    """
    assert act_quant in (None, "mxfp8")
    dim = seqs.shape[-1]
    x = seqs.reshape(-1, dim)
    t = x.shape[0]
    num_experts = router.shape[1]
    inner = gate.shape[-1]

    logits = router_logits(x, router, router_bias)
    if topk_idx is None:
        topk_idx = topk_lowest_index(logits, top_k)
    w = combine_weights(logits, topk_idx, score_fn, renormalize)
    r = route(topk_idx.numpy(), num_experts, tile_m)

    wg = gate.view(num_experts, -1, inner)
    wu = up.view(num_experts, -1, inner)
    wd = down.view(num_experts, -1, dim)

    xe = torch.zeros(r.num_rows, dim, dtype=x.dtype)
    h = torch.zeros(r.num_rows, inner, dtype=x.dtype)
    ye = torch.zeros(r.num_rows, dim, dtype=x.dtype)
    inv = torch.from_numpy(r.inv_perm.astype(np.int64))
    perm = torch.from_numpy(r.perm.astype(np.int64))

    keep = None
    if tokens is not None:
        keep = torch.zeros(t, dtype=torch.bool)
        keep[tokens] = True

    # Per-row weight in permuted order.
    row_w = torch.zeros(r.num_rows, dtype=x.dtype)
    row_w[inv.reshape(-1)] = w.reshape(-1)

    for e in range(num_experts):
        lo, n = int(r.offsets[e]), int(r.counts[e])
        if n == 0:
            continue
        rows = torch.arange(lo, lo + n)
        tok = perm[rows]
        if keep is not None:
            m = keep[tok]
            rows, tok = rows[m], tok[m]
            if rows.numel() == 0:
                continue
        u = x[tok]
        if scale_on == "input":
            u = u * row_w[rows, None]
        xe[rows] = u
        if act_quant == "mxfp8":
            # the quantiser reads bf16 rows (the dtype this option exists for): rows scaled on the
            # way in are rounded to bf16 first, as the gathered copy holds them; rows that are
            # bf16 values already pass through that unchanged
            u = mx_round(u.to(torch.bfloat16).to(u.dtype))
        he = F.silu(u @ wg[e]) * (u @ wu[e])
        if act_quant == "mxfp8":
            he = mx_round(he)
        h[rows] = he
        ye[rows] = he @ wd[e]

    base = shared_glu(x, *shared) if shared is not None else torch.zeros_like(x)
    out = base.clone()
    # Ascending expert id, starting from the base: the order scatter_add_ uses (moe.py:150).
    order = torch.argsort(topk_idx, dim=1)
    for j in range(topk_idx.shape[1]):
        slot = order[:, j]
        rows = inv[torch.arange(t), slot]
        y = ye[rows]
        if scale_on == "output":
            y = y * w[torch.arange(t), slot][:, None]
        if keep is not None:
            y = torch.where(keep[:, None], y, torch.zeros_like(y))
        out = out + y
    return SparseResult(logits, topk_idx, w, r, xe, h, ye, base, out.reshape(seqs.shape))


def dense_cpu_baseline_inputs(wl, dtype: torch.dtype):
    """Casts a workload's tensors to the dtype the CPU baseline runs in."""
    c = lambda t: None if t is None else t.to(dtype)
    shared = None
    if wl.shared_gate is not None:
        shared = (c(wl.shared_gate), c(wl.shared_up), c(wl.shared_down))
    return dict(
        seqs=c(wl.x), router=c(wl.router), gate=c(wl.gate), up=c(wl.up), down=c(wl.down),
        top_k=wl.spec.top_k, shared=shared,
        router_bias=None if wl.router_bias is None else wl.router_bias.to(dtype),
        score_fn=wl.spec.mode.score_fn, renormalize=wl.spec.mode.renormalize,
        scale_on=wl.spec.mode.scale_on,
    )

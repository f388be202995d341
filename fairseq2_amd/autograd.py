"""The layer as a differentiable function: forward through the staged kernels, backward through the
same library.

The reference layer is an ordinary composition of torch operators that ``torch.autograd``
differentiates (the trainer calls ``backward`` on the loss, ``trainer.py:586-587``).  Here the
derivation is written out once, against ``moe.py:102-157``, ``experts.py:102-112`` and
``ffn.py:374-395``:

    out[t]   = sum_k c_k * expert_{e_k}(s_k * x[t])  (+ shared(x[t]))      s_k = w_k, c_k = 1 (reference)
                                                                         or s_k = 1, c_k = w_k
    dye      = c * dout[token]                 gathered into expert order      -> fs2moe_dispatch
    dh       = dye @ Wd^T                                                      -> fs2moe_grouped_gemm
    g, u     = xe @ Wg, xe @ Wu                kept by the forward pass        -> fs2moe_grouped_swiglu_keep
                                                or computed again               -> fs2moe_grouped_gemm
    dg, du   = SwiGLU'(g, u, dh),  h = SiLU(g) u                               -> fs2moe_swiglu_backward
    dWd, dWg, dWu = h^T dye, xe^T dg, xe^T du  per expert                      -> fs2moe_grouped_wgrad
    dxe      = dg @ Wg^T + du @ Wu^T                                           -> fs2moe_grouped_gemm_sum
                                                                                  (or two fs2moe_grouped_gemm)
    dw       = <ye, dout[token]>  or  <dxe, x[token]>                          -> fs2moe_pair_dot
    dlogits  = score'(logits) dw                                               -> fs2moe_router_backward
    drouter  = x^T dlogits,  dx += dlogits @ router^T                          -> wgrad / gemm, one group
    dx      += sum_k s_k * dxe[row]            scattered back to token order   -> fs2moe_combine

With the layer's RMS normalisation in front (``decoder_layer.py:187-191``) ``x`` above is the
normalised rows ``xn`` that the router kernel wrote, and one more step turns their gradient into
that of the raw rows and of the norm's weight                                  -> fs2moe_rms_norm_backward

The discrete selection (``torch.topk``) has no gradient, as in the reference.  Intermediates are
rounded to the activation dtype between kernels, as autograd's would be.
"""

from __future__ import annotations

import torch
from torch import Tensor

from fairseq2_amd import _abi


def experts_forward(xe, counts, offsets, wg, wu, wd, e, act=None, rows_per_expert=0):
    """``(ye, g, u)`` of the grouped experts on the rows ``xe``.  Where the expert kernel can, it
    leaves the gate and the up product behind for the backward pass (what autograd would save);
    otherwise ``g`` and ``u`` are None and :func:`experts_backward` computes them again.
    ``rows_per_expert`` as for :func:`fairseq2_amd._abi.grouped_swiglu`: with a bound of up to 16 the
    kernels are those of the inference path at that size (so the values are, too)."""
    if act is not None:
        # a gate activation other than SiLU (experts.py:84-87 takes any module): the module's own
        # forward between the library's plain grouped GEMMs, in f32 with one rounding
        grp = dict(counts=counts, offsets=offsets, num_experts=e)
        g = _abi.grouped_gemm(xe, wg, _abi.W_IN_OUT, **grp)
        u = _abi.grouped_gemm(xe, wu, _abi.W_IN_OUT, **grp)
        h = (act(g.float()) * u.float()).to(xe.dtype)
        return _abi.grouped_gemm(h, wd, _abi.W_IN_OUT, **grp), g, u
    if 1 <= rows_per_expert <= 16:
        return _abi.grouped_swiglu(xe, counts, offsets, wg, wu, wd, e, rows_per_expert=rows_per_expert)[0], None, None
    if _abi.keeps_products(xe.shape[1], wd.shape[0] // e, xe.shape[0], xe.dtype):
        ye, _, g, u = _abi.grouped_swiglu_keep(xe, counts, offsets, wg, wu, wd, e)
        return ye, g, u
    return _abi.grouped_swiglu(xe, counts, offsets, wg, wu, wd, e)[0], None, None


def dense_forward(x, sg, su, sd):
    """``(y, g, u)`` of the shared expert (``nn.Linear``-oriented weights); ``g``, ``u`` as above."""
    if _abi.keeps_products(x.shape[1], sg.shape[0], x.shape[0], x.dtype):
        return _abi.dense_swiglu_keep(x, sg, su, sd)
    return _abi.dense_swiglu(x, sg, su, sd), None, None


def experts_backward(xe, dye, wg, wu, wd, g, u, e, counts, offsets, act, need_w):
    """``(dxe_g, dxe_u, d_wg, d_wu, d_wd)`` of the grouped experts: the input gradient as one
    tensor (``dxe_u`` None) where the two-source kernel runs, else as the two products whose sum it
    is; weight gradients None where ``need_w`` (gate, up, down) says so."""
    IN_OUT, OUT_IN = _abi.W_IN_OUT, _abi.W_OUT_IN
    grp = dict(counts=counts, offsets=offsets, num_experts=e)
    dh = _abi.grouped_gemm(dye, wd, OUT_IN, **grp)
    if act is not None:
        # the module's own derivative, through torch.autograd on its forward (f32, one rounding)
        with torch.enable_grad():
            g32 = g.float().requires_grad_(True)
            a32 = act(g32)
        u32, dh32 = u.float(), dh.float()
        (dg32,) = torch.autograd.grad(a32, g32, dh32 * u32)
        a32 = a32.detach()
        h, dg, du = (a32 * u32).to(xe.dtype), dg32.to(xe.dtype), (dh32 * a32).to(xe.dtype)
    elif g is None:
        g = _abi.grouped_gemm(xe, wg, IN_OUT, **grp)
        u = _abi.grouped_gemm(xe, wu, IN_OUT, **grp)
        h, dg, du = _abi.swiglu_backward(g, u, dh)  # in place over g and u
    else:
        h, dg, du = _abi.swiglu_backward(g, u, dh, in_place=False)  # g, u are autograd's to keep
    d_wd = _abi.grouped_wgrad(h, dye, **grp) if need_w[2] else None
    d_wg = _abi.grouped_wgrad(xe, dg, **grp) if need_w[0] else None
    d_wu = _abi.grouped_wgrad(xe, du, **grp) if need_w[1] else None
    # dxe = dg @ Wg^T + du @ Wu^T: one kernel and one rounding where the library has it, else the
    # two products apart (their sum is then taken where dxe is used)
    if _abi.grouped_gemm_sum_supported(dg.shape[1], xe.shape[1], dg.shape[0], dg.dtype):
        dxe_g, dxe_u = _abi.grouped_gemm_sum(dg, wg, du, wu, **grp), None
    else:
        dxe_g = _abi.grouped_gemm(dg, wg, OUT_IN, **grp)
        dxe_u = _abi.grouped_gemm(du, wu, OUT_IN, **grp)
    return dxe_g, dxe_u, d_wg, d_wu, d_wd


def dense_backward(x, dout, sg, su, sd, g_s, u_s, need_w, need_x):
    """``(dx_parts, d_sg, d_su, d_sd)`` of the shared expert: the input gradient as the two
    products whose sum it is (an empty list unless ``need_x``)."""
    IN_OUT, OUT_IN = _abi.W_IN_OUT, _abi.W_OUT_IN
    dh_s = _abi.grouped_gemm(dout, sd, IN_OUT)
    if g_s is None:
        g_s = _abi.grouped_gemm(x, sg, OUT_IN)
        u_s = _abi.grouped_gemm(x, su, OUT_IN)
        h_s, dg_s, du_s = _abi.swiglu_backward(g_s, u_s, dh_s)
    else:
        h_s, dg_s, du_s = _abi.swiglu_backward(g_s, u_s, dh_s, in_place=False)
    d_sd = _abi.grouped_wgrad(dout, h_s) if need_w[2] else None
    d_sg = _abi.grouped_wgrad(dg_s, x) if need_w[0] else None
    d_su = _abi.grouped_wgrad(du_s, x) if need_w[1] else None
    parts = [_abi.grouped_gemm(dg_s, sg, IN_OUT), _abi.grouped_gemm(du_s, su, IN_OUT)] if need_x else []
    return parts, d_sg, d_su, d_sd


def forward_saving(x, residual, router, wg, wu, wd, sg, su, sd, cfg, norm_w=None):
    """The staged forward pass; returns ``(out, saved)`` with what :func:`backward_from` needs.
    With ``cfg["norm_eps"]`` set the rows are RMS-normalised (weight ``norm_w`` or none) on the way
    into the router; the normalised rows then stand for ``x`` in every later stage and in ``saved``."""
    e, k, tile_m = cfg["num_experts"], cfg["top_k"], cfg["tile_m"]
    score_fn, renorm, scale_input = cfg["score_fn"], cfg["renormalize"], cfg["scale_input"]
    if cfg.get("norm_eps") is not None:
        x, idx, w, logits = _abi.router_topk_norm(x, norm_w, cfg["norm_eps"], router, cfg["router_bias"], k,
                                                  score_fn, renorm, want_logits=True, router_t=cfg.get("router_t"))
    else:
        idx, w, logits = _abi.router_topk(x, router, cfg["router_bias"], k, score_fn, renorm, want_logits=True,
                                          router_t=cfg.get("router_t"))
    disp = _abi.dispatch(idx, w, x, e, tile_m, scale_input, gather=True)
    ye, g, u = experts_forward(disp.xe, disp.counts, disp.offsets, wg, wu, wd, e, cfg.get("activation"),
                               rows_per_expert=x.shape[0] if x.shape[0] <= 16 else 0)
    base = g_s = u_s = None
    if sg is not None:
        base, g_s, u_s = dense_forward(x, sg, su, sd)
    out = _abi.combine(ye, disp.inv_perm, idx, w, base, not scale_input, out=base, residual=residual)
    xn = x if cfg.get("norm_eps") is not None else None
    return out, (idx, w, logits, disp.counts, disp.offsets, disp.inv_perm, disp.xe, ye, g, u, g_s, u_s, xn)


def backward_from(x, router, wg, wu, wd, sg, su, sd, saved, cfg, dout, need):
    """Gradients ``(dx, d_router, d_wg, d_wu, d_wd, d_sg, d_su, d_sd)`` (None where ``need`` -- in
    that order -- says so) from the output gradient and the intermediates of :func:`forward_saving`."""
    idx, w, logits, counts, offsets, inv_perm, xe, ye, g, u, g_s, u_s = saved[:12]
    e, tile_m = cfg["num_experts"], cfg["tile_m"]
    score_fn, renorm, scale_input = cfg["score_fn"], cfg["renormalize"], cfg["scale_input"]
    dout = dout.contiguous()
    OUT_IN = _abi.W_OUT_IN

    # output gradients in expert order (times the combine weight when it scales the output);
    # the permutation is the forward pass's: dispatch is deterministic
    dye = _abi.dispatch(idx, w, dout, e, tile_m, not scale_input, gather=True).xe
    dxe_g, dxe_u, d_wg, d_wu, d_wd = experts_backward(
        xe, dye, wg, wu, wd, g, u, e, counts, offsets, cfg.get("activation"), need[2:5])

    # combine weights -> logits -> router and x
    if scale_input:
        d_w = _abi.pair_dot(dxe_g, inv_perm, x, a2=dxe_u)
    else:
        d_w = _abi.pair_dot(ye, inv_perm, dout)
    dl = _abi.router_backward(logits, idx, w, d_w, score_fn, renorm, x.dtype)
    # the two products with the router matrix read rows of 16 bytes: with a number of experts that
    # is not a multiple of 8, zero columns are appended (they add nothing) and cut off again
    pad = -e % 8
    if pad:
        dl = torch.nn.functional.pad(dl, (0, pad))
        router = torch.nn.functional.pad(router, (0, pad))
    d_router = _abi.grouped_wgrad(x, dl)[:, :e].contiguous() if need[1] else None
    dx_parts = [_abi.grouped_gemm(dl, router, OUT_IN)] if need[0] else []

    d_sg = d_su = d_sd = None
    if sg is not None:
        parts, d_sg, d_su, d_sd = dense_backward(x, dout, sg, su, sd, g_s, u_s, need[5:8], need[0])
        dx_parts += parts

    dx = None
    if need[0]:
        # dx[t] = sum_k s_k dxe[row(t, k)] + the dense terms (at most three: router, and two of the
        # shared expert): two scatter passes, one per half of dxe, each starting from up to two dense
        # rows (the kernel's base and residual operands), everything summed in f32
        dense = dx_parts + [None] * (3 - len(dx_parts))
        if dxe_u is None and dense[2] is not None:
            dense = [dense[0] + dense[1], dense[2], None]  # one pass takes two dense terms
        t1 = _abi.combine(dxe_g, inv_perm, idx, w, dense[0], scale_input, residual=dense[1])
        dx = t1 if dxe_u is None else _abi.combine(dxe_u, inv_perm, idx, w, t1, scale_input, out=t1,
                                                   residual=dense[2])
    return dx, d_router, d_wg, d_wu, d_wd, d_sg, d_su, d_sd


class MoEFunction(torch.autograd.Function):
    """``forward(x, residual, router, wg, wu, wd, sg, su, sd, norm_w, cfg)``; ``cfg`` carries the
    integers (and ``norm_eps`` when the rows are normalised first; ``norm_w`` may then still be None)."""

    @staticmethod
    def forward(ctx, x, residual, router, wg, wu, wd, sg, su, sd, norm_w, cfg):  # noqa: D102
        out, saved = forward_saving(x, residual, router, wg, wu, wd, sg, su, sd, cfg, norm_w)
        ctx.cfg = cfg
        ctx.has_residual = residual is not None
        ctx.save_for_backward(x, router, wg, wu, wd, sg, su, sd, norm_w, *saved)
        return out

    @staticmethod
    @torch.no_grad()
    def backward(ctx, dout):  # noqa: D102
        x, router, wg, wu, wd, sg, su, sd, norm_w, *saved = ctx.saved_tensors
        n = ctx.needs_input_grad
        normed = ctx.cfg.get("norm_eps") is not None
        # through the normalisation the rows' gradient is needed for the weight's as well
        need = (n[0] or (normed and n[9]), n[2], n[3], n[4], n[5], n[6], n[7], n[8])
        xn = saved[12]
        dx, d_router, d_wg, d_wu, d_wd, d_sg, d_su, d_sd = backward_from(
            xn if normed else x, router, wg, wu, wd, sg, su, sd, tuple(saved), ctx.cfg, dout, need)
        d_norm_w = None
        if normed and dx is not None:
            dx, d_norm_w = _abi.rms_norm_backward(x, norm_w, ctx.cfg["norm_eps"], dx,
                                                  want_weight_grad=bool(n[9]))
            if not n[0]:
                dx = None
        d_res = dout if ctx.has_residual and n[1] else None
        return dx, d_res, d_router, d_wg, d_wu, d_wd, d_sg, d_su, d_sd, d_norm_w, None


def _sum_rounded_once(a: Tensor, b: Tensor | None) -> Tensor:
    return a if b is None else (a.float() + b.float()).to(a.dtype)


class GroupedExpertsFunction(torch.autograd.Function):
    """The grouped experts alone, ``forward(xe, counts, offsets, wg, wu, wd, e, act, rows_per_expert)``
    -> ``ye``: what :class:`fairseq2_amd.moe.GroupedExpertNetwork` runs when called by itself in
    training (``experts.py:201-213``)."""

    @staticmethod
    def forward(ctx, xe, counts, offsets, wg, wu, wd, e, act, rows_per_expert=0):  # noqa: D102
        ye, g, u = experts_forward(xe, counts, offsets, wg, wu, wd, e, act, rows_per_expert)
        ctx.e, ctx.act = e, act
        ctx.save_for_backward(xe, counts, offsets, wg, wu, wd, g, u)
        return ye

    @staticmethod
    @torch.no_grad()
    def backward(ctx, dye):  # noqa: D102
        xe, counts, offsets, wg, wu, wd, g, u = ctx.saved_tensors
        n = ctx.needs_input_grad
        dxe_g, dxe_u, d_wg, d_wu, d_wd = experts_backward(
            xe, dye.contiguous(), wg, wu, wd, g, u, ctx.e, counts, offsets, ctx.act, n[3:6])
        return (_sum_rounded_once(dxe_g, dxe_u) if n[0] else None), None, None, d_wg, d_wu, d_wd, None, None, None


class DenseSwiGLUFunction(torch.autograd.Function):
    """The shared expert alone, ``forward(x, sg, su, sd)`` -> ``y`` with ``nn.Linear``-oriented
    weights: :class:`fairseq2_amd.moe.GLUFeedForwardNetwork` in training (``ffn.py:374-395``)."""

    @staticmethod
    def forward(ctx, x, sg, su, sd):  # noqa: D102
        y, g, u = dense_forward(x, sg, su, sd)
        ctx.save_for_backward(x, sg, su, sd, g, u)
        return y

    @staticmethod
    @torch.no_grad()
    def backward(ctx, dy):  # noqa: D102
        x, sg, su, sd, g, u = ctx.saved_tensors
        n = ctx.needs_input_grad
        parts, d_sg, d_su, d_sd = dense_backward(x, dy.contiguous(), sg, su, sd, g, u, n[1:4], n[0])
        return (_sum_rounded_once(*parts) if n[0] else None), d_sg, d_su, d_sd

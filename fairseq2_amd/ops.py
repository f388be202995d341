"""The layer as a registered torch operator, ``torch.ops.fairseq2_amd.moe_forward``.

fairseq2 can wrap its decoder layers in ``torch.compile``
(``src/fairseq2/models/transformer_lm/compiler.py:14-17``).  A tracing compiler cannot look through
a ``ctypes`` call, so :class:`fairseq2_amd.MoE` calls the library through this operator while it is
being traced: the operator carries a shape-only ("fake") implementation for the tracer and the real
one, the whole-layer entry point of the library, for the GPU.  Outside a trace the module calls the
library directly (an operator dispatch costs more host time than a decode-sized layer takes).

Training under ``torch.compile``: the operator has an autograd formula, a second registered operator
``torch.ops.fairseq2_amd.moe_backward`` that recomputes the forward pass's intermediates (normalised
rows, routing, gathered rows, expert outputs) and runs the backward kernels of :mod:`fairseq2_amd.autograd`; a
compiled layer therefore stays one graph in training as well, for the recomputation's price.  Eager
training does not pay it (the module keeps the intermediates of its own forward pass).
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from fairseq2_amd import _abi


@torch.library.custom_op("fairseq2_amd::moe_forward", mutates_args=(), device_types="cuda")
def moe_forward(
    x: Tensor,
    router: Tensor,
    router_bias: Optional[Tensor],
    w_gate: Tensor,
    w_up: Tensor,
    w_down: Tensor,
    s_gate: Optional[Tensor],
    s_up: Optional[Tensor],
    s_down: Optional[Tensor],
    shared_gate: Optional[Tensor],
    shared_up: Optional[Tensor],
    shared_down: Optional[Tensor],
    residual: Optional[Tensor],
    norm_weight: Optional[Tensor],
    num_experts: int,
    top_k: int,
    tile_m: int,
    score_fn: int,
    renormalize: bool,
    scale_input: bool,
    normed: bool,
    norm_eps: float,
) -> Tensor:
    """``x`` is ``(T, D)``; arguments as for :func:`fairseq2_amd._abi.forward` (``s_*`` given:
    the weights are tiled e4m3 codes; ``normed``: RMS-normalise the rows first)."""
    return _abi.forward(
        x, router, router_bias, w_gate, w_up, w_down, num_experts, top_k,
        scales=None if s_gate is None else (s_gate, s_up, s_down),
        shared=None if shared_gate is None else (shared_gate, shared_up, shared_down),
        tile_m=tile_m, score_fn=score_fn, renormalize=renormalize, scale_input=scale_input,
        residual=residual, norm=(norm_weight, norm_eps) if normed else None,
        router_t=_abi.router_expert_major(router),
    )


@moe_forward.register_fake
def _moe_forward_fake(x, *args, **kwargs):
    return torch.empty_like(x)


@torch.library.custom_op("fairseq2_amd::moe_backward", mutates_args=(), device_types="cuda")
def moe_backward(
    grad_out: Tensor,
    x: Tensor,
    router: Tensor,
    router_bias: Optional[Tensor],
    w_gate: Tensor,
    w_up: Tensor,
    w_down: Tensor,
    shared_gate: Optional[Tensor],
    shared_up: Optional[Tensor],
    shared_down: Optional[Tensor],
    num_experts: int,
    top_k: int,
    tile_m: int,
    score_fn: int,
    renormalize: bool,
    scale_input: bool,
    norm_weight: Optional[Tensor],
    normed: bool,
    norm_eps: float,
) -> list[Tensor]:
    """Gradients of ``moe_forward`` for ``x``, ``router``, the three expert weights, (when given)
    the three shared-expert weights and (when given) the norm's weight, in that order."""
    from fairseq2_amd.autograd import backward_from, forward_saving

    cfg = dict(num_experts=num_experts, top_k=top_k, tile_m=tile_m, score_fn=score_fn,
               renormalize=renormalize, scale_input=scale_input, router_bias=router_bias,
               norm_eps=norm_eps if normed else None, router_t=_abi.router_expert_major(router))
    _, saved = forward_saving(x, None, router, w_gate, w_up, w_down, shared_gate, shared_up,
                              shared_down, cfg, norm_weight)
    grads = list(backward_from(saved[12] if normed else x, router, w_gate, w_up, w_down, shared_gate,
                               shared_up, shared_down, saved, cfg, grad_out, (True,) * 8))
    if normed:
        grads[0], d_norm_w = _abi.rms_norm_backward(x, norm_weight, norm_eps, grads[0])
        grads.append(d_norm_w)
    return [g for g in grads if g is not None]


@moe_backward.register_fake
def _moe_backward_fake(grad_out, x, router, router_bias, w_gate, w_up, w_down, shared_gate,
                       shared_up, shared_down, num_experts, top_k, tile_m, score_fn, renormalize,
                       scale_input, norm_weight, normed, norm_eps):
    out = [torch.empty_like(t) for t in (x, router, w_gate, w_up, w_down)]
    if shared_gate is not None:
        out += [torch.empty_like(t) for t in (shared_gate, shared_up, shared_down)]
    if normed and norm_weight is not None:
        out.append(torch.empty_like(norm_weight))
    return out


def _setup_context(ctx, inputs, output):
    (x, router, router_bias, w_gate, w_up, w_down, s_gate, s_up, s_down, shared_gate, shared_up,
     shared_down, residual, norm_weight, num_experts, top_k, tile_m, score_fn, renormalize,
     scale_input, normed, norm_eps) = inputs
    if s_gate is not None:
        ctx.unsupported = "e4m3 weights are forward-only"
        return
    ctx.unsupported = None
    ctx.ints = (num_experts, top_k, tile_m, score_fn, renormalize, scale_input)
    ctx.norm = (normed, norm_eps)
    ctx.has_residual = residual is not None
    ctx.has_shared = shared_gate is not None
    ctx.has_norm_weight = normed and norm_weight is not None
    ctx.save_for_backward(x, router, router_bias, w_gate, w_up, w_down, shared_gate, shared_up,
                          shared_down, norm_weight if normed else None)


def _backward(ctx, grad_out):
    if ctx.unsupported is not None:
        raise RuntimeError(f"fairseq2_amd::moe_forward: {ctx.unsupported}")
    x, router, router_bias, w_gate, w_up, w_down, sg, su, sd, norm_w = ctx.saved_tensors
    grads = torch.ops.fairseq2_amd.moe_backward(
        grad_out.contiguous(), x, router, router_bias, w_gate, w_up, w_down, sg, su, sd, *ctx.ints,
        norm_w, *ctx.norm)
    dx, d_router, d_wg, d_wu, d_wd = grads[:5]
    d_sg, d_su, d_sd = grads[5:8] if ctx.has_shared else (None, None, None)
    d_norm_w = grads[-1] if ctx.has_norm_weight else None
    d_res = grad_out if ctx.has_residual else None
    # one entry per argument of moe_forward
    return (dx, d_router, None, d_wg, d_wu, d_wd, None, None, None, d_sg, d_su, d_sd, d_res, d_norm_w,
            None, None, None, None, None, None, None, None)


moe_forward.register_autograd(_backward, setup_context=_setup_context)

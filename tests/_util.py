"""Shared helpers of the GPU parity tests."""

from __future__ import annotations

import numpy as np
import torch

import workloads as W
from workloads import build_module  # noqa: F401
from oracle import moe_oracle as O

TORCH_DTYPE = {"fp32": torch.float32, "bf16": torch.bfloat16}

# Output tolerance, two statements per comparison.
#   element-wise: |y - ref| <= atol + rtol * |ref| with atol tied to the output RMS (outputs are
#     zero-mean sums, so a pure relative test is ill-conditioned near zero);
#   overall: rms(y - ref) <= RMS_TOL * rms(ref).
# bf16: rtol 2e-2 (the stated bound for bf16).  Every term of an output element passes three bf16
#   roundings (the scaled or plain input row, h, the expert's output row) and the sum a fourth; each
#   is at most 2^-9 relative, so the error of an element behaves like a zero-mean variable of
#   standard deviation sigma ~ 2^-9 * rms(ref) * c, c between 1 and 2 with the SiLU gate's slope
#   (0.37 % of rms(ref) in the CPU emulation of the rounding points at K = 16 with scaled inputs,
#   tests/test_oracle_pins.py).  The largest of N such errors is about sqrt(2 ln N) sigma: 5.3 sigma
#   = 2 % of rms(ref) for the 5.6e5 elements of a 1100 x 512 output: with that many elements, K >= 8
#   and the rows scaled on the way in (a fourth rounding per term), atol = 2 % sits AT the expected
#   maximum (a seeded case did land at 1.03 of it).  Such cases, and only they, pass atol_scale = 2
#   (4e-2 * rms, 10 sigma); everything else is held to 2e-2.  The overall statement, RMS_TOL = 1e-2,
#   is the sharp one everywhere: 2.7 sigma-units above the emulation's 0.37 %.  About one drawn case
#   in a thousand still has a single element at 1.0-1.1 of the element-wise bound with few terms
#   (two cancelling expert rows under a heavy-tailed gated product); the seeded sweep settles
#   those against emulate_device_rounding below instead of widening the bound.
# fp32: rtol 1e-4, atol 1e-4 * rms, RMS_TOL 2e-5 (f32 MFMA accumulation order differs from the CPU's).
TOL = {"bf16": (2e-2, 2e-2), "fp32": (1e-4, 1e-4)}
RMS_TOL = {"bf16": 1e-2, "fp32": 2e-5}


def oracle_routing(wl: W.Workload):
    """fp64 logits -> selected experts (descending, ties to the lower id) and weights."""
    b = None if wl.router_bias is None else wl.router_bias.double()
    logits = O.router_logits(wl.x.double(), wl.router.double(), b)
    idx = O.topk_lowest_index(logits, wl.spec.top_k)
    w = O.combine_weights(logits, idx, wl.spec.mode.score_fn, wl.spec.mode.renormalize)
    return logits, idx, w


def oracle_forward(wl: W.Workload, idx, tile_m: int, tokens=None, dtype=torch.float32, act_quant="spec"):
    c = lambda t: None if t is None else t.to(dtype)
    shared = (c(wl.shared_gate), c(wl.shared_up), c(wl.shared_down)) if wl.spec.shared else None
    return O.ref_sparse_forward(
        c(wl.x), c(wl.router), c(wl.gate), c(wl.up), c(wl.down), wl.spec.top_k,
        shared=shared, router_bias=c(wl.router_bias),
        score_fn=wl.spec.mode.score_fn, renormalize=wl.spec.mode.renormalize,
        scale_on=wl.spec.mode.scale_on, tile_m=tile_m, topk_idx=idx, tokens=tokens,
        act_quant=wl.spec.act_quant if act_quant == "spec" else act_quant,
    )


def output_bound(ref: torch.Tensor, dtype: str, atol_scale: float = 1.0) -> torch.Tensor:
    """The element-wise bound of :func:`assert_output_close`: atol tied to rms(ref), plus rtol |ref|."""
    rtol, atol_rel = TOL[dtype]
    ref = ref.double()
    return atol_rel * atol_scale * float(ref.pow(2).mean().sqrt()) + rtol * ref.abs()


def assert_output_close(got: torch.Tensor, ref: torch.Tensor, dtype: str, what: str = "output",
                        atol_scale: float = 1.0):
    got = got.detach().double().cpu().reshape(ref.shape)
    ref = ref.double()
    rtol, atol_rel = TOL[dtype]
    atol_rel *= atol_scale
    rms = float(ref.pow(2).mean().sqrt())
    atol = atol_rel * rms
    err = (got - ref).abs()
    bound = output_bound(ref, dtype, atol_scale)
    worst = float((err / bound).max()) if err.numel() else 0.0
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    assert worst <= 1.0, (
        f"{what}: max err/bound = {worst:.3f} (max abs err {float(err.max()):.3e}, rms {rms:.3e}, "
        f"rtol {rtol}, atol {atol:.3e})"
    )
    err_rms = float(err.pow(2).mean().sqrt()) if err.numel() else 0.0
    assert err_rms <= RMS_TOL[dtype] * rms or rms == 0.0, (
        f"{what}: rms error {err_rms:.3e} above {RMS_TOL[dtype]} of the output rms {rms:.3e}"
    )
    print(f"  {what}: worst err/bound {worst:.3f}, rms err / rms {err_rms / rms if rms else 0.0:.2e}", flush=True)
    return worst


def emulate_device_rounding(wl: W.Workload, idx, w, residual=None):
    """The layer evaluated on the CPU in f32 with a bf16 rounding at every point where the device
    rounds (the scaled input row in the reference mode, h, the expert's output row, the final sum in
    ascending expert id): what the HIP path computes up to the order of f32 additions inside a dot
    product.  bf16 workloads without a shared expert only.  Returns the (T, D) result as f32."""
    s = wl.spec
    assert s.dtype == "bf16" and not s.shared
    t, d, e, f = s.num_tokens, s.model_dim, s.num_experts, s.inner_dim
    bf = lambda v: v.to(torch.bfloat16).float()  # noqa: E731
    x = wl.x.reshape(t, d).float()
    gate, up, down = wl.gate.float().view(e, d, f), wl.up.float().view(e, d, f), wl.down.float().view(e, f, d)
    w32 = w.float()
    out = torch.zeros(t, d) if residual is None else residual.reshape(t, d).float().clone()
    scale_in = s.mode.scale_on == "input"
    for ex in range(e):
        sel = idx == ex
        tok = sel.any(dim=1).nonzero().squeeze(1)
        if tok.numel() == 0:
            continue
        we = (w32 * sel).sum(dim=1)[tok]
        xe = bf(x[tok] * we[:, None]) if scale_in else x[tok]
        h = bf(torch.nn.functional.silu(xe @ gate[ex]) * (xe @ up[ex]))
        ye = bf(h @ down[ex])
        out[tok] += ye if scale_in else ye * we[:, None]
    return bf(out)


def assert_routing_equal(idx_gpu, disp, r: O.Routing, what: str = ""):
    """Bit-exact comparison of every integer artefact."""
    np.testing.assert_array_equal(idx_gpu.cpu().numpy(), r.topk_idx, err_msg=f"{what} topk_idx")
    np.testing.assert_array_equal(disp.counts.cpu().numpy(), r.counts, err_msg=f"{what} counts")
    np.testing.assert_array_equal(disp.offsets.cpu().numpy(), r.offsets, err_msg=f"{what} offsets")
    perm = disp.perm.cpu().numpy()
    np.testing.assert_array_equal(perm[: r.num_rows], r.perm, err_msg=f"{what} perm")
    assert (perm[r.num_rows :] == -1).all(), f"{what} perm tail"
    np.testing.assert_array_equal(disp.inv_perm.cpu().numpy(), r.inv_perm, err_msg=f"{what} inv_perm")

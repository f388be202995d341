"""The opt-in W8A8 expert path on the GPU (block-scaled e4m3 activations against e4m3 weights on the
fp8 matrix pipe) against the CPU oracle with the same quantisation (``act_quant="mxfp8"``).

Bit-exact where the arithmetic is integer-like (the quantiser: exponent bytes and codes); within the
bf16 bound of tests/_util.py for the expert outputs, whose reference is evaluated on the same
quantised inputs.  The gated product is quantised by the device from f32 sums that differ from the
oracle's in the last bits, so a code may land on the other side of a rounding boundary: compared
within one e4m3 step.  The price of the format itself, against the unquantised layer, is measured
and bounded at the end.
"""

import numpy as np
import pytest
import torch

from fairseq2_amd import _abi
import workloads as W
from oracle import moe_oracle as O
from tests._util import (
    TORCH_DTYPE, assert_output_close, assert_routing_equal, build_module, oracle_forward, oracle_routing,
)

pytestmark = pytest.mark.gpu


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("rows,d", [(1, 128), (7, 384), (300, 2048), (1025, 256)])
def test_mx_quantize_matches_oracle_bit_for_bit(gpu_device, rows, d):
    _say("mx_quantize", rows, d)
    g = torch.Generator().manual_seed(rows + d)
    x = (torch.randn(rows, d, generator=g) * torch.exp(4 * torch.randn(rows, 1, generator=g))).to(torch.bfloat16)
    x[0, :32] = 0  # a zero block
    if rows > 2:
        x[1, :8] = torch.tensor([17.0, 19.0, 448.0, -448.0, 2.0 ** -20, 28.0, -17.0, 3.0])  # exact ties
        x[2, :32] = 2.0 ** -130  # below the smallest normal float: the smallest exponent byte
        x[2, 32:64] = 3.0e38  # the largest
    want_c, want_s = O.mx_quantize(x)
    got_c, got_s = _abi.mx_quantize(x.to(gpu_device))
    assert got_s.shape == (d // 128, rows, 4)
    assert torch.equal(_abi.mx_scales_row_major(got_s).cpu(), want_s)
    assert torch.equal(_abi.mx_scales_k_major(want_s.to(gpu_device)), got_s)
    assert torch.equal(got_c.cpu(), want_c.view(torch.uint8))


def _fp8_experts(e, d, f, seed):
    g = torch.Generator().manual_seed(seed)
    gate, up = (0.05 * torch.randn(e * d, f, generator=g) for _ in range(2))
    down = 0.05 * torch.randn(e * f, d, generator=g)
    out = {}
    for name, w in (("gate", gate), ("up", up), ("down", down)):
        q, s = W.quantize_fp8_per_channel(w.to(torch.bfloat16), e)
        out[name] = (q, s, W.dequantize_fp8_per_channel(q, s))
    return out


@pytest.mark.parametrize(
    "rows,d,f",
    [
        ([300, 0, 129, 1, 256, 64], 256, 384),  # heavy, empty, just over the light bound, one row
        ([513, 40], 128, 128),                  # one unit of k, one channel tile
        ([128] * 8, 384, 640),                  # light tiles only; D, F off the 256-channel tiles
    ],
)
@pytest.mark.parametrize("mapped", [False, True])
def test_grouped_swiglu_w8a8_matches_oracle(gpu_device, rows, d, f, mapped):
    _say("grouped_swiglu_w8a8", rows, d, f, mapped)
    dev = gpu_device
    e, tile_m = len(rows), 16
    wts = _fp8_experts(e, d, f, seed=d + f)
    counts = torch.tensor(rows, dtype=torch.int32)
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum((counts + tile_m - 1) // tile_m * tile_m, 0)
    total = int(offsets[-1])
    g = torch.Generator().manual_seed(1)
    if mapped:
        # rows read through a map from a token matrix (tokens repeat, as with top-k > 1)
        tokens = 200
        xt = torch.randn(tokens, d, generator=g).to(torch.bfloat16)
        row_map = torch.full((total,), -1, dtype=torch.int32)
        for ex in range(e):
            lo = int(offsets[ex])
            row_map[lo : lo + rows[ex]] = torch.randint(0, tokens, (rows[ex],), generator=g, dtype=torch.int32)
        x_rows = xt[row_map.clamp(min=0).long()]
        src = xt
    else:
        x_rows = torch.randn(total, d, generator=g).to(torch.bfloat16)
        row_map, src = None, x_rows
    xq, xs = O.mx_quantize(src)
    pk = lambda name: _abi.pack_fp8_weights(wts[name][0].to(dev), e)  # noqa: E731
    ye, hq, hs = _abi.grouped_swiglu_w8a8(
        xq.view(torch.uint8).to(dev), _abi.mx_scales_k_major(xs.to(dev)), counts.to(dev), offsets.to(dev), pk("gate"), pk("up"), pk("down"),
        tuple(wts[n][1].to(dev) for n in ("gate", "up", "down")), e,
        row_map=None if row_map is None else row_map.to(dev),
    )
    torch.cuda.synchronize()
    hs_rows = _abi.mx_scales_row_major(hs).cpu()
    xr = O.mx_round(x_rows.double())
    for ex in range(e):
        lo, n = int(offsets[ex]), rows[ex]
        if n == 0:
            continue
        u = xr[lo : lo + n]
        wg, wu, wd = (wts[k][2].double().view(e, -1, wts[k][2].shape[1])[ex] for k in ("gate", "up", "down"))
        h_ref = torch.nn.functional.silu(u @ wg) * (u @ wu)
        h_dev = O.mx_dequantize(hq[lo : lo + n].cpu().view(torch.float8_e4m3fn), hs_rows[lo : lo + n]).double()
        # the device's codes: the oracle's, or a neighbour where the f32 sum sat on a rounding boundary:
        # one e4m3 step, which is 2^-3 of the value at most in the normal range and 2^-9 of the block's
        # scale (at most 2^-16 of its largest element) below it; twice that if the block's largest
        # element sat on a boundary and the two sides chose scales a binade apart
        h_q = O.mx_round(h_ref)
        amax = h_ref.abs().reshape(n, -1, 32).amax(-1, keepdim=True).expand(n, h_ref.shape[1] // 32, 32).reshape(n, -1)
        step = torch.maximum(h_q.abs(), h_dev.abs()) * 2.0 ** -3 + amax * 2.0 ** -15
        diff = (h_dev - h_q).abs()
        assert bool((diff <= step).all()), f"expert {ex}: h codes, worst {float((diff / step).max()):.2f} steps"
        assert float((diff > 0).double().mean()) < 2e-2, f"expert {ex}: {float((diff > 0).double().mean()):.2%} of the codes differ"
        # the output from the device's own h (so that a flipped code does not count twice)
        assert_output_close(ye[lo : lo + n], h_dev @ wd, "bf16", f"expert {ex}")


@pytest.mark.parametrize("mode,shared", [(W.RoutingMode("softmax", True, "output"), False),
                                         (W.RoutingMode("sigmoid", False, "input"), True)])
def test_layer_with_quantised_activations_matches_oracle(gpu_device, mode, shared):
    _say("w8a8 layer", mode, shared)
    spec = W.small_spec(tokens=700, model_dim=256, num_experts=8, top_k=4, inner_dim=384, dtype="bf16",
                        weight_dtype="fp8", zipf_s=1.1, shared=shared, mode=mode, seed=41, act_quant="mxfp8")
    wl = W.make_workload_from_spec(spec)
    _, idx, w = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    m = build_module(wl, gpu_device)
    assert m.experts.act_quant == "mxfp8" and m.experts.runs_w8a8(torch.bfloat16, 700 * 4)
    x = wl.x.to(torch.bfloat16).to(gpu_device)
    with torch.no_grad():
        out, gi, gw, disp = m.forward_with_routing(x)
        assert torch.equal(m(x), out), "forward() takes the same path"
    assert_routing_equal(gi, disp, ref.routing)
    assert_output_close(out, ref.out, "bf16", "against the oracle with the same quantisation", atol_scale=2.0)
    # the price of the format: against the layer without activation quantisation
    plain = oracle_forward(wl, idx, 16, dtype=torch.float64, act_quant=None).out
    rel = float((out.double().cpu() - plain).norm() / plain.norm())
    _say(f"  error of the W8A8 path against unquantised activations: {rel:.3%} of the norm")
    assert rel < 8e-2
    # a decode-sized batch of the same module does not take the fp8 pipe (a weight stream there)
    assert not m.experts.runs_w8a8(torch.bfloat16, 16 * 4)


def test_qwen3_prefill_shape_w8a8(gpu_device):
    _say("full-size qwen3_30b_a3b_w8a8")
    wl = W.make_workload("qwen3_30b_a3b_w8a8")
    spec = wl.spec
    _, idx, w = oracle_routing(wl)
    r = O.route(idx, spec.num_experts, 16)
    m = build_module(wl, gpu_device)
    x = wl.x.to(torch.bfloat16).to(gpu_device)
    with torch.no_grad():
        out, gi, gw, disp = m.forward_with_routing(x)
        again = m(x)
    torch.cuda.synchronize()
    assert m.experts.runs_w8a8(torch.bfloat16, 8192 * 8)
    assert_routing_equal(gi, disp, r, "w8a8")
    assert torch.equal(again, out), "deterministic"
    tok = torch.randperm(spec.num_tokens, generator=torch.Generator().manual_seed(123))[:192]
    ref = oracle_forward(wl, idx, 16, tokens=tok)
    got = out.reshape(-1, spec.model_dim)[tok.to(gpu_device)]
    assert_output_close(got, ref.out.reshape(-1, spec.model_dim)[tok], "bf16", "qwen3 w8a8", atol_scale=2.0)
    plain = oracle_forward(wl, idx, 16, tokens=tok, act_quant=None).out.reshape(-1, spec.model_dim)[tok]
    rel = float((got.double().cpu() - plain.double()).norm() / plain.double().norm())
    _say(f"  error against unquantised activations: {rel:.3%} of the norm")
    assert rel < 8e-2


class _Norm:
    def __init__(self, weight, eps):
        self.weight, self.eps, self.normalized_shape = weight, eps, (weight.numel(),)


def test_one_call_takes_the_fp8_pipe_and_equals_the_stages(gpu_device):
    """``FS2MOE_ACT_MXFP8`` in the whole-layer call: the module's one call (with the normalisation
    and the residual of a pre-norm decoder layer) against the same stages strung together, bit for
    bit, and the refusals of the C entry point."""
    _say("w8a8 one call")
    spec = W.small_spec(tokens=900, model_dim=256, num_experts=8, top_k=2, inner_dim=128, dtype="bf16",
                        weight_dtype="fp8", zipf_s=1.1, shared=True, mode=W.RoutingMode("softmax", True, "output"),
                        seed=5, act_quant="mxfp8")
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device)
    g = torch.Generator().manual_seed(3)
    raw = (1.7 * torch.randn(900, 256, generator=g)).to(torch.bfloat16).to(gpu_device)
    gamma = (1.0 + 0.1 * torch.randn(256, generator=g)).to(torch.bfloat16).to(gpu_device)
    norm = _Norm(gamma, 1e-5)
    assert m.experts.runs_w8a8(torch.bfloat16, 900 * 2)
    with torch.no_grad():
        for residual, nrm in ((None, None), (raw, None), (raw, norm)):
            got = m(raw, residual=residual, norm=nrm)
            args = (raw, residual, None if nrm is None else (nrm.weight, nrm.eps))
            assert torch.equal(got, m._single_call(*args, act_quant=True))
            assert torch.equal(got, m._stages(*args)[0]), "the one call and the stages differ"
            w8a16 = m._single_call(*args, act_quant=False)
            assert not torch.equal(got, w8a16), "the option changed nothing"
            rel = float((got.double() - w8a16.double()).norm() / w8a16.double().norm())
            assert rel < 8e-2, rel
    torch.cuda.synchronize()
    # the C entry point refuses the option where it does not apply
    ex = m.experts
    weights = (ex.gate_q, ex.inner_q, ex.output_q)
    scales = (ex.gate_scale, ex.inner_scale, ex.output_scale)
    common = dict(scales=scales, score_fn=_abi.SCORE_SOFTMAX, renormalize=True)
    with pytest.raises(RuntimeError, match="scale_input"):
        _abi.forward(raw, m.router.detach(), m.router_bias, *weights, 8, 2, scale_input=True, act_quant=True, **common)
    with pytest.raises(ValueError, match="e4m3"):
        _abi.forward(raw, m.router.detach(), m.router_bias, ex.gate_proj.detach(), ex.inner_proj.detach(),
                     ex.output_proj.detach(), 8, 2, scale_input=False, act_quant=True,
                     score_fn=_abi.SCORE_SOFTMAX, renormalize=True)

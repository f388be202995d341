"""GPU parity of the whole layer through the drop-in module, against the CPU oracle.

Small layers are compared element by element.  The seeded full-size shapes compare every integer
routing artefact bit for bit and the output on a sample of tokens (a token costs 6*K*D*F flops on
the CPU), plus properties that do not depend on size.
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


def _run(wl, device, tile_m=16):
    m = build_module(wl, device, tile_m)
    x = wl.x.to(TORCH_DTYPE[wl.spec.dtype]).to(device)
    with torch.no_grad():
        out, idx, w, disp = m.forward_with_routing(x)
    torch.cuda.synchronize()
    return m, x, out, idx, w, disp


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize(
    "mode,shared,zipf",
    [
        (W.RoutingMode("sigmoid", False, "input"), False, None),  # the reference layer
        (W.RoutingMode("sigmoid", False, "input"), True, None),  # + shared expert (Llama-4)
        (W.RoutingMode("softmax", True, "output"), False, 1.2),  # Mixtral / Qwen3
        (W.RoutingMode("softmax", False, "output"), True, 1.1),
    ],
)
def test_small_layer_matches_oracle(gpu_device, dtype, mode, shared, zipf):
    _say("small layer", dtype, mode, shared, zipf)
    spec = W.small_spec(tokens=600, model_dim=128, num_experts=16, top_k=4, inner_dim=192, dtype=dtype,
                        zipf_s=zipf, shared=shared, mode=mode, seed=33)
    wl = W.make_workload_from_spec(spec)
    _, idx, w = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    m, x, out, gi, gw, disp = _run(wl, gpu_device)
    assert out.shape == x.shape and out.dtype == x.dtype
    assert_routing_equal(gi, disp, ref.routing)
    np.testing.assert_allclose(gw.cpu().double().numpy(), w.numpy(), rtol=5e-5, atol=1e-6)
    assert_output_close(out, ref.out, dtype)


def test_reference_dense_formulation_agrees(gpu_device):
    # The op-for-op restatement of the reference (dense over all experts, torch.topk, scatter_add_)
    # against the device layer: same result although the device never forms the dense tensors.
    spec = W.small_spec(tokens=256, model_dim=64, num_experts=8, top_k=2, inner_dim=128, dtype="fp32", shared=True, seed=2)
    wl = W.make_workload_from_spec(spec)
    ref = O.ref_dense_forward(
        wl.x.double(), wl.router.double(), wl.gate.double(), wl.up.double(), wl.down.double(), 2,
        shared=(wl.shared_gate.double(), wl.shared_up.double(), wl.shared_down.double()),
    )
    _, _, out, *_ = _run(wl, gpu_device)
    assert_output_close(out, ref, "fp32")


@pytest.mark.parametrize("shape", [(1, 1), (1, 7), (3, 1), (2, 3, 5)])
def test_ragged_shapes_and_single_tokens(gpu_device, shape):
    spec = W.small_spec(tokens=int(np.prod(shape)), model_dim=64, num_experts=8, top_k=2, inner_dim=64, dtype="bf16", seed=4)
    wl = W.make_workload_from_spec(spec)
    wl.x = wl.x.reshape(*shape, 64)
    _, idx, _ = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    _, x, out, *_ = _run(wl, gpu_device)
    assert out.shape == (*shape, 64)
    assert_output_close(out, ref.out, "bf16")


@pytest.mark.parametrize("tokens", [1, 2, 4, 5, 8, 13, 16, 17])
@pytest.mark.parametrize("mode", ["reference", "softmax"])
def test_decode_steps_with_a_shared_expert(gpu_device, tokens, mode):
    """The token counts at which routed and shared experts stream their weights (1-4 rows on the
    vector ALUs, 5-16 on the matrix pipe; 17: the GEMM tiles), in the reference's routing mode (rows
    copied and scaled by dispatch in the stages; in the single call up to 16 tokens read through the
    permutation and scaled by the expert kernels) and in softmax mode (rows read through the
    permutation, dispatch inside the router's second kernel): against the oracle, and single call
    against stages."""
    _say("decode step", tokens, mode)
    rm = W.RoutingMode("sigmoid", False, "input") if mode == "reference" else W.RoutingMode("softmax", True, "output")
    spec = W.small_spec(tokens=tokens, model_dim=1024, num_experts=16, top_k=2, inner_dim=320, dtype="bf16",
                        shared=True, zipf_s=1.1, mode=rm, seed=50 + tokens)
    wl = W.make_workload_from_spec(spec)
    _, idx, _ = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    m, x, out, *_ = _run(wl, gpu_device)
    assert_output_close(out, ref.out, "bf16")
    with torch.no_grad():
        single = m(x)  # (out came from the stages)
    torch.cuda.synchronize()
    assert torch.equal(single, out)


@pytest.mark.parametrize("tokens", [1, 3, 4, 9, 16])
@pytest.mark.parametrize("experts,top_k", [(24, 3), (12, 5), (8, 8)])
def test_decode_steps_in_the_reference_mode_without_a_row_copy(gpu_device, tokens, experts, top_k):
    """Up to 16 bf16 tokens in the reference's routing mode: the single call makes no scaled copy of
    the rows, the streaming expert kernels multiply each row by its routing weight as they stage it
    (the weights in expert-row order written by the dispatch, which with a multiple of 8 experts runs
    inside the router's second kernel and otherwise as one block of its own).  Same bits as the
    stages with the copy, with and without the residual; and the oracle."""
    _say("decode step, reference mode", tokens, experts, top_k)
    spec = W.small_spec(tokens=tokens, model_dim=512, num_experts=experts, top_k=top_k, inner_dim=192, dtype="bf16",
                        shared=False, zipf_s=1.1, mode=W.RoutingMode("sigmoid", False, "input"), seed=70 + tokens)
    wl = W.make_workload_from_spec(spec)
    _, idx, _ = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    m, x, out, *_ = _run(wl, gpu_device)  # (the stages)
    assert_output_close(out, ref.out, "bf16")
    res = torch.randn(x.shape, generator=torch.Generator().manual_seed(tokens)).bfloat16().to(gpu_device)
    with torch.no_grad():
        single = m(x)
        single_res = m(x, residual=res)
        staged_res = m._stages(x.reshape(-1, 512), res.reshape(-1, 512))[0].view(x.shape)
    torch.cuda.synchronize()
    assert torch.equal(single, out)
    assert torch.equal(single_res, staged_res)


def test_empty_input(gpu_device):
    wl = W.make_workload_from_spec(W.small_spec(tokens=4, dtype="bf16"))
    m = build_module(wl, gpu_device)
    out = m(torch.empty(0, 5, 64, dtype=torch.bfloat16, device=gpu_device))
    assert out.shape == (0, 5, 64)


def test_top_k_equals_num_experts(gpu_device):
    spec = W.small_spec(tokens=130, model_dim=64, num_experts=4, top_k=4, inner_dim=64, dtype="fp32", seed=6)
    wl = W.make_workload_from_spec(spec)
    _, idx, _ = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    _, _, out, gi, _, disp = _run(wl, gpu_device)
    assert disp.counts.cpu().tolist() == [130] * 4
    assert_output_close(out, ref.out, "fp32")


def test_zero_router_sends_every_token_to_the_first_experts(gpu_device):
    spec = W.small_spec(tokens=300, model_dim=64, num_experts=8, top_k=2, inner_dim=64, dtype="bf16", seed=8)
    wl = W.make_workload_from_spec(spec)
    wl.router.zero_()
    _, idx, _ = oracle_routing(wl)
    assert idx.tolist() == [[0, 1]] * 300
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    _, _, out, gi, gw, disp = _run(wl, gpu_device)
    assert gi.cpu().tolist() == [[0, 1]] * 300
    assert disp.counts.cpu().tolist() == [300, 300, 0, 0, 0, 0, 0, 0]
    assert torch.equal(gw.cpu(), torch.full((300, 2), 0.5))
    assert_output_close(out, ref.out, "bf16")


def test_deterministic_and_tile_size_independent(gpu_device):
    spec = W.small_spec(tokens=900, model_dim=128, num_experts=32, top_k=4, inner_dim=128, dtype="bf16", zipf_s=1.2,
                        mode=W.RoutingMode("softmax", True, "output"), seed=10)
    wl = W.make_workload_from_spec(spec)
    outs = []
    for tile_m in (16, 16, 1, 128):
        _, _, out, *_ = _run(wl, gpu_device, tile_m)
        outs.append(out.cpu())
    for o in outs[1:]:
        assert torch.equal(o, outs[0]), "output must not depend on the run or on the padding granularity"


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("shared", [False, True])
def test_other_expert_activation(gpu_device, dtype, shared):
    """``moe_activation`` other than SiLU (the reference takes any module, ``llama4/moe.py:44``,
    ``experts.py:84-87``): the experts then run as plain grouped GEMMs of the library around the
    module's own activation.  Checked against the same formula in float64."""
    act = torch.nn.GELU(approximate="tanh")
    spec = W.small_spec(tokens=300, model_dim=128, num_experts=8, top_k=2, inner_dim=192, dtype=dtype,
                        shared=shared, seed=5)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device)
    m.experts.activation = act
    assert not m.experts.has_fused_gate
    x = wl.x.to(TORCH_DTYPE[dtype]).to(gpu_device)
    with torch.no_grad():
        out = m(x)
    _, idx, w = oracle_routing(wl)
    t, d, e, f = spec.num_tokens, spec.model_dim, spec.num_experts, spec.inner_dim
    xd = wl.x.reshape(t, d).double()
    ref = O.shared_glu(xd, wl.shared_gate.double(), wl.shared_up.double(), wl.shared_down.double()) if shared else torch.zeros(t, d, dtype=torch.float64)
    for tok in range(t):
        for j in range(spec.top_k):
            ex = int(idx[tok, j])
            u = xd[tok] * w[tok, j]
            h = act(u @ wl.gate.double()[ex * d : (ex + 1) * d]) * (u @ wl.up.double()[ex * d : (ex + 1) * d])
            ref[tok] += h @ wl.down.double()[ex * f : (ex + 1) * f]
    assert_output_close(out, ref, dtype, "GELU-gated experts")
    # the training path gives the same values (its gradients: tests/test_gpu_backward.py)
    assert torch.equal(m.requires_grad_(True)(x).detach(), out)


def test_gradient_and_device_contract(gpu_device):
    # With parameters that require a gradient the call goes through the differentiable function (its
    # gradients are checked in tests/test_gpu_backward.py) and returns the same values; so do the expert
    # modules called by themselves; the row-level entry of the experts is inference only and says so.
    wl = W.make_workload_from_spec(W.small_spec(tokens=8, dtype="bf16"))
    m = build_module(wl, gpu_device)
    x = wl.x.to(torch.bfloat16).to(gpu_device)
    with torch.no_grad():
        want = m(x)
    m.requires_grad_(True)
    got = m(x)
    assert got.requires_grad and torch.equal(got.detach(), want)
    with torch.no_grad():
        assert not m(x).requires_grad
    xe = x.reshape(1, -1, x.shape[-1]).expand(8, -1, -1).contiguous()
    with torch.no_grad():
        want_e = m.experts(xe)
    got_e = m.experts(xe)
    assert got_e.requires_grad and torch.equal(got_e.detach(), want_e)
    counts, offsets = m.experts._uniform_groups(xe.shape[1], xe.device)
    with pytest.raises(RuntimeError, match="forward-only"):
        m.experts.forward_rows(xe.reshape(-1, xe.shape[-1]), counts, offsets)
    with pytest.raises(RuntimeError, match="GPU only"):
        m.requires_grad_(False)(x.cpu())


# ------------------------------------------------------------------------------ seeded full shapes
def _full_size_case(name, gpu_device, sample):
    _say("full-size", name)
    wl = W.make_workload(name)
    spec = wl.spec
    _, idx, w = oracle_routing(wl)
    r = O.route(idx, spec.num_experts, 16)
    m, x, out, gi, gw, disp = _run(wl, gpu_device)
    assert_routing_equal(gi, disp, r, name)
    np.testing.assert_allclose(gw.cpu().double().numpy(), w.numpy(), rtol=5e-5, atol=1e-6)
    assert bool(torch.isfinite(out.float()).all())
    g = torch.Generator().manual_seed(123)
    tok = torch.randperm(spec.num_tokens, generator=g)[:sample]
    ref = oracle_forward(wl, idx, 16, tokens=tok)
    got = out.reshape(-1, spec.model_dim)[tok.to(gpu_device)]
    assert_output_close(got, ref.out.reshape(-1, spec.model_dim)[tok], spec.dtype, name)
    return wl, m, x, out, disp


def test_small_fp32_reference_config(gpu_device):
    # The reference's own CPU-runnable case, compared on every token.
    wl = W.make_workload("small_fp32")
    _, idx, w = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16)
    m, x, out, gi, gw, disp = _run(wl, gpu_device)
    assert_routing_equal(gi, disp, ref.routing)
    assert_output_close(out, ref.out, "fp32")


def test_qwen3_30b_a3b_shape(gpu_device):
    wl, m, x, out, disp = _full_size_case("qwen3_30b_a3b", gpu_device, sample=256)
    counts = disp.counts.cpu()
    assert sorted(counts.tolist(), reverse=True)[:5] == [8138, 7691, 6939, 6074, 5198]
    assert int((counts == 0).sum()) == 17
    # size-independent properties
    with torch.no_grad():
        again = m(x)
        assert torch.equal(again, out), "deterministic"
        # tokens are independent: a permutation of the tokens permutes the output
        p = torch.randperm(x.shape[0] * x.shape[1], device=x.device)
        xp = x.reshape(-1, x.shape[-1])[p].reshape(x.shape)
        outp = m(xp)
        assert torch.equal(outp.reshape(-1, x.shape[-1]), out.reshape(-1, x.shape[-1])[p])


def test_mixtral_8x7b_shape(gpu_device):
    _full_size_case("mixtral_8x7b", gpu_device, sample=256)


def test_llama4_scout_shape(gpu_device):
    wl, m, x, _, _ = _full_size_case("llama4_scout", gpu_device, sample=256)
    # Decode steps on the same weights.  At this size the single call runs the shared expert's two
    # kernels on a stream of the library's own, beside the routed path (the stages run them after it):
    # same bits, repeatedly, with other work of the caller's stream around the calls; and the oracle
    # (a token's output does not depend on the other tokens of the batch).
    d = wl.spec.model_dim
    _, idx, _ = oracle_routing(wl)
    rows = x.reshape(-1, d)
    for t in (1, 5, 16):
        _say("scout decode", t)
        xt = rows[:t].contiguous()
        tok = torch.arange(t)
        ref = oracle_forward(wl, idx, 16, tokens=tok)
        with torch.no_grad():
            staged = m._stages(xt, None)[0]
            singles = []
            for _ in range(3):
                xt.add_(0.0)  # (a kernel of the caller's in front of each call)
                singles.append(m(xt))
                singles[-1].add_(0.0)  # (and one behind it, reading the result)
        torch.cuda.synchronize()
        for got in singles:
            assert torch.equal(got, staged)
        assert_output_close(staged, ref.out.reshape(-1, d)[tok], "bf16", f"scout decode, {t} tokens")
    # the same step captured: the graph holds both streams' kernels and replays to the eager bits
    from fairseq2_amd import GraphedForward

    xs = [rows[:5].contiguous(), rows[5:10].contiguous(), rows[10:15].contiguous()]
    with torch.no_grad():
        eager = [m(xi).clone() for xi in xs]
        graphed = GraphedForward(m, xs[0])
        for rep in range(2):
            for xi, want in zip(xs, eager):
                got = graphed(xi).clone()
                torch.cuda.synchronize()
                assert torch.equal(got, want), "graph replay differs from the eager result"
                assert torch.equal(m(xi), want)  # eager work between replays


def test_qwen3_prefill_shape_with_fp8_weights(gpu_device):
    # 512 rows per expert on average: e4m3 weights go through the throughput kernel.  Same seed as the
    # bf16 case, so the routing is the same; the reference is evaluated on the de-quantised weights.
    wl, m, x, out, disp = _full_size_case("qwen3_30b_a3b_fp8", gpu_device, sample=256)
    assert m.experts.has_fp8_weights
    assert sorted(disp.counts.cpu().tolist(), reverse=True)[:5] == [8138, 7691, 6939, 6074, 5198]
    with torch.no_grad():
        assert torch.equal(m(x), out), "deterministic"


def test_qwen3_decode_fp8_shape(gpu_device):
    # Decode regime with e4m3 weights and per-output-channel scales.  The reference of the comparison
    # is the f32 evaluation with the de-quantised weights, so the bound is the bf16 one; the
    # quantisation error itself (about 2.6 % relative Frobenius norm) is a property of the format.
    wl = W.make_workload("qwen3_decode_fp8")
    _, idx, w = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16)
    m, x, out, gi, gw, disp = _run(wl, gpu_device)
    assert m.experts.has_fp8_weights
    assert_routing_equal(gi, disp, ref.routing)
    assert int((disp.counts > 0).sum()) == 44
    assert_output_close(out, ref.out, "bf16")


def test_module_fp8_quantiser_matches_the_workload_quantiser(gpu_device):
    # Same seed and draw order => same bf16 source weights; one copy is quantised on the CPU by the
    # workload generator, the other on the device by the module.  Scales agree to f32 rounding; a code
    # may differ by one step where w/scale lands on a rounding boundary.
    kw = dict(tokens=64, model_dim=128, num_experts=4, top_k=2, inner_dim=192, dtype="bf16", seed=12)
    m = build_module(W.make_workload_from_spec(W.small_spec(weight_dtype="fp8", **kw)), gpu_device)
    m2 = build_module(W.make_workload_from_spec(W.small_spec(**kw)), gpu_device)
    assert not m2.experts.has_fp8_weights
    m2.experts.quantize_fp8_()
    for name in ("gate", "inner", "output"):
        sa, sb = getattr(m.experts, name + "_scale"), getattr(m2.experts, name + "_scale")
        torch.testing.assert_close(sa, sb, rtol=1e-6, atol=0)
        qa, qb = getattr(m.experts, name + "_q"), getattr(m2.experts, name + "_q")
        assert qa.shape == qb.shape and qa.dtype == torch.float8_e4m3fn
        differ = (qa.view(torch.uint8) != qb.view(torch.uint8)).float().mean().item()
        assert differ < 1e-3, f"{name}: {differ:.2e} of the codes differ"
        assert float((qa.float() - qb.float()).abs().max()) <= 32.0  # at most one e4m3 step (top binade)


@pytest.mark.parametrize("tokens", [96, 3])
def test_graphed_forward_replays_match_eager(gpu_device, tokens):
    """A captured graph of the layer, replayed several times with eager work and synchronisations
    between the replays, gives the eager result bit for bit every time (96 tokens: the GEMM kernels;
    3 tokens: the experts as streams over their weights)."""
    from fairseq2_amd import GraphedForward

    wl = W.make_workload_from_spec(W.small_spec(dtype="bf16", shared=True, seed=11, tokens=tokens))
    m = build_module(wl, gpu_device)
    xs = [wl.x.to(torch.bfloat16).to(gpu_device)]
    g = torch.Generator().manual_seed(5)
    for _ in range(3):
        xs.append(torch.randn(wl.x.shape, generator=g).to(torch.bfloat16).to(gpu_device))
    with torch.no_grad():
        eager = [m(x).clone() for x in xs]
        graphed = GraphedForward(m, xs[0])
        for rep in range(2):
            for x, want in zip(xs, eager):
                got = graphed(x).clone()
                torch.cuda.synchronize()
                assert torch.equal(got, want), "graph replay differs from the eager result"
                again = m(x)  # eager work between replays
                torch.cuda.synchronize()
                assert torch.equal(again, want)
    with pytest.raises(ValueError):
        graphed(xs[0][:, :1])
    # the whole pre-norm feed-forward step, x + layer(rms_norm(x)), as one graph
    norm = _RMSNorm(torch.full((wl.spec.model_dim,), 1.25, dtype=torch.bfloat16, device=gpu_device), 1e-5,
                    wl.spec.model_dim)
    with torch.no_grad():
        eager = [m(x, residual=x, norm=norm).clone() for x in xs]
        graphed = GraphedForward(m, xs[0], add_input=True, norm=norm)
        for rep in range(2):
            for x, want in zip(xs, eager):
                got = graphed(x).clone()
                torch.cuda.synchronize()
                assert torch.equal(got, want), "graph replay of the pre-norm step differs from the eager result"
                m(x)  # eager work between replays



@pytest.mark.parametrize(
    "dtype,weight_dtype,mode,shared,tokens",
    [
        ("bf16", None, W.RoutingMode("sigmoid", False, "input"), True, 300),  # reference mode + shared
        ("bf16", None, W.RoutingMode("softmax", True, "output"), False, 300),  # fused gather
        ("fp32", None, W.RoutingMode("sigmoid", False, "input"), False, 77),
        ("bf16", "fp8", W.RoutingMode("softmax", True, "output"), False, 40),  # e4m3 weights
        # a few tokens: the single call dispatches in the router's second kernel, the module's stages separately
        ("bf16", None, W.RoutingMode("softmax", True, "output"), False, 1),
        ("bf16", None, W.RoutingMode("softmax", False, "output"), True, 4),
        ("bf16", "fp8", W.RoutingMode("softmax", True, "output"), False, 3),
    ],
)
def test_single_call_entry_point_equals_the_module(gpu_device, dtype, weight_dtype, mode, shared, tokens):
    """``fs2moe_forward`` strings the same stages together inside the library: same bits."""
    from fairseq2_amd import _abi
    from fairseq2_amd.moe import _SCORE_FNS

    _say("single call", dtype, weight_dtype, mode, shared, tokens)
    spec = W.small_spec(tokens=tokens, model_dim=128, num_experts=8, top_k=2, inner_dim=192, dtype=dtype,
                        weight_dtype=weight_dtype, zipf_s=1.1, shared=shared, mode=mode, seed=21)
    wl = W.make_workload_from_spec(spec)
    m, x, out, *_ = _run(wl, gpu_device)
    ex = m.experts
    if weight_dtype == "fp8":
        weights = (ex.gate_q, ex.inner_q, ex.output_q)
        scales = (ex.gate_scale, ex.inner_scale, ex.output_scale)
    else:
        weights = (ex.gate_proj.detach(), ex.inner_proj.detach(), ex.output_proj.detach())
        scales = None
    sh = None
    if shared:
        se = m.shared_expert
        sh = (se.gate_proj.weight.detach(), se.inner_proj.weight.detach(), se.output_proj.weight.detach())
    x2 = x.reshape(-1, 128)
    got = _abi.forward(
        x2, m.router.detach(), m.router_bias, *weights, 8, 2, scales=scales, shared=sh, tile_m=16,
        score_fn=_SCORE_FNS[mode.score_fn], renormalize=mode.renormalize, scale_input=mode.scale_on == "input",
        router_t=m.router.detach().t().contiguous(),  # as the module passes it
    )
    torch.cuda.synchronize()
    assert torch.equal(got, out.reshape(-1, 128))


@pytest.mark.parametrize(
    "tokens,e,k,tile_m",
    [
        (33, 8, 2, 16),       # two tiles, the second with one token
        (300, 8, 2, 16),
        (1000, 24, 1, 16),    # groups of 8 experts that do not divide the block's threads
        (2500, 64, 8, 1),     # no padding rows at all
        (4100, 256, 32, 8),   # the two-fragment router, 1024 pairs per tile
        (16384, 16, 4, 16),   # the most tiles the tile form takes
        (16385, 16, 4, 16),   # one more: the counting kernel's form again
    ],
)
def test_single_call_dispatches_like_the_dispatch_call(gpu_device, tokens, e, k, tile_m):
    """Inside ``fs2moe_forward`` the router of an (E, D) matrix counts and ranks its own tiles of 32
    tokens and one more kernel finishes the dispatch: the selection, the counts, the offsets and
    both permutations, read back from the head of the workspace, against ``fs2moe_router_topk`` +
    ``fs2moe_dispatch``, integer for integer; and the layer's output against the stages'."""
    _say("single call dispatch", tokens, e, k, tile_m)
    d, f = 128, 64
    g = torch.Generator().manual_seed(tokens + e)
    x = torch.randn(tokens, d, generator=g).bfloat16().to(gpu_device)
    router = (torch.randn(d, e, generator=g) * 0.3).bfloat16().to(gpu_device)
    # a few experts that nobody chooses, and ties between neighbours
    bias = torch.zeros(e)
    bias[e // 2:: 5] = -30.0
    bias = bias.to(gpu_device)
    router[:, 1] = router[:, 0]
    wg = (torch.randn(e * d, f, generator=g) * 0.1).bfloat16().to(gpu_device)
    wu = (torch.randn(e * d, f, generator=g) * 0.1).bfloat16().to(gpu_device)
    wd = (torch.randn(e * f, d, generator=g) * 0.1).bfloat16().to(gpu_device)
    rt = router.t().contiguous()
    lib = _abi.load()
    assert lib.fs2moe_router_takes_out_in(tokens, d, e, _abi.BF16) == 1
    ws = torch.zeros(lib.fs2moe_forward_workspace_bytes(tokens, d, e, k, f, 0, tile_m, _abi.BF16),
                     dtype=torch.uint8, device=gpu_device)
    out = _abi.forward(x, router, bias, wg, wu, wd, e, k, tile_m=tile_m, score_fn=_abi.SCORE_SOFTMAX,
                       renormalize=True, scale_input=False, workspace=ws, router_t=rt)
    idx, w, _ = _abi.router_topk(x, router, bias, k, _abi.SCORE_SOFTMAX, True, router_t=rt)
    dsp = _abi.dispatch(idx, w, x, e, tile_m, False, gather=False)
    torch.cuda.synchronize()
    # the head of the workspace: T x K indices, T x K weights, E counts, E + 1 offsets, max_rows of
    # perm, T x K of inv_perm, each from the next multiple of 256 bytes on
    rows = _abi.max_rows(tokens, k, e, tile_m)
    at = 0
    parts = []
    for n in (tokens * k, tokens * k, e, e + 1, rows, tokens * k):
        parts.append(ws[at: at + 4 * n].view(torch.int32))
        at += (4 * n + 255) // 256 * 256
    assert torch.equal(parts[0].view(tokens, k), idx), "the selection (which also places the parts)"
    assert torch.equal(parts[1].view(torch.float32).view(tokens, k), w)
    assert torch.equal(parts[2], dsp.counts) and int(dsp.counts.sum()) == tokens * k
    assert int((dsp.counts == 0).sum()) > 0 or e == 8
    assert torch.equal(parts[3], dsp.offsets)
    assert torch.equal(parts[5].view(tokens, k), dsp.inv_perm)
    assert torch.equal(parts[4], dsp.perm)
    ye, _ = _abi.grouped_swiglu(x, dsp.counts, dsp.offsets, wg, wu, wd, e, row_map=dsp.perm)
    assert torch.equal(out, _abi.combine(ye, dsp.inv_perm, idx, w, None, True))


def test_expert_major_copy_of_the_router_follows_the_parameter(gpu_device):
    """The derived (E, D) copy the bf16 router reads: made once, made again after an in-place update,
    after a move and for another tensor (also one that reuses a freed tensor's address), and kept
    with its owner, not under an address."""
    from fairseq2_amd import _abi

    _say("router copy")
    spec = W.small_spec(tokens=100, model_dim=128, num_experts=8, top_k=2, inner_dim=64, dtype="bf16", seed=3)
    m = build_module(W.make_workload_from_spec(spec), gpu_device)
    first = m._router_expert_major()
    assert first.shape == (8, 128) and torch.equal(first, m.router.detach().t())
    assert m._router_expert_major() is first, "kept between calls"
    x = torch.randn(100, 128, generator=torch.Generator().manual_seed(1)).bfloat16().to(gpu_device)
    with torch.no_grad():
        before = m(x)
        m.router.mul_(-1.0)  # an optimizer step's kind of update
        second = m._router_expert_major()
        assert second is not first and torch.equal(second, m.router.detach().t())
        after = m(x)
        idx_now = _abi.router_topk(x, m.router.detach(), m.router_bias, 2, router_t=second)[0]
        idx_plain = _abi.router_topk(x, m.router.detach(), m.router_bias, 2)[0]
    assert torch.equal(idx_now, idx_plain) and not torch.equal(before, after)
    # tensors that come and go at one address: each gets its own copy
    seen = set()
    for i in range(4):
        r = torch.full((128, 8), float(i), dtype=torch.bfloat16, device=gpu_device)
        seen.add(r.data_ptr())
        assert float(_abi.router_expert_major(r)[0, 0]) == float(i)
        del r
    assert _abi.router_expert_major(torch.zeros(4, 4, device=gpu_device)) is None, "f32: no copy"
    with torch.inference_mode():
        made_here = torch.zeros(128, 8, dtype=torch.bfloat16, device=gpu_device)
        assert _abi.router_expert_major(made_here) is None, "no version counter to watch: no copy"
        assert torch.equal(m(x), after), "a module made outside runs inside inference mode as before"


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("shared", [False, True])
def test_residual_is_added_in_the_same_accumulation(gpu_device, dtype, shared):
    """``module(x, residual=r)`` against ``r + layer(x)`` of the oracle, through both the single-call
    and the staged path."""
    _say("residual", dtype, shared)
    spec = W.small_spec(tokens=200, model_dim=128, num_experts=8, top_k=2, inner_dim=192, dtype=dtype,
                        shared=shared, seed=31)
    wl = W.make_workload_from_spec(spec)
    _, idx, _ = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    g = torch.Generator().manual_seed(5)
    res = torch.randn(wl.x.shape, generator=g).to(TORCH_DTYPE[dtype])
    m, x, out, *_ = _run(wl, gpu_device)
    res_d = res.to(gpu_device)
    with torch.no_grad():
        got = m(x, residual=res_d)
        staged = m._stages(x.reshape(-1, 128), res_d.reshape(-1, 128))[0].view(x.shape)
    assert torch.equal(got, staged)
    assert torch.equal(res_d, res.to(gpu_device)), "the residual is left untouched"
    assert_output_close(got, ref.out + res.double(), dtype, "residual + layer")
    # the separate addition rounds the layer output and then the sum, the fused one only the sum:
    # they differ by at most those roundings
    eps = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -23
    two_step = out.double() + res_d.double()
    bound = eps * (out.double().abs() + two_step.abs() + got.double().abs())
    assert bool(((got.double() - two_step).abs() <= bound).all())


class _RMSNorm:
    """The attributes of fairseq2.nn.RMSNorm the module reads (nn/normalization.py:166-232)."""

    def __init__(self, weight, eps, dim):
        self.weight, self.bias, self.eps, self.normalized_shape = weight, None, eps, (dim,)


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize(
    "mode,shared,weights",
    [
        (W.RoutingMode("sigmoid", False, "input"), True, None),   # reference mode: rows are copied
        (W.RoutingMode("softmax", True, "output"), False, None),  # rows read through the permutation
        (W.RoutingMode("softmax", True, "output"), False, "fp8"),
        (W.RoutingMode("softmax", True, "output"), False, "prefill"),  # above 4096 tokens
        # up to 32 bf16 tokens: the router's second kernel also dispatches
        (W.RoutingMode("softmax", True, "output"), False, "tokens=1"),
        (W.RoutingMode("softmax", True, "output"), True, "tokens=3"),
        (W.RoutingMode("sigmoid", True, "output"), False, "tokens=4"),
        (W.RoutingMode("sigmoid", False, "input"), False, "tokens=2"),  # rows scaled by the expert kernels
        # decode steps with a shared expert
        (W.RoutingMode("sigmoid", False, "input"), True, "tokens=5"),
        (W.RoutingMode("softmax", True, "output"), True, "tokens=16"),
    ],
)
def test_pre_norm_and_residual_in_one_call(gpu_device, dtype, mode, shared, weights):
    """``module(x, residual=x, norm=n)`` is the feed-forward step of a pre-norm decoder layer
    (decoder_layer.py:187-204): x + layer(rms_norm(x)).  Checked against the module run on the
    normalised rows (bit for bit: same kernels behind the normalisation) and against the oracle
    evaluated on those rows."""
    if weights == "fp8" and dtype == "fp32":
        pytest.skip("e4m3 weights go with bf16 activations")
    _say("pre-norm", dtype, mode, shared, weights)
    # up to 4096 tokens the rows are normalised by a small kernel in front of the router (300, 1300);
    # above that inside the router kernel (4200)
    tokens = 1300 if shared else 300
    if weights == "prefill":
        tokens, weights = 4200, None
    elif weights is not None and weights.startswith("tokens="):
        tokens, weights = int(weights[7:]), None
    spec = W.small_spec(tokens=tokens, model_dim=128, num_experts=8, top_k=2, inner_dim=192, dtype=dtype,
                        weight_dtype=weights, shared=shared, mode=mode, seed=41)
    wl = W.make_workload_from_spec(spec)
    td = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(8)
    raw = (2.5 * torch.randn(wl.x.shape, generator=g)).to(td)
    gamma = (1.0 + 0.2 * torch.randn(128, generator=g)).to(td)
    m = build_module(wl, gpu_device, 16)
    norm = _RMSNorm(gamma.to(gpu_device), 1e-5, 128)
    raw_d = raw.to(gpu_device)
    with torch.no_grad():
        got = m(raw_d, residual=raw_d, norm=norm)
        xn = _abi.router_topk_norm(raw_d.reshape(-1, 128), norm.weight, norm.eps, m.router.detach(),
                                   m.router_bias, m.top_k)[0].view(raw.shape)
        two_calls = m(xn, residual=raw_d)
        staged = m._stages(raw_d.reshape(-1, 128), raw_d.reshape(-1, 128), (norm.weight, norm.eps))[0]
    torch.cuda.synchronize()
    assert torch.equal(got, two_calls)
    assert torch.equal(got, staged.view(raw.shape))
    assert torch.equal(raw_d, raw.to(gpu_device)), "the input is left untouched"
    # the oracle on the rows the device normalised (checked against the oracle's norm in the
    # router test), plus the residual
    step = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -20
    want_xn = O.rms_norm(raw, gamma, 1e-5).double()
    assert bool(((xn.cpu().double() - want_xn).abs() <= step * want_xn.abs()).all())
    wl.x = xn.cpu().float()
    _, idx, _ = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64)
    assert_output_close(got, ref.out + raw.double(), dtype, "x + layer(norm(x))")


def test_pre_norm_in_place(gpu_device):
    """With the normalisation in front, the raw rows are read by the router only, so the result
    may be written over them: fs2moe_forward_norm with out == x == residual."""
    _say("pre-norm in place")
    spec = W.small_spec(tokens=100, model_dim=128, num_experts=8, top_k=2, inner_dim=64, dtype="bf16",
                        mode=W.RoutingMode("softmax", True, "output"), seed=43)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device, 16)
    x = wl.x.to(torch.bfloat16).to(gpu_device).reshape(-1, 128)
    gamma = torch.ones(128, dtype=torch.bfloat16, device=gpu_device)
    with torch.no_grad():
        want = m(x, residual=x, norm=_RMSNorm(gamma, 1e-6, 128))
    lib = _abi.load()
    t, d = x.shape
    ex = m.experts
    sizes = (t, d, 8, 2, 64, 0, 16, _abi.BF16)
    ws = torch.empty(lib.fs2moe_forward_norm_workspace_bytes(*sizes), dtype=torch.uint8, device=gpu_device)
    assert ws.numel() > lib.fs2moe_forward_workspace_bytes(*sizes)
    buf = x.clone()
    p = lambda t_: None if t_ is None else t_.data_ptr()  # noqa: E731
    rc = lib.fs2moe_forward_norm(
        p(buf), p(gamma), 1e-6, p(buf), p(m.router), p(m.router_bias), p(ex.gate_proj), p(ex.inner_proj),
        p(ex.output_proj), None, None, None, None, None, None, t, d, 8, 2, 64, 0, 16, _abi.BF16,
        _abi.BF16, _abi.SCORE_SOFTMAX, 1, 0, p(ws), ws.numel(), p(buf),
        torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.fs2moe_last_error()
    torch.cuda.synchronize()
    assert torch.equal(buf, want)


@pytest.mark.parametrize("case", ["plain", "residual+norm", "fp8", "shared"])
def test_module_under_torch_compile(gpu_device, case):
    """fairseq2 may wrap its layers in torch.compile (transformer_lm/compiler.py:14-17).  Traced,
    the module calls the library through torch.ops.fairseq2_amd.moe_forward: one graph, no break,
    the same bits as the eager call.  (Backend aot_eager: tracing and the operator's shape-only
    implementation are what is exercised; no code generator is involved.)"""
    _say("torch.compile", case)
    spec = W.small_spec(tokens=96, model_dim=128, num_experts=8, top_k=2, inner_dim=64, dtype="bf16",
                        weight_dtype="fp8" if case == "fp8" else None, shared=case == "shared",
                        mode=W.RoutingMode("softmax", True, "output"), seed=51)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device, 16)
    x = wl.x.to(torch.bfloat16).to(gpu_device)
    norm = _RMSNorm(torch.ones(128, dtype=torch.bfloat16, device=gpu_device), 1e-5, 128)
    if case == "residual+norm":
        fn = lambda t: m(t, residual=t, norm=norm)  # noqa: E731
    else:
        fn = lambda t: m(t)  # noqa: E731
    with torch.no_grad():
        want = fn(x)
        compiled = torch.compile(fn, backend="aot_eager", fullgraph=True)
        got = compiled(x)
        again = compiled(x)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(again, want)


# --------------------------------------------------------------------------- interface rows
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_grouped_expert_network_in_the_reference_calling_convention(gpu_device, dtype):
    """``GroupedExpertNetwork.forward((E, n, D))`` is how the reference calls its experts
    (experts.py:201-213): every expert gets the same number of rows.  Each expert against the oracle's
    textbook SwiGLU in f64; the call launches nothing but the expert kernels, so it records into a HIP
    graph, and the replays give the eager bits."""
    from fairseq2_amd.moe import GroupedExpertNetwork

    _say("GroupedExpertNetwork.forward", dtype)
    e, n, d, f = 6, 37, 128, 192
    td = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(17)
    net = GroupedExpertNetwork(e, d, f, device=gpu_device, dtype=td).requires_grad_(False)
    wg = (0.05 * torch.randn(e * d, f, generator=g)).to(td)
    wu = (0.05 * torch.randn(e * d, f, generator=g)).to(td)
    wd = (0.05 * torch.randn(e * f, d, generator=g)).to(td)
    net.load_state_dict({"gate_proj": wg, "inner_proj": wu, "output_proj": wd})
    x = torch.randn(e, n, d, generator=g).to(td)
    xd = x.to(gpu_device)
    with torch.no_grad():
        y = net(xd)
        y2 = net(xd)
    torch.cuda.synchronize()
    assert y.shape == (e, n, d) and y.dtype == td and torch.equal(y, y2)
    for ex in range(e):
        want = O.glu_expert(x[ex].double(), wg.double().view(e, d, f)[ex], wu.double().view(e, d, f)[ex],
                            wd.double().view(e, f, d)[ex])
        assert_output_close(y[ex], want, dtype, f"expert {ex}")
    with pytest.raises(ValueError):
        net(xd[:, :, : d // 2])
    # graph-clean: counts and offsets are built once, the call is kernels only
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.no_grad():
        net(xd)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph), torch.no_grad():
        yg = net(xd)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(yg, y)
        with torch.no_grad():
            net(xd)  # eager work between replays


@pytest.mark.parametrize("fp8", [False, True])
def test_llama4_checkpoint_names_load_and_run(gpu_device, fp8):
    """A Meta-format Llama-4 state dict (llama4/interop.py:126-136) goes through
    ``load_llama4_moe_layer`` into the module on the GPU, optionally packed to e4m3, and the forward
    pass is the oracle's on the same tensors (on the de-quantised ones with fp8)."""
    from fairseq2_amd import MoE
    from fairseq2_amd.checkpoint import load_llama4_moe_layer

    _say("llama4 checkpoint", fp8)
    d, e, f, t = 128, 8, 192, 200
    g = torch.Generator().manual_seed(23)
    r = lambda *s: (0.05 * torch.randn(*s, generator=g)).to(torch.bfloat16)  # noqa: E731
    p = "layers.2.feed_forward."
    sd = {
        "tok_embeddings.weight": r(10, d),
        p + "router_DE": (4.0 * r(d, e)),
        p + "experts.moe_w_in_eD_F": r(e * d, f),
        p + "experts.moe_w_swiglu_eD_F": r(e * d, f),
        p + "experts.moe_w_out_eF_D": r(e * f, d),
        p + "w_in_shared_FD.weight": r(f, d),
        p + "w_swiglu_FD.weight": r(f, d),
        p + "w_out_shared_DF.weight": r(d, f),
        p + "running_gate_stats_3E": r(3, e),
        p + "experts._extra_state": r(1),
    }
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        m = MoE(d, f, True, e, 1.0, 1, inner_dim_scale=1.0, auto_scale=False)
    finally:
        torch.set_default_dtype(prev)
    m = m.to(gpu_device).requires_grad_(False)
    load_llama4_moe_layer(m, sd, 2, fp8=fp8)
    assert m.experts.has_fp8_weights == fp8
    x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
    with torch.no_grad():
        out, gi, gw, disp = m.forward_with_routing(x.to(gpu_device))
        again = m(x.to(gpu_device))
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    gate, up, down = (sd[p + n].float() for n in ("experts.moe_w_in_eD_F", "experts.moe_w_swiglu_eD_F",
                                                  "experts.moe_w_out_eF_D"))
    if fp8:
        # the codes the module holds (quantised on the device: where w / scale lands on a rounding
        # boundary torch's device cast may pick the other neighbour than the CPU's, and both are
        # valid e4m3 images of the weight), de-quantised
        ex = m.experts
        gate, up, down = (
            W.dequantize_fp8_per_channel(_abi.unpack_fp8_weights(q, e).cpu(), s.cpu())
            for q, s in ((ex.gate_q, ex.gate_scale), (ex.inner_q, ex.inner_scale), (ex.output_q, ex.output_scale))
        )
        for deq_w, name in ((gate, "experts.moe_w_in_eD_F"), (down, "experts.moe_w_out_eF_D")):
            # ... and they ARE images of the checkpoint's weights: within one e4m3 step (2^-3 relative,
            # 2^-9 * 448 * scale below the normal range), most within half of one
            rel = (deq_w - sd[p + name].float()).abs() / sd[p + name].float().abs().clamp_min(1e-3)
            assert float(rel.max()) <= 0.126 and float(rel.mean()) < 0.03
    shared = tuple(sd[p + n].double() for n in ("w_in_shared_FD.weight", "w_swiglu_FD.weight", "w_out_shared_DF.weight"))
    logits = O.router_logits(x.reshape(-1, d).double(), sd[p + "router_DE"].double(), None)
    idx = O.topk_lowest_index(logits, 1)
    ref = O.ref_sparse_forward(x.double(), sd[p + "router_DE"].double(), gate.double(), up.double(), down.double(), 1,
                               shared=shared, tile_m=m.tile_m, topk_idx=idx)
    assert_routing_equal(gi, disp, ref.routing, "llama4 checkpoint")
    assert_output_close(out, ref.out, "bf16", "llama4 checkpoint")
    # loading plain weights afterwards drops the derived e4m3 buffers
    if fp8:
        load_llama4_moe_layer(m, sd, 2, fp8=False)
        assert not m.experts.has_fp8_weights


def test_scout_constructor_arguments_of_the_reference_factory(gpu_device):
    """The module as the Llama-4 factory constructs it for Scout (llama4/factory.py:123-135:
    inner dim 4 * 5120 * 1.2 = 24576, scale 2/3, auto-scaled by capacity + shared, rounded up to a
    multiple of 2048) has the 8192-wide experts of the workload, and computes the same as the module
    built with the inner dim given outright."""
    from fairseq2_amd import MoE

    _say("scout ctor")
    wl = W.make_workload("llama4_scout")
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        m = MoE(5120, 24576, True, 16, 1.0, 1, inner_dim_to_multiple=2048)
    finally:
        torch.set_default_dtype(prev)
    assert m.experts.inner_dim == 8192 and m.shared_expert.gate_proj.weight.shape == (8192, 5120)
    direct = build_module(wl, gpu_device)
    m.load_state_dict(direct.state_dict(), strict=True)
    m = m.to(gpu_device).requires_grad_(False).eval()
    x = wl.x.to(torch.bfloat16).to(gpu_device)[:, :512]
    with torch.no_grad():
        assert torch.equal(m(x), direct(x))


def test_autocast_is_honoured(gpu_device):
    """Under torch.autocast (trainer.py:650-656) an f32 input is cast to the autocast dtype when the
    module holds its parameters in it; the result comes back in that dtype and equals the call on
    the cast input.  Parameters of another dtype are not cast silently."""
    _say("autocast")
    wl = W.make_workload_from_spec(W.small_spec(tokens=64, model_dim=128, num_experts=8, top_k=2, inner_dim=64,
                                                dtype="bf16", seed=3))
    m = build_module(wl, gpu_device)
    x32 = wl.x.float().to(gpu_device)
    with torch.no_grad():
        want = m(x32.to(torch.bfloat16))
        with torch.autocast("cuda", dtype=torch.bfloat16):
            got = m(x32)
            got_res = m(x32, residual=x32)
        assert got.dtype == torch.bfloat16 and torch.equal(got, want)
        assert torch.equal(got_res, m(x32.to(torch.bfloat16), residual=x32.to(torch.bfloat16)))
        with pytest.raises(TypeError, match="parameters"):
            m(x32)  # no autocast: dtype mismatch is an error
        wl32 = W.make_workload_from_spec(W.small_spec(tokens=64, model_dim=128, num_experts=8, top_k=2,
                                                      inner_dim=64, dtype="fp32", seed=3))
        m32 = build_module(wl32, gpu_device)
        with torch.autocast("cuda", dtype=torch.bfloat16), pytest.raises(TypeError, match="autocast"):
            m32(x32.to(torch.bfloat16))


def test_reference_arithmetic_in_bf16(gpu_device):
    """The reference run in bf16 rounds the logits to bf16 before torch.topk and the sigmoid, keeps the
    scores in bf16 and accumulates scatter_add_ in bf16 (moe.py:109-150 on bf16 tensors).  The device
    keeps f32 logits and weights and rounds the output once: a deliberate refinement.  Its selection
    must still be a valid top-k of the bf16-rounded logits (it resolves their ties by the f32 values),
    and its output must agree with the reference's own bf16 result within the bf16 bound."""
    _say("reference arithmetic in bf16")
    spec = W.small_spec(tokens=200, model_dim=128, num_experts=8, top_k=2, inner_dim=96, dtype="bf16", seed=77)
    wl = W.make_workload_from_spec(spec)
    m, x, out, gi, gw, disp = _run(wl, gpu_device)
    b = lambda t_: t_.to(torch.bfloat16)  # noqa: E731
    logits_bf16 = (b(wl.x).reshape(-1, 128) @ b(wl.router)).float()
    chosen = torch.gather(logits_bf16, 1, gi.cpu().long())
    rest = logits_bf16.scatter(1, gi.cpu().long(), float("-inf")).max(dim=1).values
    assert bool((chosen.min(dim=1).values >= rest).all()), "not a top-k of the bf16-rounded logits"
    assert bool((chosen[:, :-1] >= chosen[:, 1:]).all())
    dense_bf16 = O.ref_dense_forward(b(wl.x), b(wl.router), b(wl.gate), b(wl.up), b(wl.down), 2)
    # where both selections agree (every token here unless a bf16 tie was resolved the other way)
    ref_idx = torch.topk(b(wl.x).reshape(-1, 128) @ b(wl.router), 2, dim=1).indices
    same = (torch.sort(ref_idx, dim=1).values == torch.sort(gi.cpu().long(), dim=1).values).all(dim=1)
    assert float(same.float().mean()) > 0.9
    got = out.reshape(-1, 128).cpu()[same]
    # both sides carry bf16 rounding here, and the reference's side more of it (scores rounded to
    # bf16 scale whole rows, scatter_add_ rounds after every addition): twice the element-wise room
    assert_output_close(got, dense_bf16.reshape(-1, 128)[same].double(), "bf16", "vs the reference in bf16",
                        atol_scale=2.0)


def test_layer_arguments_are_validated_before_the_gpu_reads_them(gpu_device):
    """fs2moe_forward takes raw pointers: the binding refuses tensors whose shape, dtype or device
    does not match the sizes, instead of letting a kernel read out of bounds."""
    _say("argument validation")
    wl = W.make_workload_from_spec(W.small_spec(tokens=32, model_dim=128, num_experts=8, top_k=2, inner_dim=64,
                                                dtype="bf16", seed=5))
    m = build_module(wl, gpu_device)
    ex = m.experts
    x = wl.x.to(torch.bfloat16).to(gpu_device).reshape(-1, 128)
    w = (ex.gate_proj.detach(), ex.inner_proj.detach(), ex.output_proj.detach())
    good = _abi.forward(x, m.router.detach(), None, *w, 8, 2)
    assert good.shape == x.shape
    with pytest.raises(ValueError, match="router"):
        _abi.forward(x, m.router.detach()[:, :4].contiguous(), None, *w, 8, 2)
    with pytest.raises(ValueError, match="router"):
        _abi.forward(x, m.router.detach().float(), None, *w, 8, 2)
    with pytest.raises(ValueError, match="gate weights"):
        _abi.forward(x, m.router.detach(), None, w[0][:-8].contiguous(), w[1], w[2], 8, 2)
    with pytest.raises(ValueError, match="up weights"):
        _abi.forward(x, m.router.detach(), None, w[0], w[1].cpu(), w[2], 8, 2)
    with pytest.raises(ValueError, match="router_bias"):
        _abi.forward(x, m.router.detach(), torch.zeros(8, dtype=torch.bfloat16, device=gpu_device), *w, 8, 2)
    with pytest.raises(ValueError, match="shared"):
        _abi.forward(x, m.router.detach(), None, *w, 8, 2, shared=(w[0], w[0], w[0]))
    # an fp8 module whose buffers were cast by .to(dtype) keeps its codes (they are integer buffers)
    ex.quantize_fp8_()
    m.to(torch.bfloat16)
    assert ex.gate_q.dtype == torch.float8_e4m3fn and ex.gate_scale.dtype == torch.float32
    with torch.no_grad():
        m(x)

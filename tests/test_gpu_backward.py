"""Backward pass on the GPU against ``torch.autograd`` through the CPU oracle in float64.

The oracle's dense formulation follows the reference layer operator for operator (``moe.py:102-157``),
so differentiating it with autograd gives what the reference's trainer gets (``trainer.py:586-587``).
Stage tests check each backward entry point on its own; the layer tests check every gradient of the
module (input, residual, router, expert weights, shared-expert weights) in all routing modes.

Tolerances: gradients are sums of products like the outputs, with one more rounding per intermediate
(dye, dh, dg/du, dxe are each stored in the activation dtype), so the bf16 bounds are those of the
forward output widened by sqrt(2): element-wise 3e-2 relative + 6e-2 of the tensor's rms, 1.5e-2 of
the rms overall; fp32 2e-4 / 2e-4 / 5e-5.  The rms is taken over the entries that are not exactly zero
in the reference (experts without tokens have zero weight gradients).
"""

import pytest
import torch

from fairseq2_amd import _abi
import workloads as W
from oracle import moe_oracle as O
from tests._util import TORCH_DTYPE, assert_output_close, build_module

pytestmark = pytest.mark.gpu

GRAD_TOL = {"bf16": (3e-2, 6e-2, 1.5e-2), "fp32": (2e-4, 2e-4, 5e-5)}


def _say(*a):
    print(*a, flush=True)


# Entries of a float64 reference gradient below this are rounding noise around an exact zero (for
# example every router gradient with one selected expert and renormalised weights: w = s / s = 1
# whatever the logits), not values to scale a tolerance by.
STRUCTURAL_ZERO = 1e-12


def assert_grad_close(got, ref, dtype, what, blocks=1, rms_slack=1.0):
    """``blocks``: the leading dimension is split into that many equal blocks, each compared on its
    own scale.  The experts of a layer see inputs of very different size (a softmax weight of 0.5 or
    of 0.01 in front of the gate), so their weight gradients differ by orders of magnitude, and an
    element that is a cancelling sum over an expert's two or three rows carries the rounding error
    of its terms, which scale with THAT expert's gradient, not with the rms over all experts.
    ``rms_slack`` widens the overall statement where nothing averages (a single token)."""
    got = got.detach().double().cpu().reshape(ref.shape)
    ref = ref.double()
    rtol, atol_rel, rms_tol = GRAD_TOL[dtype]
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    if blocks > 1:
        got, ref = got.reshape(blocks, -1), ref.reshape(blocks, -1)
    else:
        got, ref = got.reshape(1, -1), ref.reshape(1, -1)
    # the scale of the entries that are not structurally zero (an expert without tokens has a zero
    # weight gradient; such entries would otherwise deflate the scale of the others)
    nz = ref.abs() > STRUCTURAL_ZERO
    n_nz = nz.sum(1).clamp(min=1)
    rms = ((ref * nz).pow(2).sum(1) / n_nz).sqrt()  # per block
    err = (got - ref).abs()
    live = rms > 0
    bound = atol_rel * rms[:, None] + rtol * ref.abs()
    worst = float((err[live] / bound[live]).max()) if bool(live.any()) else 0.0
    err_rms = ((err * nz).pow(2).sum(1) / n_nz).sqrt()
    rel_rms = float((err_rms[live] / rms[live]).max()) if bool(live.any()) else 0.0
    # where the reference is zero the result is too, to the last rounding of what flows into it
    zero_err = float(err[~nz].max()) if bool((~nz).any()) else 0.0
    scale = float(rms.max())
    print(f"  {what}: worst err/bound {worst:.3f}, rms err / rms {rel_rms:.2e}, at zeros {zero_err:.1e}", flush=True)
    assert zero_err <= (atol_rel * scale if scale > 0 else 1e-6), (
        f"{what}: {zero_err:.3e} where the reference is zero (scale {scale:.3e})")
    assert worst <= 1.0, f"{what}: max err/bound {worst:.3f} (rms {scale:.3e})"
    assert rel_rms <= rms_tol * rms_slack, f"{what}: rms error {rel_rms:.3e} of the rms, above {rms_tol * rms_slack}"


def assert_layer_grads_close(module, x_grad, ref, dtype, tokens):
    """Every gradient of the layer against the reference's.  Expert weights are compared expert by
    expert (see assert_grad_close).  With fewer than 8 tokens nothing averages in the router's
    gradient (one token: an outer product of its row with a difference of K rounded dot products),
    so the overall statement gets twice the room there."""
    assert_grad_close(x_grad, ref["x"], dtype, "d x")
    e = module.experts.num_local_experts
    for name, p in module.named_parameters():
        assert p.grad is not None and p.grad.dtype == p.dtype and p.grad.shape == p.shape, name
        assert_grad_close(p.grad, ref[name], dtype, f"d {name}",
                          blocks=e if name.startswith("experts.") else 1,
                          rms_slack=2.0 if name == "router" and tokens < 8 else 1.0)


# ------------------------------------------------------------------------------------- stage tests
def _groups(rows_per_expert, pad=16):
    counts = torch.tensor(rows_per_expert, dtype=torch.int32)
    padded = (counts + pad - 1) // pad * pad
    offsets = torch.zeros(len(rows_per_expert) + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(padded, 0)
    return counts, offsets


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("layout", ["in_out", "out_in"])
@pytest.mark.parametrize("rows,k,n", [([5, 0, 300, 64, 1], 64, 96), ([130, 257], 128, 64), ([40, 3, 0, 77], 72, 40)])
def test_grouped_gemm_both_orientations(gpu_device, dtype, layout, rows, k, n):
    _say("grouped_gemm", dtype, layout, rows, k, n)
    dt = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(k + n)
    e = len(rows)
    counts, offsets = _groups(rows)
    total = int(offsets[-1])
    a = torch.randn(total, k, generator=g).to(dt)
    b = (0.1 * torch.randn(e, k, n, generator=g)).to(dt)
    stored = b.reshape(e * k, n) if layout == "in_out" else b.transpose(1, 2).contiguous().reshape(e * n, k)
    dev = gpu_device
    c = _abi.grouped_gemm(a.to(dev), stored.to(dev), _abi.W_IN_OUT if layout == "in_out" else _abi.W_OUT_IN,
                          counts.to(dev), offsets.to(dev), e)
    for ex in range(e):
        lo, cnt = int(offsets[ex]), int(counts[ex])
        if cnt:
            ref = a[lo : lo + cnt].double() @ b[ex].double()
            assert_grad_close(c[lo : lo + cnt], ref, dtype, f"expert {ex}")
    # one matrix, all rows
    d = _abi.grouped_gemm(a.to(dev), stored[: (k if layout == "in_out" else n)].contiguous().to(dev),
                          _abi.W_IN_OUT if layout == "in_out" else _abi.W_OUT_IN)
    assert_grad_close(d, a.double() @ b[0].double(), dtype, "dense")


@pytest.mark.parametrize("rows,k,n", [([5, 0, 300, 64, 1, 700], 192, 128), ([130, 257], 64, 72), ([0, 0, 9], 128, 256)])
def test_grouped_gemm_sum_adds_two_products(gpu_device, rows, k, n):
    """``a1 @ B1^T + a2 @ B2^T`` in one kernel against f64, and against the two products apart."""
    _say("grouped_gemm_sum", rows, k, n)
    dev = gpu_device
    g = torch.Generator().manual_seed(k * n)
    e = len(rows)
    counts, offsets = _groups(rows)
    total = int(offsets[-1])
    assert _abi.grouped_gemm_sum_supported(k, n, total, torch.bfloat16)
    assert not _abi.grouped_gemm_sum_supported(k, n, total, torch.float32)
    assert not _abi.grouped_gemm_sum_supported(k + 8, n, total, torch.bfloat16)
    a1, a2 = (torch.randn(total, k, generator=g).to(torch.bfloat16) for _ in range(2))
    b1, b2 = ((0.1 * torch.randn(e, n, k, generator=g)).to(torch.bfloat16) for _ in range(2))
    c, o = counts.to(dev), offsets.to(dev)
    out = _abi.grouped_gemm_sum(a1.to(dev), b1.reshape(e * n, k).to(dev), a2.to(dev), b2.reshape(e * n, k).to(dev), c, o, e)
    for ex in range(e):
        lo, cnt = int(offsets[ex]), int(counts[ex])
        if cnt:
            ref = a1[lo : lo + cnt].double() @ b1[ex].double().t() + a2[lo : lo + cnt].double() @ b2[ex].double().t()
            assert_grad_close(out[lo : lo + cnt], ref, "bf16", f"expert {ex}")
    # one matrix each, all rows
    dense = _abi.grouped_gemm_sum(a1.to(dev), b1[0].contiguous().to(dev), a2.to(dev), b2[0].contiguous().to(dev))
    assert_grad_close(dense, a1.double() @ b1[0].double().t() + a2.double() @ b2[0].double().t(), "bf16", "dense")


@pytest.mark.parametrize("rows,d,f", [([5, 0, 300, 64, 1, 700], 128, 192), ([130, 257], 64, 64), ([0, 0, 9], 256, 128)])
def test_grouped_swiglu_keep_leaves_the_two_products(gpu_device, rows, d, f):
    """The training-forward variant of the expert kernel: same ``ye`` and ``h`` as the inference
    one, bit for bit, plus the gate and the up product as two separate GEMMs give them."""
    _say("grouped_swiglu_keep", rows, d, f)
    dev = gpu_device
    g = torch.Generator().manual_seed(d + f)
    e = len(rows)
    counts, offsets = _groups(rows)
    total = int(offsets[-1])
    assert _abi.keeps_products(d, f, total, torch.bfloat16)
    assert not _abi.keeps_products(d, f, total, torch.float32)
    assert not _abi.keeps_products(d + 8, f, total, torch.bfloat16)
    x = torch.randn(total, d, generator=g).to(torch.bfloat16).to(dev)
    wg, wu = ((0.2 * torch.randn(e * d, f, generator=g)).to(torch.bfloat16).to(dev) for _ in range(2))
    wd = (0.2 * torch.randn(e * f, d, generator=g)).to(torch.bfloat16).to(dev)
    c, o = counts.to(dev), offsets.to(dev)
    ye0, h0 = _abi.grouped_swiglu(x, c, o, wg, wu, wd, e)
    ye, h, gate, up = _abi.grouped_swiglu_keep(x, c, o, wg, wu, wd, e)
    gate_ref = _abi.grouped_gemm(x, wg, _abi.W_IN_OUT, c, o, e)
    up_ref = _abi.grouped_gemm(x, wu, _abi.W_IN_OUT, c, o, e)
    for ex in range(e):
        lo, cnt = int(offsets[ex]), int(counts[ex])
        sl = slice(lo, lo + cnt)
        assert torch.equal(ye[sl], ye0[sl]) and torch.equal(h[sl], h0[sl]), f"expert {ex}: ye / h differ"
        assert torch.equal(gate[sl], gate_ref[sl]), f"expert {ex}: gate product"
        assert torch.equal(up[sl], up_ref[sl]), f"expert {ex}: up product"
        if cnt:
            ref = x[sl].double().cpu() @ wg.double().cpu().reshape(e, d, f)[ex]
            assert_grad_close(gate[sl], ref, "bf16", f"expert {ex} gate product")
    # through a row map
    perm = torch.randperm(total, generator=g).to(torch.int32)
    xs = torch.empty_like(x)
    xs[perm.long().to(dev)] = x
    ye2, _, gate2, up2 = _abi.grouped_swiglu_keep(xs, c, o, wg, wu, wd, e, row_map=perm.to(dev))
    for ex in range(e):
        sl = slice(int(offsets[ex]), int(offsets[ex]) + int(counts[ex]))
        assert torch.equal(ye2[sl], ye0[sl]) and torch.equal(gate2[sl], gate[sl]) and torch.equal(up2[sl], up[sl])


def test_full_size_weight_gradient_and_kept_products(gpu_device):
    """The Qwen3 prefill shape's own routing (65536 rows over 128 experts, from none to thousands of
    rows each): the weight gradient and the kept products of sampled experts against torch's f32
    matmul on the same device, every empty expert's gradient exactly zero."""
    wl = W.make_workload("qwen3_30b_a3b", with_weights=False)
    spec = wl.spec
    dev = gpu_device
    d, f, e = spec.model_dim, spec.inner_dim, spec.num_experts
    x = wl.x.reshape(-1, d).to(torch.bfloat16).to(dev)
    m = spec.mode
    idx, w, _ = _abi.router_topk(x, wl.router.to(torch.bfloat16).to(dev), wl.router_bias.to(dev), spec.top_k,
                                 _abi.SCORE_SOFTMAX if m.score_fn == "softmax" else _abi.SCORE_SIGMOID,
                                 m.renormalize, want_logits=True)
    disp = _abi.dispatch(idx, w, x, e, 16, False, gather=True)
    counts, offsets = disp.counts.cpu(), disp.offsets.cpu()
    rows = disp.xe.shape[0]
    g = torch.Generator().manual_seed(11)
    dy = torch.randn(rows, f, generator=g).to(torch.bfloat16).to(dev)
    dw = _abi.grouped_wgrad(disp.xe, dy, disp.counts, disp.offsets, e).view(e, d, f)
    order = torch.argsort(counts, descending=True)
    sample = [int(order[0]), int(order[len(order) // 4]), int(order[len(order) // 2])]
    sample += [int(i) for i in torch.nonzero(counts > 0).flatten()[-2:]]
    for ex in sample:
        lo, cnt = int(offsets[ex]), int(counts[ex])
        ref = disp.xe[lo : lo + cnt].float().t() @ dy[lo : lo + cnt].float()
        _say(f"  expert {ex}: {cnt} rows")
        assert_grad_close(dw[ex], ref.double().cpu(), "bf16", f"weight gradient of expert {ex} ({cnt} rows)")
    for ex in torch.nonzero(counts == 0).flatten().tolist():
        assert not bool(dw[ex].any()), f"expert {ex} has no rows but a gradient"
    # the kept products of the training forward
    wg, wu = ((0.05 * torch.randn(e * d, f, generator=g)).to(torch.bfloat16).to(dev) for _ in range(2))
    wd = (0.05 * torch.randn(e * f, d, generator=g)).to(torch.bfloat16).to(dev)
    ye, h, gate, up = _abi.grouped_swiglu_keep(disp.xe, disp.counts, disp.offsets, wg, wu, wd, e)
    ye0, h0 = _abi.grouped_swiglu(disp.xe, disp.counts, disp.offsets, wg, wu, wd, e)
    for ex in sample:
        lo, cnt = int(offsets[ex]), int(counts[ex])
        sl = slice(lo, lo + cnt)
        assert torch.equal(ye[sl], ye0[sl]) and torch.equal(h[sl], h0[sl])
        ref = disp.xe[sl].float() @ wg.view(e, d, f)[ex].float()
        assert_grad_close(gate[sl], ref.double().cpu(), "bf16", f"gate product of expert {ex}")
        ref = disp.xe[sl].float() @ wu.view(e, d, f)[ex].float()
        assert_grad_close(up[sl], ref.double().cpu(), "bf16", f"up product of expert {ex}")


@pytest.mark.parametrize("name", ["mixtral_8x7b", "llama4_scout"])
def test_full_size_training_step_of_the_other_shapes(gpu_device, name):
    """One training step of the module at the Mixtral and the Llama-4 Scout prefill shapes (8192
    tokens): the weight gradients of sampled experts, and of the shared expert, against the chain
    rule spelled out in torch f32 on the same device from the module's own routing
    (``moe.py:131-150``, ``experts.py:107-112``); every gradient finite, an expert without tokens
    with none.  The values of the training forward are the inference path's."""
    import torch.nn.functional as F

    wl = W.make_workload(name)
    s = wl.spec
    dev = gpu_device
    d, f, e, k = s.model_dim, s.inner_dim, s.num_experts, s.top_k
    m = build_module(wl, dev).train().requires_grad_(True)
    x = wl.x.to(torch.bfloat16).to(dev).requires_grad_(True)
    gen = torch.Generator().manual_seed(13)
    dout = torch.randn(wl.x.shape, generator=gen).to(torch.bfloat16).to(dev)
    out = m(x)
    with torch.no_grad():
        assert torch.equal(out, m(x))
    out.backward(dout)
    torch.cuda.synchronize()
    for n_, p_ in m.named_parameters():
        assert p_.grad is not None and bool(torch.isfinite(p_.grad).all()), n_
    assert bool(torch.isfinite(x.grad).all())
    rows, g2 = x.detach().reshape(-1, d), dout.reshape(-1, d)
    idx, w, _ = _abi.router_topk(rows, m.router.detach(), m.router_bias, k, _abi.SCORE_SOFTMAX
                                 if s.mode.score_fn == "softmax" else _abi.SCORE_SIGMOID, s.mode.renormalize)
    counts = torch.bincount(idx.flatten().long(), minlength=e).cpu()
    order = torch.argsort(counts, descending=True)
    scale_in = s.mode.scale_on == "input"
    bf = lambda t: t.to(torch.bfloat16).float()  # noqa: E731
    for ex in {int(order[0]), int(order[e // 2]), int(order[-1])}:
        sel = idx == ex
        tok = sel.any(dim=1).nonzero().squeeze(1)
        wg, wu, wd = (p_.detach().view(e, -1, p_.shape[1])[ex].float()
                      for p_ in (m.experts.gate_proj, m.experts.inner_proj, m.experts.output_proj))
        got = [p_.grad.view(e, -1, p_.shape[1])[ex]
               for p_ in (m.experts.gate_proj, m.experts.inner_proj, m.experts.output_proj)]
        _say(f"  {name}: expert {ex}, {tok.numel()} tokens")
        if tok.numel() == 0:
            assert not any(bool(t.any()) for t in got)
            continue
        we = (w * sel).sum(dim=1)[tok][:, None]
        xe = bf(rows[tok].float() * we) if scale_in else rows[tok].float()
        dye = g2[tok].float() if scale_in else bf(g2[tok].float() * we)
        gate, up = bf(xe @ wg), bf(xe @ wu)
        sig = torch.sigmoid(gate)
        h = bf(F.silu(gate) * up)
        dh = bf(dye @ wd.t())
        dg = bf(dh * up * (sig * (1 + gate * (1 - sig))))
        du = bf(dh * F.silu(gate))
        for what, got_t, ref in (("gate_proj", got[0], xe.t() @ dg), ("inner_proj", got[1], xe.t() @ du),
                                 ("output_proj", got[2], h.t() @ dye)):
            assert_grad_close(got_t, ref.double().cpu(), "bf16", f"{name}: d {what} of expert {ex}")
    if s.shared:
        se = m.shared_expert
        sg, su, sd = (p_.weight.detach().float() for p_ in (se.gate_proj, se.inner_proj, se.output_proj))
        xf, gf = rows.float(), g2.float()
        gate, up = bf(xf @ sg.t()), bf(xf @ su.t())
        sig = torch.sigmoid(gate)
        h = bf(F.silu(gate) * up)
        dh = bf(gf @ sd)
        dg = bf(dh * up * (sig * (1 + gate * (1 - sig))))
        du = bf(dh * F.silu(gate))
        assert_grad_close(se.output_proj.weight.grad, (gf.t() @ h).double().cpu(), "bf16", f"{name}: d shared output_proj")
        assert_grad_close(se.gate_proj.weight.grad, (dg.t() @ xf).double().cpu(), "bf16", f"{name}: d shared gate_proj")
        assert_grad_close(se.inner_proj.weight.grad, (du.t() @ xf).double().cpu(), "bf16", f"{name}: d shared inner_proj")


def test_dense_swiglu_keep_leaves_the_two_products(gpu_device):
    """The shared expert's training forward: ``y`` as the inference kernel gives it, bit for bit, and
    the two products as two GEMMs give them."""
    dev = gpu_device
    g = torch.Generator().manual_seed(3)
    t, d, f = 300, 128, 192
    x = torch.randn(t, d, generator=g).to(torch.bfloat16).to(dev)
    wg, wu = ((0.2 * torch.randn(f, d, generator=g)).to(torch.bfloat16).to(dev) for _ in range(2))
    wd = (0.2 * torch.randn(d, f, generator=g)).to(torch.bfloat16).to(dev)
    y0 = _abi.dense_swiglu(x, wg, wu, wd)
    y, gate, up = _abi.dense_swiglu_keep(x, wg, wu, wd)
    assert torch.equal(y, y0)
    assert torch.equal(gate, _abi.grouped_gemm(x, wg, _abi.W_OUT_IN))
    assert torch.equal(up, _abi.grouped_gemm(x, wu, _abi.W_OUT_IN))
    assert_grad_close(gate, x.double().cpu() @ wg.double().cpu().t(), "bf16", "gate product")


def test_backward_twice_gives_the_same_gradients(gpu_device):
    """The kept products are autograd's saved tensors: a backward pass must leave them as they are
    (``retain_graph=True`` and a second pass is how a trainer accumulates two losses)."""
    wl = W.make_workload_from_spec(W.small_spec(dtype="bf16", tokens=96, num_experts=8, model_dim=128, inner_dim=128, seed=5))
    m = build_module(wl, gpu_device).train().requires_grad_(True)
    x = wl.x.to(torch.bfloat16).to(gpu_device).requires_grad_(True)
    out = m(x)
    go = torch.randn_like(out)
    out.backward(go, retain_graph=True)
    first = [x.grad.clone()] + [p.grad.clone() for p in m.parameters()]
    x.grad = None
    for p in m.parameters():
        p.grad = None
    out.backward(go)
    second = [x.grad] + [p.grad for p in m.parameters()]
    for a, b in zip(first, second):
        assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("rows,m,n", [
    ([5, 0, 300, 64, 1], 64, 96), ([130, 257], 136, 264), ([33], 8, 8), ([0, 0], 128, 128),
    # 32 experts or more: two experts share a round of blocks when the tile grid divides by four
    # (1024 / 256 row blocks here, then 4 column blocks); an odd count leaves the last one alone
    ([(7 * i) % 90 for i in range(33)], 1024, 264), ([(11 * i) % 70 for i in range(35)], 72, 1024),
    ([40 + i for i in range(32)], 520, 520),
])
def test_grouped_wgrad_matches_torch(gpu_device, dtype, rows, m, n):
    _say("grouped_wgrad", dtype, rows, m, n)
    dt = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(m + n)
    e = len(rows)
    counts, offsets = _groups(rows)
    total = max(int(offsets[-1]), 1)
    # padding rows hold garbage on purpose: they must not enter the sum
    a = torch.randn(total, m, generator=g).to(dt)
    b = torch.randn(total, n, generator=g).to(dt)
    dev = gpu_device
    dw = _abi.grouped_wgrad(a.to(dev), b.to(dev), counts.to(dev), offsets.to(dev), e)
    assert dw.shape == (e * m, n)
    for ex in range(e):
        lo, cnt = int(offsets[ex]), int(counts[ex])
        ref = a[lo : lo + cnt].double().T @ b[lo : lo + cnt].double()
        got = dw[ex * m : (ex + 1) * m]
        if cnt == 0:
            assert float(got.float().abs().max()) == 0.0, "an expert without rows has a zero gradient"
        else:
            assert_grad_close(got, ref, dtype, f"expert {ex}")
    # through a row map, and as one group
    perm = torch.randperm(total, generator=g).to(torch.int32)
    dw2 = _abi.grouped_wgrad(a[perm.long()].contiguous().to(dev), b.to(dev), counts.to(dev), offsets.to(dev), e,
                             a_row_map=torch.argsort(perm).to(torch.int32).to(dev))
    assert torch.equal(dw2, dw), "row map"
    one = _abi.grouped_wgrad(a.to(dev), b.to(dev))
    assert_grad_close(one, a.double().T @ b.double(), dtype, "one group")


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_swiglu_backward_matches_autograd(gpu_device, dtype):
    dt = TORCH_DTYPE[dtype]
    gen = torch.Generator().manual_seed(5)
    g0, u0, dh = (2.0 * torch.randn(77, 40, generator=gen) for _ in range(3))
    g0, u0, dh = g0.to(dt), u0.to(dt), dh.to(dt)
    g64, u64 = g0.double().requires_grad_(), u0.double().requires_grad_()
    h64 = torch.nn.functional.silu(g64) * u64
    h64.backward(dh.double())
    h, dg, du = _abi.swiglu_backward(g0.to(gpu_device), u0.to(gpu_device), dh.to(gpu_device))
    assert_grad_close(h, h64.detach(), dtype, "h")
    assert_grad_close(dg, g64.grad, dtype, "dg")
    assert_grad_close(du, u64.grad, dtype, "du")


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_pair_dot(gpu_device, dtype):
    dt = TORCH_DTYPE[dtype]
    gen = torch.Generator().manual_seed(6)
    t, k, d, rows = 50, 3, 72, 400
    a, a2 = torch.randn(rows, d, generator=gen).to(dt), torch.randn(rows, d, generator=gen).to(dt)
    b = torch.randn(t, d, generator=gen).to(dt)
    ar = torch.randint(0, rows, (t, k), generator=gen).to(torch.int32)
    dev = gpu_device
    got = _abi.pair_dot(a.to(dev), ar.to(dev), b.to(dev))
    ref = (a.double()[ar.long()] * b.double()[:, None, :]).sum(-1)
    torch.testing.assert_close(got.double().cpu(), ref, rtol=1e-5, atol=1e-4)
    got2 = _abi.pair_dot(a.to(dev), ar.to(dev), b.to(dev), a2=a2.to(dev))
    ref2 = ((a.float() + a2.float()).double()[ar.long()] * b.double()[:, None, :]).sum(-1)
    torch.testing.assert_close(got2.double().cpu(), ref2, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("score_fn,renorm", [("sigmoid", False), ("sigmoid", True), ("softmax", False), ("softmax", True)])
@pytest.mark.parametrize("e,k", [(16, 4), (128, 8), (8, 8), (200, 3)])
def test_router_backward_matches_autograd(gpu_device, score_fn, renorm, e, k):
    gen = torch.Generator().manual_seed(e + k)
    t = 37
    logits = (2.0 * torch.randn(t, e, generator=gen)).float()
    idx = O.topk_lowest_index(logits.double(), k)
    l64 = logits.double().requires_grad_()
    w64 = O.combine_weights(l64, idx, score_fn, renorm)
    d_w = torch.randn(t, k, generator=gen).float()
    w64.backward(d_w.double())
    dev = gpu_device
    code = _abi.SCORE_SOFTMAX if score_fn == "softmax" else _abi.SCORE_SIGMOID
    dl = _abi.router_backward(logits.to(dev), idx.to(torch.int32).to(dev), w64.detach().float().to(dev),
                              d_w.to(dev), code, renorm, torch.float32)
    torch.testing.assert_close(dl.double().cpu(), l64.grad, rtol=2e-4, atol=2e-6)


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_backward_stages_drop_pairs_with_invalid_expert_ids(gpu_device, dtype):
    """An expert id outside [0, E) selects nothing in the forward stages (dispatch gives such a pair
    no row, combine skips it); the backward stages follow: its weight gradient is zero and it takes
    no part in the renormalisation.  Also pair_dot on operands that are not 16-byte aligned."""
    dt = TORCH_DTYPE[dtype]
    dev = gpu_device
    gen = torch.Generator().manual_seed(11)
    t, k, e, d, tile_m = 41, 3, 8, 72, 16
    logits = (1.5 * torch.randn(t, e, generator=gen)).float()
    idx = O.topk_lowest_index(logits.double(), k).to(torch.int32)
    bad = torch.rand(t, k, generator=gen) < 0.25
    bad[0], bad[1] = True, False  # a token with no valid pair at all, and one untouched
    idx[bad & (torch.arange(t)[:, None] % 2 == 0)] = -1
    idx[bad & (torch.arange(t)[:, None] % 2 == 1)] = e
    valid = (idx >= 0) & (idx < e)
    x = torch.randn(t, d, generator=gen).to(dt)
    disp = _abi.dispatch(idx.to(dev), None, x.to(dev), e, tile_m, False, gather=False)
    inv = disp.inv_perm.cpu()
    assert ((inv < 0) == ~valid).all()
    # pair_dot: rows of the expert-major buffer against the token's row
    ye = torch.randn(disp.max_rows, d, generator=gen).to(dt)
    got = _abi.pair_dot(ye.to(dev), disp.inv_perm, x.to(dev)).cpu()
    ref = (ye.double()[inv.clamp(min=0).long()] * x.double()[:, None, :]).sum(-1) * valid
    torch.testing.assert_close(got.double(), ref, rtol=1e-5, atol=1e-4)
    assert (got[~valid] == 0).all()
    # the same through views that start 2 (bf16) or 4 (fp32) bytes off a 16-byte boundary
    pad = lambda v: torch.cat([v.new_zeros(1), v.reshape(-1)]).to(dev)[1:].view(v.shape)  # noqa: E731
    got_u = _abi.pair_dot(pad(ye), disp.inv_perm, pad(x)).cpu()
    torch.testing.assert_close(got_u.double(), ref, rtol=1e-5, atol=1e-4)
    # router_backward, sigmoid scores renormalised over the VALID selected experts
    l64 = logits.double().requires_grad_()
    s = torch.sigmoid(l64).gather(1, idx.clamp(0, e - 1).long()) * valid
    w64 = s / s.sum(1, keepdim=True).clamp(min=1e-300)
    d_w = torch.randn(t, k, generator=gen).float() * valid
    w64.backward(d_w.double())
    dl = _abi.router_backward(logits.to(dev), idx.to(dev), w64.detach().float().to(dev), d_w.to(dev),
                              _abi.SCORE_SIGMOID, True, torch.float32)
    keep = valid.any(1)  # a token without a valid pair has no defined weights
    torch.testing.assert_close(dl.double().cpu()[keep], l64.grad[keep], rtol=2e-4, atol=2e-6)


# ------------------------------------------------------------------------------------- whole layer
MODES = {
    "reference": W.RoutingMode("sigmoid", False, "input"),
    "sigmoid_renorm_output": W.RoutingMode("sigmoid", True, "output"),
    "softmax_renorm_output": W.RoutingMode("softmax", True, "output"),
    "softmax_input": W.RoutingMode("softmax", False, "input"),
}


def _reference_gradients(wl, grad_out, residual, activation=None):
    """float64 autograd through the dense restatement of the reference layer."""
    s = wl.spec
    c = lambda t: None if t is None else t.double().clone().requires_grad_(True)  # noqa: E731
    x, router, gate, up, down = c(wl.x), c(wl.router), c(wl.gate), c(wl.up), c(wl.down)
    shared = (c(wl.shared_gate), c(wl.shared_up), c(wl.shared_down)) if s.shared else None
    res = c(residual)
    out = O.ref_dense_forward(
        x, router, gate, up, down, s.top_k, shared=shared,
        router_bias=None if wl.router_bias is None else wl.router_bias.double(),
        score_fn=s.mode.score_fn, renormalize=s.mode.renormalize, scale_on=s.mode.scale_on,
        **({} if activation is None else {"activation": activation}),
    )
    if res is not None:
        out = out + res
    out.backward(grad_out.double())
    grads = {"x": x.grad, "router": router.grad, "experts.gate_proj": gate.grad,
             "experts.inner_proj": up.grad, "experts.output_proj": down.grad}
    if shared is not None:
        grads.update({"shared_expert.gate_proj.weight": shared[0].grad,
                      "shared_expert.inner_proj.weight": shared[1].grad,
                      "shared_expert.output_proj.weight": shared[2].grad})
    if res is not None:
        grads["residual"] = res.grad
    return out.detach(), grads


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize(
    "mode,shared,zipf,with_residual,shape",
    [
        ("reference", False, None, False, dict(tokens=300, model_dim=64, num_experts=8, top_k=2, inner_dim=96)),
        ("reference", True, None, True, dict(tokens=257, model_dim=128, num_experts=16, top_k=1, inner_dim=64)),
        ("sigmoid_renorm_output", False, 1.0, False, dict(tokens=200, model_dim=72, num_experts=8, top_k=3, inner_dim=40)),
        ("softmax_renorm_output", False, 1.2, True, dict(tokens=500, model_dim=128, num_experts=32, top_k=8, inner_dim=192)),
        ("softmax_input", True, 1.1, False, dict(tokens=130, model_dim=64, num_experts=8, top_k=4, inner_dim=128)),
        # one to three rows per expert, the experts' inputs scaled by softmax weights of very different
        # size: weight-gradient entries are cancelling sums of two or three products
        ("softmax_input", False, 1.0, False, dict(tokens=33, model_dim=256, num_experts=20, top_k=8, inner_dim=64)),
        ("softmax_input", True, 1.0, False, dict(tokens=33, model_dim=256, num_experts=24, top_k=8, inner_dim=256)),
        # a single token: nothing averages in the router's gradient
        ("softmax_renorm_output", True, 1.0, False, dict(tokens=1, model_dim=192, num_experts=24, top_k=4, inner_dim=128)),
        # one selected expert with renormalised weights: w = 1 whatever the logits, a zero router gradient
        ("sigmoid_renorm_output", True, 1.0, True, dict(tokens=257, model_dim=192, num_experts=8, top_k=1, inner_dim=64)),
        # past 256 experts and top-16 (the backward kernels' tables and per-token loops at the library's limits)
        ("softmax_renorm_output", False, 1.0, False, dict(tokens=70, model_dim=64, num_experts=384, top_k=24, inner_dim=32)),
    ],
)
def test_layer_gradients_match_autograd_of_the_reference(gpu_device, dtype, mode, shared, zipf, with_residual, shape):
    _say("layer backward", dtype, mode, shared, zipf, with_residual, shape)
    spec = W.small_spec(dtype=dtype, zipf_s=zipf, shared=shared, mode=MODES[mode], seed=11, **shape)
    wl = W.make_workload_from_spec(spec)
    dt = TORCH_DTYPE[dtype]
    gen = torch.Generator().manual_seed(99)
    grad_out = torch.randn(wl.x.shape, generator=gen).to(dt).float()
    residual = torch.randn(wl.x.shape, generator=gen).to(dt).float() if with_residual else None
    ref_out, ref = _reference_gradients(wl, grad_out, residual)

    m = build_module(wl, gpu_device, tile_m=16).train().requires_grad_(True)
    x = wl.x.to(dt).to(gpu_device).requires_grad_(True)
    res = None if residual is None else residual.to(dt).to(gpu_device).requires_grad_(True)
    out = m(x) if res is None else m(x, residual=res)
    assert out.requires_grad and out.shape == x.shape
    with torch.no_grad():
        plain = m(x.detach()) if res is None else m(x.detach(), residual=res.detach())
    assert torch.equal(out.detach(), plain), "the training path computes the forward pass's values"
    out.backward(grad_out.to(dt).to(gpu_device))
    torch.cuda.synchronize()

    if res is not None:
        assert torch.equal(res.grad.float().cpu(), grad_out), "the residual's gradient is the output's"
    assert_layer_grads_close(m, x.grad, ref, dtype, spec.num_tokens)
    if spec.top_k == 1 and spec.mode.renormalize:
        assert float(ref["router"].abs().max()) <= STRUCTURAL_ZERO, "w = 1: the reference's router gradient is zero"


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("mode,shared", [("reference", True), ("softmax_renorm_output", False)])
def test_gradients_with_another_gate_activation(gpu_device, dtype, mode, shared):
    """``moe_activation`` other than SiLU (``llama4/moe.py:44``, ``experts.py:84-87`` take any
    module): the module's own derivative between the library's GEMMs, against float64 autograd
    through the same dense restatement with that activation."""
    act = torch.nn.GELU(approximate="tanh")
    spec = W.small_spec(tokens=257, model_dim=128, num_experts=16, top_k=2, inner_dim=192, dtype=dtype,
                        shared=shared, zipf_s=1.0, mode=MODES[mode], seed=21)
    wl = W.make_workload_from_spec(spec)
    dt = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(5)
    grad_out = torch.randn(wl.x.shape, generator=g).to(dt).float()
    _, ref = _reference_gradients(wl, grad_out, None, activation=act)
    m = build_module(wl, gpu_device)
    m.experts.activation = act
    m.train().requires_grad_(True)
    x = wl.x.to(dt).to(gpu_device).requires_grad_(True)
    m(x).backward(grad_out.to(dt).to(gpu_device))
    assert_grad_close(x.grad, ref["x"], dtype, "d x")
    for name, p in m.named_parameters():
        assert_grad_close(p.grad, ref[name], dtype, f"d {name}")


@pytest.mark.parametrize("dtype,num_experts,top_k", [("fp32", 12, 2), ("bf16", 12, 3), ("bf16", 3, 1), ("fp32", 100, 4)])
def test_gradients_with_a_number_of_experts_that_is_not_a_multiple_of_8(gpu_device, dtype, num_experts, top_k):
    """The reference takes any number of experts; the products with the router matrix are padded
    with zero columns where the kernels want rows of 16 bytes."""
    spec = W.small_spec(tokens=200, model_dim=128, num_experts=num_experts, top_k=top_k, inner_dim=64,
                        dtype=dtype, shared=num_experts == 12, zipf_s=1.0, seed=31)
    wl = W.make_workload_from_spec(spec)
    dt = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(6)
    grad_out = torch.randn(wl.x.shape, generator=g).to(dt).float()
    _, ref = _reference_gradients(wl, grad_out, None)
    m = build_module(wl, gpu_device).train().requires_grad_(True)
    x = wl.x.to(dt).to(gpu_device).requires_grad_(True)
    m(x).backward(grad_out.to(dt).to(gpu_device))
    assert_grad_close(x.grad, ref["x"], dtype, "d x")
    for name, p in m.named_parameters():
        assert p.grad.shape == p.shape
        assert_grad_close(p.grad, ref[name], dtype, f"d {name}")


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("t,d,with_weight", [(1, 64, True), (37, 200, True), (300, 2048, True), (129, 72, False),
                                             (5, 4104, True), (70, 100, True), (2100, 256, True)])
def test_rms_norm_backward_matches_autograd_of_the_oracle(gpu_device, dtype, t, d, with_weight):
    """``fs2moe_rms_norm_backward`` against float64 autograd through the oracle's restatement of
    ``torch.nn.functional.rms_norm`` (``nn/normalization.py:234-236``)."""
    dt = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(t * 1000 + d)
    x = (torch.randn(t, d, generator=g) * 1.7 + 0.3).to(dt)
    w = (1.0 + 0.2 * torch.randn(d, generator=g)).to(dt) if with_weight else None
    dy = torch.randn(t, d, generator=g).to(dt)
    eps = 1e-5
    x64 = x.double().requires_grad_(True)
    w64 = None if w is None else w.double().requires_grad_(True)
    O.rms_norm(x64, w64, eps).backward(dy.double())
    dx, dw = _abi.rms_norm_backward(x.to(gpu_device), None if w is None else w.to(gpu_device), eps,
                                    dy.to(gpu_device))
    assert_grad_close(dx, x64.grad, dtype, "d x")
    if w is None:
        assert dw is None
    else:
        assert_grad_close(dw, w64.grad, dtype, "d weight")
        # without the weight's gradient the rows' is the same, bit for bit, and needs no scratch
        dx2, none = _abi.rms_norm_backward(x.to(gpu_device), w.to(gpu_device), eps, dy.to(gpu_device),
                                           want_weight_grad=False)
        assert none is None and torch.equal(dx2, dx)


class _RMSNorm(torch.nn.Module):
    """What the layer reads of ``fairseq2.nn.RMSNorm`` (``nn/normalization.py:166-254``)."""

    def __init__(self, dim, dtype, device, weight=True):
        super().__init__()
        g = torch.Generator().manual_seed(dim)
        self.weight = torch.nn.Parameter((1.0 + 0.2 * torch.randn(dim, generator=g)).to(dtype).to(device)) if weight else None
        self.bias, self.eps, self.normalized_shape = None, 1e-5, (dim,)


@pytest.mark.parametrize("mode,shared,with_weight", [("reference", True, True), ("softmax_renorm_output", False, True),
                                                     ("reference", False, False)])
def test_gradients_through_the_normalisation_in_front_fp32(gpu_device, mode, shared, with_weight):
    """``layer(seqs, residual=seqs, norm=layer_norm)`` in training (the feed-forward half of a
    pre-norm decoder layer, ``decoder_layer.py:187-204``) against float64 autograd through the
    oracle's norm and the dense restatement of the layer.  f32 only: in bf16 the device routes the
    rounded normalised rows, whose near-ties the float64 path resolves differently (the bf16 case
    is the composition test below)."""
    spec = W.small_spec(tokens=300, model_dim=128, num_experts=16, top_k=2, inner_dim=96, dtype="fp32",
                        shared=shared, zipf_s=1.0, mode=MODES[mode], seed=41)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device).train().requires_grad_(True)
    norm = _RMSNorm(spec.model_dim, torch.float32, gpu_device, with_weight)
    g = torch.Generator().manual_seed(8)
    grad_out = torch.randn(wl.x.shape, generator=g)
    # reference: the norm in float64 in front of the dense restatement, the raw rows as residual
    s = wl.spec
    c = lambda t: None if t is None else t.double().clone().requires_grad_(True)  # noqa: E731
    x, router, gate, up, down = c(wl.x), c(wl.router), c(wl.gate), c(wl.up), c(wl.down)
    sh = (c(wl.shared_gate), c(wl.shared_up), c(wl.shared_down)) if s.shared else None
    nw = None if norm.weight is None else c(norm.weight.detach().cpu())
    out = x + O.ref_dense_forward(
        O.rms_norm(x, nw, norm.eps), router, gate, up, down, s.top_k, shared=sh,
        router_bias=None if wl.router_bias is None else wl.router_bias.double(),
        score_fn=s.mode.score_fn, renormalize=s.mode.renormalize, scale_on=s.mode.scale_on)
    out.backward(grad_out.double())
    xd = wl.x.to(gpu_device).requires_grad_(True)
    got = m(xd, residual=xd, norm=norm)
    assert_output_close(got, out.detach(), "fp32", "pre-norm layer, training path")
    got.backward(grad_out.to(gpu_device))
    assert_grad_close(xd.grad, x.grad, "fp32", "d x")
    if nw is not None:
        assert_grad_close(norm.weight.grad, nw.grad, "fp32", "d norm weight")
    ref = {"router": router.grad, "experts.gate_proj": gate.grad, "experts.inner_proj": up.grad,
           "experts.output_proj": down.grad}
    if sh is not None:
        ref.update({"shared_expert.gate_proj.weight": sh[0].grad, "shared_expert.inner_proj.weight": sh[1].grad,
                    "shared_expert.output_proj.weight": sh[2].grad})
    for name, p in m.named_parameters():
        assert_grad_close(p.grad, ref[name], "fp32", f"d {name}")


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_gradients_through_the_normalisation_compose(gpu_device, dtype):
    """The same call in bf16, checked piece by piece on the device's own normalised rows: the
    layer's gradients are those of the layer without ``norm`` on ``xn`` (bit for bit: same kernels,
    same inputs), and the rows' gradient is ``fs2moe_rms_norm_backward`` of that layer's input
    gradient plus the residual's.  (Each piece is checked against the oracle by its own test.)"""
    dt = TORCH_DTYPE[dtype]
    spec = W.small_spec(tokens=700, model_dim=256, num_experts=16, top_k=4, inner_dim=128, dtype=dtype,
                        shared=True, zipf_s=1.0, seed=43)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device).train().requires_grad_(True)
    norm = _RMSNorm(spec.model_dim, dt, gpu_device)
    g = torch.Generator().manual_seed(9)
    grad_out = torch.randn(wl.x.shape, generator=g).to(dt).to(gpu_device)
    xd = wl.x.to(dt).to(gpu_device).requires_grad_(True)
    out = m(xd, residual=xd, norm=norm)
    with torch.no_grad():
        assert torch.equal(out, m(xd, residual=xd, norm=norm))  # the inference path's values
    out.backward(grad_out)
    got = {n: p.grad.clone() for n, p in m.named_parameters()}
    got_x, got_nw = xd.grad.clone(), norm.weight.grad.clone()
    m.zero_grad()
    rows = xd.detach().reshape(-1, spec.model_dim)
    xn = _abi.router_topk_norm(rows, norm.weight.detach(), norm.eps, m.router.detach(), m.router_bias,
                               m.top_k)[0].requires_grad_(True)
    m(xn).backward(grad_out.reshape(xn.shape))
    for n, p in m.named_parameters():
        assert torch.equal(p.grad, got[n]), n
    dx, dnw = _abi.rms_norm_backward(rows, norm.weight.detach(), norm.eps, xn.grad)
    assert torch.equal(dnw, got_nw)
    want_x = (dx.float() + grad_out.reshape(xn.shape).float()).to(dt).view(got_x.shape)
    # autograd adds the two gradients of xd in the tensors' dtype: one more rounding than want_x has
    torch.testing.assert_close(got_x.float(), want_x.float(), rtol=2 ** -7 if dtype == "bf16" else 1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("e,n,d,f,act", [(6, 37, 128, 192, None), (4, 300, 256, 128, None), (3, 50, 72, 40, None),
                                         (4, 64, 128, 64, "gelu"), (5, 3, 128, 192, None), (2, 1, 64, 64, None)])
def test_grouped_expert_network_alone_is_differentiable(gpu_device, dtype, e, n, d, f, act):
    """``GroupedExpertNetwork.forward((E, n, D))`` (``experts.py:201-213``) under autograd: the
    gradients of its input and of the three weights against float64 autograd through the oracle's
    expert, and the training call's values are the inference call's."""
    from fairseq2_amd.moe import GroupedExpertNetwork

    td = TORCH_DTYPE[dtype]
    gen = torch.Generator().manual_seed(e * 100 + n)
    activation = torch.nn.GELU(approximate="tanh") if act else None
    net = GroupedExpertNetwork(e, d, f, activation=activation, device=gpu_device, dtype=td)
    wg = (0.08 * torch.randn(e * d, f, generator=gen)).to(td)
    wu = (0.08 * torch.randn(e * d, f, generator=gen)).to(td)
    wd = (0.08 * torch.randn(e * f, d, generator=gen)).to(td)
    net.load_state_dict({"gate_proj": wg, "inner_proj": wu, "output_proj": wd})
    x = torch.randn(e, n, d, generator=gen).to(td)
    dy = torch.randn(e, n, d, generator=gen).to(td)
    c = lambda t: t.double().clone().requires_grad_(True)  # noqa: E731
    x64, wg64, wu64, wd64 = c(x), c(wg), c(wu), c(wd)
    fn = torch.nn.functional.silu if activation is None else activation
    ref = torch.stack([(fn(x64[i] @ wg64.view(e, d, f)[i]) * (x64[i] @ wu64.view(e, d, f)[i])) @ wd64.view(e, f, d)[i]
                       for i in range(e)])
    if activation is None:  # the same thing as the oracle states it
        torch.testing.assert_close(ref[0], O.glu_expert(x64[0], wg64.view(e, d, f)[0], wu64.view(e, d, f)[0],
                                                        wd64.view(e, f, d)[0]))
    ref.backward(dy.double())
    xd = x.to(gpu_device).requires_grad_(True)
    y = net(xd)
    with torch.no_grad():
        assert torch.equal(y, net(xd))
    y.backward(dy.to(gpu_device))
    assert_grad_close(xd.grad, x64.grad, dtype, "d x")
    assert_grad_close(net.gate_proj.grad, wg64.grad, dtype, "d gate_proj")
    assert_grad_close(net.inner_proj.grad, wu64.grad, dtype, "d inner_proj")
    assert_grad_close(net.output_proj.grad, wd64.grad, dtype, "d output_proj")
    # frozen weights: only the input's gradient, the same bits
    net.requires_grad_(False)
    x2 = x.to(gpu_device).requires_grad_(True)
    net(x2).backward(dy.to(gpu_device))
    assert torch.equal(x2.grad, xd.grad) and net.gate_proj.grad is not None


@pytest.mark.parametrize("dtype", ["fp32", "bf16"])
@pytest.mark.parametrize("shape,d,f", [((2, 37), 128, 192), ((700,), 256, 128), ((3, 5, 7), 72, 40)])
def test_glu_feed_forward_network_alone_is_differentiable(gpu_device, dtype, shape, d, f):
    """``GLUFeedForwardNetwork.forward`` (``ffn.py:374-395``) under autograd, against float64
    autograd through the oracle's shared expert."""
    from fairseq2_amd.moe import GLUFeedForwardNetwork

    td = TORCH_DTYPE[dtype]
    gen = torch.Generator().manual_seed(d + f)
    net = GLUFeedForwardNetwork(d, f, inner_dim_scale=1.0, device=gpu_device, dtype=td)
    sg = (0.08 * torch.randn(f, d, generator=gen)).to(td)
    su = (0.08 * torch.randn(f, d, generator=gen)).to(td)
    sd = (0.08 * torch.randn(d, f, generator=gen)).to(td)
    net.load_state_dict({"gate_proj.weight": sg, "inner_proj.weight": su, "output_proj.weight": sd})
    x = torch.randn(*shape, d, generator=gen).to(td)
    dy = torch.randn(*shape, d, generator=gen).to(td)
    c = lambda t: t.double().clone().requires_grad_(True)  # noqa: E731
    x64, sg64, su64, sd64 = c(x), c(sg), c(su), c(sd)
    O.shared_glu(x64, sg64, su64, sd64).backward(dy.double())
    xd = x.to(gpu_device).requires_grad_(True)
    y = net(xd)
    with torch.no_grad():
        assert torch.equal(y, net(xd))
    y.backward(dy.to(gpu_device))
    assert_grad_close(xd.grad, x64.grad, dtype, "d x")
    assert_grad_close(net.gate_proj.weight.grad, sg64.grad, dtype, "d gate_proj")
    assert_grad_close(net.inner_proj.weight.grad, su64.grad, dtype, "d inner_proj")
    assert_grad_close(net.output_proj.weight.grad, sd64.grad, dtype, "d output_proj")


def test_frozen_parameters_get_no_gradient_and_unsupported_cases_say_so(gpu_device):
    wl = W.make_workload_from_spec(W.small_spec(dtype="bf16", tokens=64, num_experts=8, inner_dim=128, seed=3))
    m = build_module(wl, gpu_device)  # frozen
    x = wl.x.to(torch.bfloat16).to(gpu_device).requires_grad_(True)
    out = m(x)
    out.sum().backward()
    assert x.grad is not None and all(p.grad is None for p in m.parameters())

    m.experts.activation = torch.nn.PReLU().to(gpu_device)
    with pytest.raises(RuntimeError, match="parameters of its own"):
        m(x)
    m.experts.activation = torch.nn.SiLU()
    m.experts.quantize_fp8_()
    with pytest.raises(RuntimeError, match="inference format"):
        m(x)


@pytest.mark.parametrize("shared,with_residual,with_norm", [(False, False, False), (True, True, False), (True, True, True)])
def test_training_step_under_torch_compile(gpu_device, shared, with_residual, with_norm):
    """A compiled layer in training mode (transformer_lm/compiler.py:14-17 wraps layers that the
    trainer then differentiates): the registered operator carries an autograd formula, so the trace is
    one graph, and its gradients are those of the eager training path (same kernels: bit-equal)."""
    _say("compiled training step", shared, with_residual)
    spec = W.small_spec(tokens=200, model_dim=128, num_experts=8, top_k=2, inner_dim=64, dtype="bf16",
                        shared=shared, mode=W.RoutingMode("softmax", True, "output"), zipf_s=1.0, seed=21)
    wl = W.make_workload_from_spec(spec)
    gen = torch.Generator().manual_seed(5)
    g = torch.randn(wl.x.shape, generator=gen).to(torch.bfloat16).to(gpu_device)

    def grads(compiled):
        m = build_module(wl, gpu_device).train().requires_grad_(True)
        norm = _RMSNorm(spec.model_dim, torch.bfloat16, gpu_device) if with_norm else None
        x = wl.x.to(torch.bfloat16).to(gpu_device).requires_grad_(True)
        fn = (lambda t: m(t, residual=t, norm=norm)) if with_residual else (lambda t: m(t))  # noqa: E731
        if compiled:
            fn = torch.compile(fn, backend="aot_eager", fullgraph=True)
        out = fn(x)
        out.backward(g)
        torch.cuda.synchronize()
        params = {n: p.grad for n, p in m.named_parameters()}
        if norm is not None:
            params["norm.weight"] = norm.weight.grad
        return out.detach(), x.grad, params

    out_e, dx_e, dp_e = grads(False)
    out_c, dx_c, dp_c = grads(True)
    assert torch.equal(out_c, out_e)
    assert torch.equal(dx_c, dx_e)
    for n in dp_e:
        assert dp_c[n] is not None and torch.equal(dp_c[n], dp_e[n]), n

"""Pins the CPU oracle by what the mathematics fixes.

The reference has no test, fixture or golden vector for the MoE path, so each
oracle function is checked against something written independently of it:
pure-Python brute force, closed forms, a second formulation, or a reduction to
a simpler routine.  Each check is chosen so that a dropped term, a transposed
operand or a wrong index fails it.
"""

import math
import random

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import moe_oracle as O


# ---------------------------------------------------------------- inner-dim rule
def test_inner_dim_scout_closed_form():
    # llama4_scout_17b_16e: model_dim 5120, ffn_inner_dim = int(5120*4*1.2) = 24576 is passed with
    # inner_dim_scale 2/3, multiple 2048, shared expert on, capacity_factor 1.0.
    assert int(5120 * 4 * 1.2) == 24576
    assert (
        O.expert_inner_dim(24576, True, 1.0, inner_dim_scale=2 / 3, inner_dim_to_multiple=2048) == 8192
    )


@pytest.mark.parametrize(
    "inner,shared,cap,scale,mult,auto,want",
    [
        (768, False, 1.0, 1.0, 1, False, 768),  # exact F from outside
        (3000, False, 1.0, 2 / 3, 1, True, 2000),  # int(3000*2/3)=2000
        (3000, True, 1.0, 2 / 3, 1, True, 1000),  # /(1+1)
        (3000, True, 2.0, 2 / 3, 1, True, 666),  # int(2000/3)
        (3000, True, 2.0, 2 / 3, 256, True, 768),  # round 666 up to 256s
        (1000, False, 1.0, 1.0, 256, False, 1024),
        (1024, False, 1.0, 1.0, 256, False, 1024),  # already a multiple
        (100, False, 4.0, 1.0, 1, True, 25),
    ],
)
def test_inner_dim_hand_cases(inner, shared, cap, scale, mult, auto, want):
    got = O.expert_inner_dim(
        inner, shared, cap, inner_dim_scale=scale, inner_dim_to_multiple=mult, auto_scale=auto
    )
    assert got == want


# ---------------------------------------------------------------------- router
def test_router_logits_brute_force():
    rng = random.Random(1)
    t, d, e = 5, 7, 4
    x = [[rng.uniform(-1, 1) for _ in range(d)] for _ in range(t)]
    r = [[rng.uniform(-1, 1) for _ in range(e)] for _ in range(d)]
    b = [rng.uniform(-1, 1) for _ in range(e)]
    want = [[sum(x[i][k] * r[k][j] for k in range(d)) + b[j] for j in range(e)] for i in range(t)]
    got = O.router_logits(
        torch.tensor(x, dtype=torch.float64).reshape(1, t, d),
        torch.tensor(r, dtype=torch.float64),
        torch.tensor(b, dtype=torch.float64),
    )
    assert got.shape == (t, e)
    np.testing.assert_allclose(got.numpy(), np.array(want), rtol=1e-13, atol=1e-13)


def _topk_python(row, k):
    def key(j):
        v = row[j]
        if math.isnan(v):
            return (0, 0.0, j)
        return (1, -v, j)

    return sorted(range(len(row)), key=key)[:k]


def test_topk_rule_vs_python_sort():
    rng = random.Random(2)
    rows = []
    for _ in range(200):
        # few distinct values => many exact ties
        rows.append([float(rng.randint(-2, 2)) for _ in range(12)])
    rows.append([1.0, float("nan"), 3.0, 2.0, float("inf"), float("-inf")] + [0.0] * 6)
    rows.append([0.0] * 12)
    rows.append([float("-inf")] * 12)
    rows.append([float("nan")] * 3 + [5.0] * 9)
    for k in (1, 2, 5, 12):
        got = O.topk_lowest_index(torch.tensor(rows), k).tolist()
        want = [_topk_python(r, k) for r in rows]
        assert got == want


def test_topk_rule_tie_examples():
    l = torch.zeros(2, 8)
    assert O.topk_lowest_index(l, 2).tolist() == [[0, 1], [0, 1]]
    l = torch.tensor([[1.0, 3.0, 3.0, 2.0]])
    assert O.topk_lowest_index(l, 2).tolist() == [[1, 2]]
    assert O.topk_lowest_index(l, 3).tolist() == [[1, 2, 3]]
    # NaN above +inf, as torch.topk ranks it
    l = torch.tensor([[1.0, float("nan"), 3.0, 2.0, float("inf"), float("-inf")]])
    assert O.topk_lowest_index(l, 3).tolist() == [[1, 4, 2]]
    assert torch.topk(l, 3, dim=1).indices.tolist() == [[1, 4, 2]]


def test_topk_matches_torch_when_untied():
    g = torch.Generator().manual_seed(3)
    l = torch.randn(500, 128, generator=g, dtype=torch.float64)
    got = O.topk_lowest_index(l, 8)
    want = torch.topk(l, 8, dim=1).indices
    assert torch.equal(got, want)


# --------------------------------------------------------------- score functions
def test_sigmoid_weights_closed_form():
    l = torch.tensor([[0.0, 1.5, -2.0, 0.25]], dtype=torch.float64)
    idx = torch.tensor([[1, 3]])
    w = O.combine_weights(l, idx, "sigmoid", False)
    want = [1 / (1 + math.exp(-1.5)), 1 / (1 + math.exp(-0.25))]
    np.testing.assert_allclose(w.numpy()[0], want, rtol=1e-14)


def test_softmax_weights_closed_forms():
    g = torch.Generator().manual_seed(4)
    l = torch.randn(50, 16, generator=g, dtype=torch.float64)
    idx = O.topk_lowest_index(l, 4)
    full = [[math.exp(v) for v in row] for row in l.tolist()]
    w_plain = O.combine_weights(l, idx, "softmax", False)
    w_renorm = O.combine_weights(l, idx, "softmax", True)
    for t in range(50):
        z = sum(full[t])
        sel = [full[t][j] for j in idx[t].tolist()]
        np.testing.assert_allclose(w_plain[t].numpy(), [s / z for s in sel], rtol=1e-12)
        np.testing.assert_allclose(w_renorm[t].numpy(), [s / sum(sel) for s in sel], rtol=1e-12)
    assert torch.allclose(w_renorm.sum(1), torch.ones(50, dtype=torch.float64), atol=1e-14)
    # softmax over all -> top-k -> divide by selected sum == softmax over selected logits
    np.testing.assert_allclose(
        (w_plain / w_plain.sum(1, keepdim=True)).numpy(), w_renorm.numpy(), rtol=1e-12
    )


# ------------------------------------------------------------ routing artefacts
def _route_python(idx, num_experts, tile_m):
    t, k = len(idx), len(idx[0])
    pairs = sorted((idx[i][s], i, s) for i in range(t) for s in range(k))  # expert-major, token-ascending
    counts = [0] * num_experts
    for e, _, _ in pairs:
        counts[e] += 1
    offsets = [0]
    for c in counts:
        offsets.append(offsets[-1] + (c + tile_m - 1) // tile_m * tile_m)
    perm = [-1] * offsets[-1]
    inv = [[None] * k for _ in range(t)]
    seen = [0] * num_experts
    for e, i, s in pairs:
        row = offsets[e] + seen[e]
        seen[e] += 1
        perm[row] = i
        inv[i][s] = row
    return counts, offsets, perm, inv


@pytest.mark.parametrize("tile_m", [1, 4, 16])
def test_route_vs_python(tile_m):
    g = torch.Generator().manual_seed(5)
    l = torch.randn(77, 10, generator=g)
    l[:, 7] = -100.0  # an expert nobody selects
    idx = O.topk_lowest_index(l, 3)
    r = O.route(idx, 10, tile_m)
    counts, offsets, perm, inv = _route_python(idx.tolist(), 10, tile_m)
    assert r.counts.tolist() == counts and counts[7] == 0
    assert r.offsets.tolist() == offsets
    assert r.perm.tolist() == perm
    assert r.inv_perm.tolist() == inv
    assert r.num_rows == offsets[-1]


def test_route_matches_reference_score_matrix_order():
    # The canonical order is the row-major non-zeros of the (E, T) score matrix (moe.py:115-119).
    g = torch.Generator().manual_seed(6)
    logits = torch.randn(40, 6, generator=g)
    scores, ti = torch.topk(logits, 2, dim=1)
    dense = torch.full_like(logits, float("-inf")).scatter_(1, ti, scores).transpose(0, 1)
    nz = torch.nonzero(dense > float("-inf"))  # rows sorted (e, t)
    r = O.route(O.topk_lowest_index(logits, 2), 6, 1)
    assert r.perm.tolist() == nz[:, 1].tolist()
    assert r.counts.tolist() == (dense > float("-inf")).sum(1).tolist()
    # bijection and inverse
    assert int(r.counts.sum()) == 40 * 2
    flat = r.inv_perm.reshape(-1)
    assert sorted(flat.tolist()) == list(range(80))
    assert (r.perm[flat] == np.repeat(np.arange(40), 2)).all()


# ------------------------------------------------------------------ whole layer
def _silu(v):
    return v / (1.0 + math.exp(-v))


def _moe_python(x, router, bias, wg, wu, wd, k, score_fn, renorm, scale_on, shared):
    """Textbook layer in pure-Python floats.  wg/wu: [E][D][F]; wd: [E][F][D]."""
    t, d = len(x), len(x[0])
    e, f = len(wg), len(wg[0][0])
    out = []
    for i in range(t):
        logit = [sum(x[i][a] * router[a][j] for a in range(d)) + (bias[j] if bias else 0.0) for j in range(e)]
        sel = _topk_python(logit, k)
        if score_fn == "sigmoid":
            w = [1 / (1 + math.exp(-logit[j])) for j in sel]
        else:
            ex = [math.exp(v) for v in logit]
            z = sum(ex[j] for j in sel) if renorm else sum(ex)
            w = [ex[j] / z for j in sel]
        if shared:
            gs, us, ds = shared  # (F, D), (F, D), (D, F)
            hh = [
                _silu(sum(x[i][a] * gs[b][a] for a in range(d))) * sum(x[i][a] * us[b][a] for a in range(d))
                for b in range(f)
            ]
            y = [sum(hh[b] * ds[a][b] for b in range(f)) for a in range(d)]
        else:
            y = [0.0] * d
        for j, wj in sorted(zip(sel, w)):
            u = [x[i][a] * wj for a in range(d)] if scale_on == "input" else x[i]
            hh = [
                _silu(sum(u[a] * wg[j][a][b] for a in range(d))) * sum(u[a] * wu[j][a][b] for a in range(d))
                for b in range(f)
            ]
            ye = [sum(hh[b] * wd[j][b][a] for b in range(f)) for a in range(d)]
            s = 1.0 if scale_on == "input" else wj
            y = [y[a] + s * ye[a] for a in range(d)]
        out.append(y)
    return out


@pytest.mark.parametrize(
    "score_fn,renorm,scale_on,use_bias,use_shared",
    [
        ("sigmoid", False, "input", False, False),  # the reference layer
        ("sigmoid", False, "input", False, True),  # with shared expert
        ("softmax", True, "output", True, False),  # Mixtral / Qwen3 convention
        ("softmax", False, "output", True, True),
        ("sigmoid", False, "output", False, False),
    ],
)
def test_layer_vs_pure_python(score_fn, renorm, scale_on, use_bias, use_shared):
    rng = random.Random(11)
    t, d, e, f, k = 6, 5, 4, 7, 2  # all different so a transposed operand cannot slip through
    u = lambda *shape: (
        [u(*shape[1:]) for _ in range(shape[0])] if len(shape) > 1 else [rng.uniform(-1, 1) for _ in range(shape[0])]
    )
    x, router = u(t, d), u(d, e)
    bias = u(e) if use_bias else None
    wg, wu, wd = u(e, d, f), u(e, d, f), u(e, f, d)
    shared = (u(f, d), u(f, d), u(d, f)) if use_shared else None
    want = _moe_python(x, router, bias, wg, wu, wd, k, score_fn, renorm, scale_on, shared)

    T = lambda v: torch.tensor(v, dtype=torch.float64)
    kw = dict(
        shared=tuple(T(s) for s in shared) if shared else None,
        router_bias=T(bias) if bias else None,
        score_fn=score_fn,
        renormalize=renorm,
        scale_on=scale_on,
    )
    args = (T(x).reshape(2, 3, d), T(router), T(wg).reshape(e * d, f), T(wu).reshape(e * d, f), T(wd).reshape(e * f, d), k)
    sparse = O.ref_sparse_forward(*args, **kw)
    dense = O.ref_dense_forward(*args, **kw)
    assert sparse.out.shape == (2, 3, d)
    np.testing.assert_allclose(sparse.out.reshape(t, d).numpy(), np.array(want), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(dense.reshape(t, d).numpy(), np.array(want), rtol=1e-12, atol=1e-13)


@pytest.mark.parametrize("mode", [("sigmoid", False, "input"), ("softmax", True, "output")])
@pytest.mark.parametrize("tile_m", [1, 16])
def test_dense_equals_sparse(mode, tile_m):
    g = torch.Generator().manual_seed(12)
    t, d, e, f, k = 64, 32, 8, 48, 2
    x = torch.randn(4, 16, d, generator=g, dtype=torch.float64)
    router = torch.randn(d, e, generator=g, dtype=torch.float64)
    wg = 0.1 * torch.randn(e * d, f, generator=g, dtype=torch.float64)
    wu = 0.1 * torch.randn(e * d, f, generator=g, dtype=torch.float64)
    wd = 0.1 * torch.randn(e * f, d, generator=g, dtype=torch.float64)
    kw = dict(score_fn=mode[0], renormalize=mode[1], scale_on=mode[2])
    dense = O.ref_dense_forward(x, router, wg, wu, wd, k, **kw)
    sp = O.ref_sparse_forward(x, router, wg, wu, wd, k, tile_m=tile_m, **kw)
    assert torch.allclose(dense, sp.out, rtol=1e-12, atol=1e-13)
    # intermediates are consistent with one another
    r = sp.routing
    rows = torch.from_numpy(r.inv_perm.astype(np.int64))
    tok = torch.from_numpy(r.perm.astype(np.int64))
    valid = tok >= 0
    assert int(valid.sum()) == t * k
    assert torch.all(sp.xe[~valid] == 0) and torch.all(sp.ye[~valid] == 0)
    xs = x.reshape(-1, d)
    for s in range(k):
        got = sp.xe[rows[:, s]]
        want = xs * sp.topk_w[:, s : s + 1] if mode[2] == "input" else xs
        assert torch.allclose(got, want, rtol=1e-14, atol=0)


def test_single_expert_reduces_to_glu_ffn():
    # E=1, K=1: every token goes to the only expert with weight sigmoid(logit); the layer is a plain
    # GLU network on the scaled input, which the shared-expert routine computes with transposed weights.
    g = torch.Generator().manual_seed(13)
    t, d, f = 10, 6, 9
    x = torch.randn(1, t, d, generator=g, dtype=torch.float64)
    router = torch.randn(d, 1, generator=g, dtype=torch.float64)
    wg, wu = torch.randn(d, f, generator=g, dtype=torch.float64), torch.randn(d, f, generator=g, dtype=torch.float64)
    wd = torch.randn(f, d, generator=g, dtype=torch.float64)
    out = O.ref_sparse_forward(x, router, wg, wu, wd, 1).out
    scaled = x * torch.sigmoid(x @ router)
    want = O.shared_glu(scaled, wg.T.contiguous(), wu.T.contiguous(), wd.T.contiguous())
    assert torch.allclose(out, want, rtol=1e-12, atol=1e-13)
    # and the textbook formula without helper routines
    want2 = ((scaled @ wg) / (1 + torch.exp(-(scaled @ wg))) * (scaled @ wu)) @ wd
    assert torch.allclose(out, want2, rtol=1e-12, atol=1e-13)


def test_all_experts_selected():
    # K=E: no zeros anywhere in the dense formulation; the layer is a plain sum over experts.
    g = torch.Generator().manual_seed(14)
    t, d, e, f = 12, 8, 3, 5
    x = torch.randn(1, t, d, generator=g, dtype=torch.float64)
    router = torch.randn(d, e, generator=g, dtype=torch.float64)
    wg, wu = torch.randn(e * d, f, generator=g, dtype=torch.float64), torch.randn(e * d, f, generator=g, dtype=torch.float64)
    wd = torch.randn(e * f, d, generator=g, dtype=torch.float64)
    want = torch.zeros(t, d, dtype=torch.float64)
    xs = x.reshape(t, d)
    s = torch.sigmoid(xs @ router)
    for j in range(e):
        u = xs * s[:, j : j + 1]
        want += O.glu_expert(u, wg[j * d : (j + 1) * d], wu[j * d : (j + 1) * d], wd[j * f : (j + 1) * f])
    for fn in (O.ref_dense_forward, lambda *a: O.ref_sparse_forward(*a).out):
        assert torch.allclose(fn(x, router, wg, wu, wd, e).reshape(t, d), want, rtol=1e-12, atol=1e-13)


def test_zero_router_uses_tie_rule():
    g = torch.Generator().manual_seed(15)
    t, d, e, f, k = 9, 4, 5, 3, 2
    x = torch.randn(1, t, d, generator=g, dtype=torch.float64)
    router = torch.zeros(d, e, dtype=torch.float64)
    wg, wu = torch.randn(e * d, f, generator=g, dtype=torch.float64), torch.randn(e * d, f, generator=g, dtype=torch.float64)
    wd = torch.randn(e * f, d, generator=g, dtype=torch.float64)
    sp = O.ref_sparse_forward(x, router, wg, wu, wd, k)
    assert sp.topk_idx.tolist() == [[0, 1]] * t
    assert sp.routing.counts.tolist() == [t, t, 0, 0, 0]
    xs = x.reshape(t, d) * 0.5  # sigmoid(0)
    want = O.glu_expert(xs, wg[:d], wu[:d], wd[:f]) + O.glu_expert(xs, wg[d : 2 * d], wu[d : 2 * d], wd[f : 2 * f])
    assert torch.allclose(sp.out.reshape(t, d), want, rtol=1e-12, atol=1e-13)


def test_output_weighting_is_linear_in_the_weights():
    # With scale_on="output" the layer is linear in the combine weights; with "input" it is not.
    g = torch.Generator().manual_seed(16)
    t, d, e, f, k = 20, 8, 4, 6, 2
    x = torch.randn(1, t, d, generator=g, dtype=torch.float64)
    router = torch.randn(d, e, generator=g, dtype=torch.float64)
    wg, wu = torch.randn(e * d, f, generator=g, dtype=torch.float64), torch.randn(e * d, f, generator=g, dtype=torch.float64)
    wd = torch.randn(e * f, d, generator=g, dtype=torch.float64)
    a = O.ref_sparse_forward(x, router, wg, wu, wd, k, score_fn="softmax", renormalize=False, scale_on="output")
    b = O.ref_sparse_forward(x, router, wg, wu, wd, k, score_fn="softmax", renormalize=True, scale_on="output")
    ratio = (b.topk_w / a.topk_w)[:, :1]  # renormalisation rescales all of a token's weights alike
    assert torch.allclose(b.out.reshape(t, d), a.out.reshape(t, d) * ratio, rtol=1e-12, atol=1e-13)


def test_combine_order_is_ascending_expert_like_scatter_add():
    # In fp32 the summation order is visible; the oracle must add in ascending expert id from the base.
    g = torch.Generator().manual_seed(17)
    t, d, e, f, k = 256, 16, 8, 24, 4
    x = torch.randn(1, t, d, generator=g)
    router = torch.randn(d, e, generator=g)
    wg, wu = torch.randn(e * d, f, generator=g), torch.randn(e * d, f, generator=g)
    wd = torch.randn(e * f, d, generator=g)
    sh = (torch.randn(f, d, generator=g), torch.randn(f, d, generator=g), torch.randn(d, f, generator=g))
    sp = O.ref_sparse_forward(x, router, wg, wu, wd, k, shared=sh)
    # rebuild from the oracle's own per-row outputs with scatter_add_ in expert order
    out = sp.base.clone()
    perm = torch.from_numpy(sp.routing.perm.astype(np.int64))
    rows = torch.nonzero(perm >= 0).reshape(-1)
    out.scatter_add_(0, perm[rows].reshape(-1, 1).expand(-1, d), sp.ye[rows])
    assert torch.equal(out, sp.out.reshape(t, d))


def test_token_subset_evaluation():
    g = torch.Generator().manual_seed(18)
    t, d, e, f, k = 50, 8, 6, 10, 2
    x = torch.randn(1, t, d, generator=g, dtype=torch.float64)
    router = torch.randn(d, e, generator=g, dtype=torch.float64)
    wg, wu = torch.randn(e * d, f, generator=g, dtype=torch.float64), torch.randn(e * d, f, generator=g, dtype=torch.float64)
    wd = torch.randn(e * f, d, generator=g, dtype=torch.float64)
    full = O.ref_sparse_forward(x, router, wg, wu, wd, k).out.reshape(t, d)
    tok = torch.tensor([0, 7, 33, 49])
    part = O.ref_sparse_forward(x, router, wg, wu, wd, k, tokens=tok).out.reshape(t, d)
    assert torch.allclose(part[tok], full[tok], rtol=1e-13, atol=1e-14)


# ----------------------------------------------------------------------- RMS norm in front
def test_rms_norm_vs_pure_python():
    rng = random.Random(5)
    rows, dim, eps = 3, 7, 1e-5
    x = [[rng.uniform(-2, 2) for _ in range(dim)] for _ in range(rows)]
    w = [rng.uniform(0.5, 1.5) for _ in range(dim)]
    want = []
    for row in x:
        ms = sum(v * v for v in row) / dim
        want.append([v / math.sqrt(ms + eps) * g for v, g in zip(row, w)])
    got = O.rms_norm(torch.tensor(x, dtype=torch.float64), torch.tensor(w, dtype=torch.float64), eps)
    assert torch.allclose(got, torch.tensor(want, dtype=torch.float64), rtol=1e-12, atol=0)


def test_rms_norm_closed_forms():
    # a constant row c normalises to c / sqrt(c^2 + eps); without eps to +-1
    x = torch.full((2, 16), -3.0)
    assert torch.equal(O.rms_norm(x, None, 0.0), torch.full((2, 16), -1.0))
    got = O.rms_norm(x, None, 7.0)  # 9 + 7 = 16
    assert torch.allclose(got, torch.full((2, 16), -0.75), rtol=1e-6)
    # eps = 0: invariant under scaling the row by a power of two (exact in floating point),
    # and the output has unit mean square
    g = torch.Generator().manual_seed(3)
    y = torch.randn(5, 64, generator=g)
    assert torch.equal(O.rms_norm(4.0 * y, None, 0.0), O.rms_norm(y, None, 0.0))
    assert torch.allclose(O.rms_norm(y, None, 0.0).pow(2).mean(-1), torch.ones(5), rtol=1e-5)
    # the weight multiplies element by element
    w = torch.randn(64, generator=g)
    assert torch.equal(O.rms_norm(y, w, 1e-5), O.rms_norm(y, None, 1e-5) * w)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_vs_library_routine(dtype):
    """torch.nn.functional.rms_norm is the routine RMSNorm.forward calls
    (nn/normalization.py:234-236): the oracle's restatement must round where it rounds."""
    g = torch.Generator().manual_seed(9)
    x = (2.0 * torch.randn(33, 96, generator=g)).to(dtype)
    w = (1.0 + 0.2 * torch.randn(96, generator=g)).to(dtype)
    got = O.rms_norm(x, w, 1e-5)
    want = F.rms_norm(x, (96,), w, 1e-5)
    assert got.dtype == dtype
    if dtype == torch.float32:
        assert torch.allclose(got, want, rtol=2e-6, atol=0)
    else:
        assert torch.equal(got, want)  # one rounding, at the end
        # and a deliberately double-rounded evaluation is NOT what the routine computes
        xf = x.float()
        twice = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).to(dtype) * w
        assert not torch.equal(twice, want)


def test_sigmoid_renormalised_weights_closed_form():
    """combine_weights(sigmoid, renormalize=True): sigma(l_e) / sum over the selected of sigma(l_j).
    Closed forms: equal logits give 1/K each whatever their value; logits (0, +inf-ish) give
    (1/3, 2/3) since sigma(0) = 1/2 and sigma(40) = 1; the weights of a token sum to one; scaling all
    selected sigmoids by a common factor (logit pairs (a, b) with sigma(a) = 2 sigma(b)) gives 2/3, 1/3."""
    k = 3
    logits = torch.tensor([[1.7, 1.7, 1.7, -5.0], [-2.0, -2.0, -2.0, -9.0]], dtype=torch.float64)
    idx = O.topk_lowest_index(logits, k)
    w = O.combine_weights(logits, idx, "sigmoid", True)
    assert torch.allclose(w, torch.full((2, k), 1.0 / 3.0, dtype=torch.float64), atol=1e-15)
    logits = torch.tensor([[0.0, 40.0, -50.0]], dtype=torch.float64)
    idx = O.topk_lowest_index(logits, 2)  # descending: expert 1, then expert 0
    w = O.combine_weights(logits, idx, "sigmoid", True)
    assert idx.tolist() == [[1, 0]]
    assert torch.allclose(w, torch.tensor([[2.0 / 3.0, 1.0 / 3.0]], dtype=torch.float64), atol=1e-12)
    # sigma(a) = 2 sigma(b) with sigma(b) = 0.3: a = logit(0.6), b = logit(0.3)
    a, b = math.log(0.6 / 0.4), math.log(0.3 / 0.7)
    logits = torch.tensor([[b, -30.0, a]], dtype=torch.float64)
    idx = O.topk_lowest_index(logits, 2)
    w = O.combine_weights(logits, idx, "sigmoid", True)
    assert idx.tolist() == [[2, 0]]
    assert torch.allclose(w, torch.tensor([[2.0 / 3.0, 1.0 / 3.0]], dtype=torch.float64), atol=1e-12)
    # random logits: rows sum to one and the ratios are the ratios of the plain sigmoids
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(50, 9, generator=g, dtype=torch.float64)
    idx = O.topk_lowest_index(logits, 4)
    w = O.combine_weights(logits, idx, "sigmoid", True)
    plain = O.combine_weights(logits, idx, "sigmoid", False)
    assert torch.allclose(w.sum(dim=1), torch.ones(50, dtype=torch.float64), atol=1e-14)
    assert torch.allclose(w * plain[:, :1], plain * w[:, :1], atol=1e-15)
    # not renormalised, for contrast: the plain sigmoids, which do not sum to one
    assert torch.allclose(plain, torch.sigmoid(torch.gather(logits, 1, idx)), atol=0)


def test_bf16_rounding_budget_of_the_device_pipeline():
    """The error budget behind the bf16 tolerance (tests/_util.py): the layer evaluated in f32 with a
    bf16 rounding wherever the device rounds, against the f64 oracle, in the configuration with the
    most roundings per output element (every one of 16 experts selected, scaled input rows).  The
    overall error is a few tenths of a percent of the output's rms, well inside RMS_TOL, and every
    element is inside the element-wise bound (the largest errors sit on the largest elements, where
    the final rounding alone is 2^-9 of the value: they are what rtol is for)."""
    import workloads as W
    from tests._util import RMS_TOL, TOL, emulate_device_rounding, oracle_forward, oracle_routing

    spec = W.small_spec(tokens=300, model_dim=256, num_experts=16, top_k=16, inner_dim=192, dtype="bf16",
                        zipf_s=1.5, mode=W.RoutingMode("sigmoid", False, "input"), seed=1012)
    wl = W.make_workload_from_spec(spec)
    _, idx, w = oracle_routing(wl)
    ref = oracle_forward(wl, idx, 16, dtype=torch.float64).out.reshape(-1, 256)
    emu = emulate_device_rounding(wl, idx, w).double()
    err = (emu - ref).abs()
    rms = float(ref.pow(2).mean().sqrt())
    sigma = float(err.pow(2).mean().sqrt()) / rms
    assert 5e-4 < sigma < 6e-3, sigma  # ~ 2^-9 .. 3 * 2^-9
    assert sigma < 0.6 * RMS_TOL["bf16"]
    rtol, atol_rel = TOL["bf16"]
    assert atol_rel == 2e-2
    # this configuration (K >= 8 terms, each rounded a fourth time on the way in) is the one the GPU
    # tests give twice the element-wise room (atol_scale = 2): with it every element is well inside,
    worst = float((err / (2 * atol_rel * rms + rtol * ref.abs())).max())
    assert worst < 0.6, worst
    # while at the default the same elements come close to the bound: no room for the tail of a
    # larger output
    assert 0.6 < float((err / (atol_rel * rms + rtol * ref.abs())).max()) < 1.0


# ------------------------------------------------------------------ block-scaled e4m3 (act_quant)
def _e4m3_values():
    """Every finite e4m3fn value by the format's definition (1 sign, 4 exponent bits with bias 7,
    3 mantissa bits, no infinities, 0x7f / 0xff are NaN), in pure Python: code -> value."""
    vals = {}
    for code in range(256):
        if code & 0x7F == 0x7F:
            continue
        s, e, m = code >> 7, (code >> 3) & 15, code & 7
        v = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        vals[code] = -v if s else v
    return vals


def test_mx_block_exponent_closed_forms():
    f32 = torch.float32
    n = torch.arange(-20, 21)
    top = torch.ldexp(torch.tensor(448.0), n)  # 448 * 2^n fits exactly: X = n
    assert O.mx_block_exponent(top).tolist() == n.tolist()
    above = torch.nextafter(top, torch.tensor(float("inf")))  # one ulp more needs the next exponent
    assert O.mx_block_exponent(above).tolist() == (n + 1).tolist()
    assert O.mx_block_exponent(torch.tensor([1.0, 1.75, 1.7500001, 2.0, 224.0, 255.9, 256.0], dtype=f32)).tolist() == [
        -8, -8, -7, -7, -1, 0, 0]
    assert O.mx_block_exponent(torch.tensor([0.0, 1e-45, 2.0 ** -127], dtype=f32)).tolist() == [-127, -127, -127]
    assert O.mx_block_exponent(torch.tensor([2.0 ** -126, 2.9e38, 3e38], dtype=f32)).tolist() == [-127, 119, 120]
    # the defining property on random magnitudes: amax / 2^X <= 448 < amax / 2^(X - 1)
    g = torch.Generator().manual_seed(5)
    a = torch.exp(20 * torch.rand(4096, generator=g) - 10).to(f32)
    x = O.mx_block_exponent(a)
    assert bool((torch.ldexp(a.double(), -x) <= 448).all())
    assert bool((torch.ldexp(a.double(), -(x - 1)) > 448).all())


def test_mx_quantize_is_the_nearest_code_with_ties_to_even():
    """Brute force over the table of all codes: the quantised value of every element is the e4m3
    value nearest to element / 2^X, and on a tie the one with the even code."""
    vals = _e4m3_values()
    table = sorted((v, c) for c, v in vals.items() if c < 0x80)  # non-negative half
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(24, 64, generator=g) * torch.exp(3 * torch.randn(24, 1, generator=g))).to(torch.bfloat16)
    x[0, :32] = 0
    x[1, :4] = torch.tensor([17.0, 19.0, 448.0, 0.0009765625])  # exact ties below a larger element
    x[1, 4] = 28.0
    codes, sb = O.mx_quantize(x)
    got = codes.view(torch.uint8).reshape(24, 2, 32)
    for r in range(24):
        for b in range(2):
            blk = x[r, 32 * b : 32 * b + 32].double()
            amax = float(blk.abs().max())
            xexp = int(sb[r, b]) - 127
            if amax == 0:
                assert xexp == -127 and int(got[r, b].sum()) == 0
                continue
            assert amax / 2.0 ** xexp <= 448 < amax / 2.0 ** (xexp - 1)
            for i in range(32):
                t = abs(float(blk[i])) / 2.0 ** xexp
                best = min(table, key=lambda vc: (abs(vc[0] - t), vc[1] & 1))
                want = best[1] | (0x80 if float(blk[i]) < 0 else 0)
                have = int(got[r, b, i])
                assert vals[have] == vals[want], (r, b, i, float(blk[i]), have, want)
    # and the round trip: exact for what e4m3 holds, within 2^-4 of the value (normal range) or
    # 2^-10 of the block's scale (below it) otherwise
    back = O.mx_dequantize(codes, sb).double().reshape(24, 2, 32)
    xs = x.double().reshape(24, 2, 32)
    scale = torch.ldexp(torch.ones(24, 2, dtype=torch.float64), sb.to(torch.int32) - 127).unsqueeze(-1)
    err = (back - xs).abs()
    assert bool((err <= torch.maximum(xs.abs() * 2.0 ** -4, scale * 2.0 ** -10) + 1e-300).all())
    pow2 = torch.ldexp(torch.ones(1, 32), torch.arange(-3, 5).repeat(4).unsqueeze(0))
    assert torch.equal(O.mx_round(pow2), pow2)


def test_sparse_forward_with_quantised_activations_is_the_layer_on_rounded_inputs():
    """act_quant="mxfp8" against the composition written out by hand for one expert and one token
    per row group: round the rows, multiply, gate, round the product, multiply."""
    g = torch.Generator().manual_seed(3)
    t, d, f, e = 6, 64, 32, 2
    x = torch.randn(t, d, generator=g, dtype=torch.float64).to(torch.bfloat16).double()  # bf16 rows
    router = torch.randn(d, e, generator=g, dtype=torch.float64)
    gate, up = (0.2 * torch.randn(e * d, f, generator=g, dtype=torch.float64) for _ in range(2))
    down = 0.2 * torch.randn(e * f, d, generator=g, dtype=torch.float64)
    res = O.ref_sparse_forward(x, router, gate, up, down, 1, score_fn="softmax", renormalize=True,
                               scale_on="output", act_quant="mxfp8")
    plain = O.ref_sparse_forward(x, router, gate, up, down, 1, score_fn="softmax", renormalize=True,
                                 scale_on="output")
    assert torch.equal(res.topk_idx, plain.topk_idx), "the router sees the unrounded rows"
    want = torch.zeros(t, d, dtype=torch.float64)
    for i in range(t):
        ex = int(res.topk_idx[i, 0])
        u = O.mx_round(x[i : i + 1])
        h = torch.nn.functional.silu(u @ gate.view(e, d, f)[ex]) * (u @ up.view(e, d, f)[ex])
        want[i] = (O.mx_round(h) @ down.view(e, f, d)[ex])[0]  # weight 1: one expert, renormalised
    torch.testing.assert_close(res.out, want, rtol=1e-12, atol=1e-12)
    rel = float((res.out - plain.out).norm() / plain.out.norm())
    # the format's noise: three mantissa bits leave every element off by up to 2^-4 of its size
    # (3.6 % rms), at two places of the pipeline, so some 5-6 % of the output's norm
    assert 2e-2 < rel < 1e-1, rel

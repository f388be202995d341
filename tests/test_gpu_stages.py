"""GPU parity of each stage, called through the C ABI, against the CPU oracle."""

import numpy as np
import pytest
import torch

from fairseq2_amd import _abi
import workloads as W
from oracle import moe_oracle as O
from tests._util import TORCH_DTYPE, assert_output_close, assert_routing_equal, oracle_routing

pytestmark = pytest.mark.gpu

MODES = {
    "reference": W.RoutingMode("sigmoid", False, "input"),
    "softmax_renorm": W.RoutingMode("softmax", True, "output"),
    "softmax_plain": W.RoutingMode("softmax", False, "output"),
    "sigmoid_renorm": W.RoutingMode("sigmoid", True, "output"),
}


def _say(*a):
    print(*a, flush=True)


# ------------------------------------------------------------------------------------------ router
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize(
    "tokens,d,e,k,mode,zipf",
    [
        (333, 64, 8, 2, "reference", None),
        (1000, 256, 128, 8, "softmax_renorm", 1.2),
        (257, 136, 16, 1, "reference", None),
        (100, 512, 200, 16, "softmax_plain", 1.1),
        (64, 72, 5, 5, "sigmoid_renorm", None),  # K == E
        (31, 64, 1, 1, "reference", None),  # E == 1
        (50, 128, 256, 16, "softmax_renorm", 1.0),  # the largest E the matrix-pipe router takes
        (70, 128, 512, 32, "softmax_renorm", 1.0),  # the largest E and K the library takes
        (33, 200, 384, 24, "sigmoid_renorm", None),
        # bf16 with D >= 512 and few tokens: several blocks share a token tile
        (64, 2048, 128, 8, "softmax_renorm", 1.2),   # 8 blocks per tile
        (33, 1024, 256, 16, "softmax_plain", 1.0),   # two-fragment kernel, 8 blocks per tile
        (3000, 576, 24, 3, "reference", None),       # 2 blocks per tile, 9 chunks: uneven shares
        (1, 512, 8, 2, "sigmoid_renorm", None),
    ],
)
def test_router_matches_oracle(gpu_device, dtype, tokens, d, e, k, mode, zipf):
    _say("router", dtype, tokens, d, e, k, mode)
    spec = W.small_spec(tokens=tokens, model_dim=d, num_experts=e, top_k=k, inner_dim=8, dtype=dtype,
                        zipf_s=zipf, mode=MODES[mode], seed=tokens)
    wl = W.make_workload_from_spec(spec, with_weights=False)
    logits, idx, w = oracle_routing(wl)
    dt = TORCH_DTYPE[dtype]
    x = wl.x.reshape(-1, d).to(dt).to(gpu_device)
    bias = None if wl.router_bias is None else wl.router_bias.to(gpu_device)
    gi, gw, gl = _abi.router_topk(
        x, wl.router.to(dt).to(gpu_device), bias, k, _abi.SCORE_SOFTMAX if "softmax" in mode else _abi.SCORE_SIGMOID,
        spec.mode.renormalize, want_logits=True,
    )
    np.testing.assert_allclose(gl.cpu().double().numpy(), logits.numpy(), rtol=1e-5, atol=2e-5)
    assert torch.equal(gi.cpu().long(), idx), "selected experts differ from the oracle"
    np.testing.assert_allclose(gw.cpu().double().numpy(), w.numpy(), rtol=5e-5, atol=1e-6)
    # without the scratch buffer one block per 32 tokens walks all of D: same selection, logits
    # equal up to the f32 summation order
    si, sw, sl = _abi.router_topk(
        x, wl.router.to(dt).to(gpu_device), bias, k, _abi.SCORE_SOFTMAX if "softmax" in mode else _abi.SCORE_SIGMOID,
        spec.mode.renormalize, want_logits=True, split=False,
    )
    np.testing.assert_allclose(sl.cpu().double().numpy(), logits.numpy(), rtol=1e-5, atol=2e-5)
    assert torch.equal(si.cpu().long(), idx), "selected experts differ from the oracle (one block per tile)"
    np.testing.assert_allclose(sw.cpu().double().numpy(), w.numpy(), rtol=5e-5, atol=1e-6)
    splits = _abi.load().fs2moe_router_workspace_bytes(x.shape[0], d, e, _abi.dtype_code(dt)) > 0
    assert splits == (dtype == "bf16" and d >= 512 and tokens <= 4096)
    if not splits:
        assert torch.equal(gl, sl) and torch.equal(gw, sw)


@pytest.mark.parametrize(
    "tokens,d,e,k,mode,zipf",
    [
        (1, 2048, 128, 8, "softmax_renorm", 1.2),    # the decode step of the benchmark's layer
        (4, 2048, 128, 8, "softmax_renorm", None),
        (3, 4096, 8, 2, "softmax_renorm", None),
        (2, 5120, 16, 1, "sigmoid_renorm", None),
        (4, 2048, 256, 16, "softmax_plain", 1.0),
        (3, 8192, 64, 6, "reference", None),
        (4, 520, 32, 4, "softmax_plain", None),      # 9 chunks of the model dimension over 2 blocks
        (1, 8, 8, 8, "reference", None),             # one 16-byte chunk per row, K == E
        (2, 1024, 24, 3, "softmax_renorm", None),
        (5, 2048, 128, 8, "softmax_renorm", None),
    ],
)
def test_router_of_a_few_tokens(gpu_device, tokens, d, e, k, mode, zipf):
    """The token counts of a decode step at the model and expert counts of the known layers:
    against the oracle, and with the normalisation in front."""
    _say("router, few tokens", tokens, d, e, k, mode)
    spec = W.small_spec(tokens=tokens, model_dim=d, num_experts=e, top_k=k, inner_dim=8, dtype="bf16",
                        zipf_s=zipf, mode=MODES[mode], seed=tokens + d)
    wl = W.make_workload_from_spec(spec, with_weights=False)
    logits, idx, w = oracle_routing(wl)
    x = wl.x.reshape(-1, d).bfloat16().to(gpu_device)
    router = wl.router.bfloat16().to(gpu_device)
    bias = None if wl.router_bias is None else wl.router_bias.to(gpu_device)
    score = _abi.SCORE_SOFTMAX if "softmax" in mode else _abi.SCORE_SIGMOID
    gi, gw, gl = _abi.router_topk(x, router, bias, k, score, spec.mode.renormalize, want_logits=True)
    np.testing.assert_allclose(gl.cpu().double().numpy(), logits.numpy(), rtol=1e-5, atol=2e-5)
    assert torch.equal(gi.cpu().long(), idx), "selected experts differ from the oracle"
    np.testing.assert_allclose(gw.cpu().double().numpy(), w.numpy(), rtol=5e-5, atol=1e-6)
    # the normalisation in front: the rows, and the routing of those rows
    g = torch.Generator().manual_seed(d)
    gamma = (1.0 + 0.3 * torch.randn(d, generator=g)).bfloat16().to(gpu_device)
    xn, ni, nw, nl = _abi.router_topk_norm(x, gamma, 1e-5, router, bias, k, score,
                                           spec.mode.renormalize, want_logits=True)
    want = O.rms_norm(x.cpu(), gamma.cpu(), 1e-5).double()
    assert bool(((xn.cpu().double() - want).abs() <= 2.0 ** -7 * want.abs()).all())
    pi, pw, pl = _abi.router_topk(xn, router, bias, k, score, spec.mode.renormalize, want_logits=True)
    assert torch.equal(ni, pi) and torch.equal(nw, pw) and torch.equal(nl, pl)
    # up to 32 tokens the router's blocks normalise the columns they read; more tokens go through a
    # kernel in front: the same rows among 40 come out with the same bits
    many = torch.cat([x, x.flip(0).repeat(40, 1)[: 40 - tokens]])
    xn40 = _abi.router_topk_norm(many, gamma, 1e-5, router, bias, k, score, spec.mode.renormalize)[0]
    assert torch.equal(xn40[:tokens], xn)


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize(
    "tokens,d,e,k,with_weight",
    [
        (257, 256, 16, 4, True),    # a last block of one row (normalised by the kernel in front)
        (1500, 256, 16, 4, True),   # up to 4096 tokens a small kernel in front normalises the rows
        (1101, 2048, 128, 8, True),
        (1100, 100, 10, 2, True),
        (4100, 256, 16, 4, True),   # beyond 4096 tokens the MFMA routers normalise on the way
        (4133, 128, 8, 2, False),
        (4133, 100, 10, 2, True),   # ... and so does the FMA router
        (8192, 512, 128, 8, True),  # the prefill token count
        (64, 2048, 128, 8, True),   # the decode shape
        (100, 96, 24, 3, False),    # no elementwise weight
        (45, 100, 10, 2, True),     # D, E off the 16-byte grid: element-wise path, FMA router
        (1, 64, 8, 8, True),
    ],
)
def test_router_with_norm_in_front(gpu_device, dtype, tokens, d, e, k, with_weight):
    """fs2moe_router_topk_norm: the normalised rows against the oracle's rms_norm (the reduction
    order of the mean differs, so a value may land on the neighbouring number), and the routing bit
    for bit against the plain router run on those rows."""
    _say("router+norm", dtype, tokens, d, e, k, with_weight)
    td = TORCH_DTYPE[dtype]
    g = torch.Generator().manual_seed(tokens + d)
    x = (3.0 * torch.randn(tokens, d, generator=g) * torch.rand(tokens, 1, generator=g)).to(td)
    x[0] = 0.0  # a zero row: rsqrt(eps) stays finite and the row stays zero
    weight = (1.0 + 0.3 * torch.randn(d, generator=g)).to(td) if with_weight else None
    router = (0.2 * torch.randn(d, e, generator=g)).to(td)
    bias = 0.1 * torch.randn(e, generator=g)
    eps = 1e-5
    xd = x.to(gpu_device)
    xn, idx, w, logits = _abi.router_topk_norm(
        xd, None if weight is None else weight.to(gpu_device), eps, router.to(gpu_device),
        bias.to(gpu_device), k, _abi.SCORE_SOFTMAX, True, want_logits=True)
    idx2, w2, logits2 = _abi.router_topk(xn, router.to(gpu_device), bias.to(gpu_device), k,
                                         _abi.SCORE_SOFTMAX, True, want_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(xd, x.to(gpu_device)), "the input rows are left untouched"
    want = O.rms_norm(x, weight, eps)
    step = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -20
    got = xn.cpu().double()
    assert bool(((got - want.double()).abs() <= step * want.double().abs()).all())
    assert bool((got[0] == 0).all())
    if dtype == "bf16":
        assert (xn.cpu() == want).float().mean() > 0.98
    assert torch.equal(idx, idx2) and torch.equal(w, w2) and torch.equal(logits, logits2)


@pytest.mark.parametrize(
    "tokens,d,e,k,mode,zipf",
    [
        (8192, 2048, 128, 8, "softmax_renorm", 1.2),  # the benchmark's layer
        (33, 128, 8, 2, "reference", None),           # one step, a last block of one token
        (4100, 256, 16, 4, "softmax_plain", None),
        (4200, 1024, 256, 16, "sigmoid_renorm", 1.0),  # two expert fragments per wave
        (4130, 384, 136, 3, "softmax_renorm", None),   # experts off the fragment size
        (5000, 5120, 16, 1, "reference", None),
    ],
)
def test_router_reading_an_expert_major_matrix(gpu_device, tokens, d, e, k, mode, zipf):
    """The router given its matrix as (E, D) (ROUTER_OUT_IN): the same selection as the oracle's,
    logits equal up to summation order, with exact ties, and with the
    normalisation in front bit for bit what the plain call makes of the normalised rows."""
    _say("router (E, D)", tokens, d, e, k, mode)
    lib = _abi.load()
    assert lib.fs2moe_router_takes_out_in(tokens, d, e, _abi.dtype_code(torch.bfloat16)) == 1
    assert lib.fs2moe_router_takes_out_in(tokens, d, e, _abi.dtype_code(torch.float32)) == 0
    assert lib.fs2moe_router_takes_out_in(32, d, e, _abi.dtype_code(torch.bfloat16)) == 0
    # few tokens of a wide model: several blocks share a token tile, and those kernels read (D, E)
    assert lib.fs2moe_router_takes_out_in(64, 2048, 128, _abi.dtype_code(torch.bfloat16)) == 0
    assert lib.fs2moe_router_takes_out_in(tokens, d + 8, e, _abi.dtype_code(torch.bfloat16)) == 0
    spec = W.small_spec(tokens=tokens, model_dim=d, num_experts=e, top_k=k, inner_dim=8, dtype="bf16",
                        zipf_s=zipf, mode=MODES[mode], seed=tokens + e)
    wl = W.make_workload_from_spec(spec, with_weights=False)
    logits, idx, w = oracle_routing(wl)
    x = wl.x.reshape(-1, d).bfloat16().to(gpu_device)
    router = wl.router.bfloat16().to(gpu_device)
    router_t = router.t().contiguous()
    bias = None if wl.router_bias is None else wl.router_bias.to(gpu_device)
    score = _abi.SCORE_SOFTMAX if "softmax" in mode else _abi.SCORE_SIGMOID
    gi, gw, gl = _abi.router_topk(x, router, bias, k, score, spec.mode.renormalize, want_logits=True,
                                  router_t=router_t)
    np.testing.assert_allclose(gl.cpu().double().numpy(), logits.numpy(), rtol=1e-5, atol=2e-5)
    assert torch.equal(gi.cpu().long(), idx), "selected experts differ from the oracle"
    np.testing.assert_allclose(gw.cpu().double().numpy(), w.numpy(), rtol=5e-5, atol=1e-6)
    # the (D, E) form of the same call: the same experts; logits up to the order of the sums
    pi, pw, pl = _abi.router_topk(x, router, bias, k, score, spec.mode.renormalize, want_logits=True)
    assert torch.equal(pi, gi)
    np.testing.assert_allclose(gl.cpu().numpy(), pl.cpu().numpy(), rtol=1e-5, atol=2e-5)
    # with the normalisation in front
    g = torch.Generator().manual_seed(d)
    gamma = (1.0 + 0.3 * torch.randn(d, generator=g)).bfloat16().to(gpu_device)
    xn, ni, nw, nl = _abi.router_topk_norm(x, gamma, 1e-5, router, bias, k, score, spec.mode.renormalize,
                                           want_logits=True, router_t=router_t)
    xn2 = _abi.router_topk_norm(x, gamma, 1e-5, router, bias, k, score, spec.mode.renormalize)[0]
    assert torch.equal(xn, xn2), "the normalised rows do not depend on the router's layout"
    qi, qw, ql = _abi.router_topk(xn, router, bias, k, score, spec.mode.renormalize, want_logits=True,
                                  router_t=router_t)
    assert torch.equal(ni, qi) and torch.equal(nw, qw) and torch.equal(nl, ql)
    # exact ties and special values: small integers make every sum exact
    gi2 = torch.Generator().manual_seed(7)
    xi = torch.randint(-2, 3, (tokens, d), generator=gi2).float()
    ri = torch.randint(-1, 2, (d, e), generator=gi2).float()
    xi[0] = 0.0
    if e > 7:
        ri[:, 7] = ri[:, 3]
    want = xi.double() @ ri.double()
    ti, _, tl = _abi.router_topk(xi.bfloat16().to(gpu_device), ri.bfloat16().to(gpu_device), None, k,
                                 want_logits=True, router_t=ri.t().contiguous().bfloat16().to(gpu_device))
    assert torch.equal(tl.cpu().double(), want)
    assert torch.equal(ti.cpu().long(), O.topk_lowest_index(want, k))


def test_router_refuses_an_expert_major_matrix_where_it_does_not_read_one(gpu_device):
    x = torch.zeros(16, 64, dtype=torch.bfloat16, device=gpu_device)
    r = torch.zeros(8, 64, dtype=torch.bfloat16, device=gpu_device)
    idx = torch.empty(16, 2, dtype=torch.int32, device=gpu_device)
    w = torch.empty(16, 2, dtype=torch.float32, device=gpu_device)
    lib = _abi.load()
    rc = lib.fs2moe_router_topk(x.data_ptr(), r.data_ptr(), None, 16, 64, 8, 2, _abi.dtype_code(x.dtype),
                                _abi.SCORE_SIGMOID | _abi.ROUTER_OUT_IN, 0, idx.data_ptr(), w.data_ptr(),
                                None, None, 0, None)
    assert rc != 0 and b"fs2moe_router_takes_out_in" in lib.fs2moe_last_error()


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
def test_router_ties_resolve_to_lower_expert_id(gpu_device, dtype):
    # Small-integer operands: every partial sum is exact in f32 whatever the order, so exact ties
    # are common and the tie rule is the only thing that decides.
    g = torch.Generator().manual_seed(5)
    t, d, e, k = 512, 64, 24, 6
    x = torch.randint(-2, 3, (t, d), generator=g).float()
    r = torch.randint(-1, 2, (d, e), generator=g).float()
    x[0] = 0.0  # all logits zero: selects experts 0..k-1
    r[:, 7] = r[:, 3]  # two identical experts
    logits = x.double() @ r.double()
    idx = O.topk_lowest_index(logits, k)
    assert idx[0].tolist() == list(range(k))
    dt = TORCH_DTYPE[dtype]
    gi, gw, gl = _abi.router_topk(x.to(dt).to(gpu_device), r.to(dt).to(gpu_device), None, k, want_logits=True)
    assert torch.equal(gl.cpu().double(), logits)
    assert torch.equal(gi.cpu().long(), idx)
    # every selection is sorted by (descending logit, ascending id)
    sel = torch.gather(logits, 1, gi.cpu().long())
    assert bool(((sel[:, :-1] > sel[:, 1:]) | ((sel[:, :-1] == sel[:, 1:]) & (gi.cpu()[:, :-1] < gi.cpu()[:, 1:]))).all())


def test_router_nan_and_inf_order(gpu_device):
    # NaN ranks above +inf (as torch.topk does), -0.0 ties with +0.0.
    d, e = 8, 6
    r = torch.zeros(d, e)
    r[0] = torch.tensor([1.0, -1.0, 0.0, 2.0, 0.5, -0.0])
    x = torch.zeros(4, d)
    x[0, 0] = float("inf")  # logits: inf, -inf, nan, inf, inf, nan
    x[1, 0] = 1.0  # 1, -1, 0, 2, .5, -0
    x[2, 0] = float("nan")  # all nan
    x[3, 0] = -1.0  # -1, 1, -0, -2, -.5, 0
    logits = x @ r
    want = O.topk_lowest_index(logits, 4)
    assert want.tolist() == [[2, 5, 0, 3], [3, 0, 4, 2], [0, 1, 2, 3], [1, 2, 5, 4]]
    gi, _, _ = _abi.router_topk(x.to(gpu_device), r.to(gpu_device), None, 4)
    assert gi.cpu().tolist() == want.tolist()


# ---------------------------------------------------------------------------------------- dispatch
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("tile_m", [1, 16, 128])
@pytest.mark.parametrize("scale_input", [False, True])
def test_dispatch_matches_oracle(gpu_device, dtype, tile_m, scale_input):
    _say("dispatch", dtype, tile_m, scale_input)
    t, d, e, k = 1500, 128, 40, 4
    spec = W.small_spec(tokens=t, model_dim=d, num_experts=e, top_k=k, inner_dim=8, dtype=dtype, zipf_s=1.2, seed=9)
    wl = W.make_workload_from_spec(spec, with_weights=False)
    _, idx, w = oracle_routing(wl)
    r = O.route(idx, e, tile_m)
    assert (r.counts == 0).any(), "the case should contain an expert without tokens"
    dt = TORCH_DTYPE[dtype]
    x = wl.x.reshape(t, d).to(dt).to(gpu_device)
    gi = idx.to(torch.int32).to(gpu_device)
    gw = w.float().to(gpu_device)
    disp = _abi.dispatch(gi, gw, x, e, tile_m, scale_input)
    np.testing.assert_array_equal(disp.counts.cpu().numpy(), r.counts)
    np.testing.assert_array_equal(disp.offsets.cpu().numpy(), r.offsets)
    perm = disp.perm.cpu().numpy()
    np.testing.assert_array_equal(perm[: r.num_rows], r.perm)
    assert (perm[r.num_rows:] == -1).all()
    np.testing.assert_array_equal(disp.inv_perm.cpu().numpy(), r.inv_perm)
    # gathered rows: exact copies (or the f32 product rounded once), zeros on padding rows
    xe = disp.xe[: r.num_rows].float().cpu()
    xs = x.float().cpu()
    want = torch.zeros(r.num_rows, d)
    rows = torch.from_numpy(r.inv_perm.astype(np.int64))
    for s in range(k):
        src = xs * gw.cpu()[:, s : s + 1] if scale_input else xs
        want[rows[:, s]] = src.to(dt).float()
    assert torch.equal(xe, want)


@pytest.mark.parametrize("tokens,e,k", [(1, 8, 2), (200, 256, 16), (256, 128, 8), (257, 128, 8), (700, 24, 4),
                                        (5000, 40, 3), (1100, 384, 24), (16384, 8, 1), (16500, 16, 2)])
def test_dispatch_without_row_copy_matches_oracle(gpu_device, tokens, e, k):
    # at most 256 tokens take the one-kernel path; up to 64 counting blocks (16384 tokens) two kernels,
    # the second doing the scan in every block (with top-3 its blocks of 256 pairs straddle counting
    # blocks); more the three-kernel path: same artefacts
    _say("dispatch index only", tokens, e, k)
    spec = W.small_spec(tokens=tokens, model_dim=64, num_experts=e, top_k=k, inner_dim=8, dtype="bf16",
                        zipf_s=1.1, seed=tokens + e)
    wl = W.make_workload_from_spec(spec, with_weights=False)
    _, idx, w = oracle_routing(wl)
    for tile_m in (1, 16):
        r = O.route(idx.numpy(), e, tile_m)
        x = wl.x.reshape(-1, 64).to(torch.bfloat16).to(gpu_device)
        disp = _abi.dispatch(idx.to(torch.int32).to(gpu_device), w.float().to(gpu_device), x, e, tile_m, False, gather=False)
        assert disp.xe is None
        assert_routing_equal(idx.to(torch.int32), disp, r, f"T={tokens} tile_m={tile_m}")


def test_dispatch_single_token_and_all_to_one(gpu_device):
    # T = 1 and "every token picks the same experts" (maximum collision on the histogram)
    for t in (1, 700):
        idx = torch.tensor([[3, 0]], dtype=torch.int32).repeat(t, 1)
        x = torch.randn(t, 64, generator=torch.Generator().manual_seed(t))
        r = O.route(idx, 5, 16)
        disp = _abi.dispatch(idx.to(gpu_device), None, x.to(gpu_device), 5, 16, False)
        assert disp.counts.cpu().tolist() == [t, 0, 0, t, 0]
        np.testing.assert_array_equal(disp.inv_perm.cpu().numpy(), r.inv_perm)
        np.testing.assert_array_equal(disp.perm.cpu().numpy()[: r.num_rows], r.perm)
        assert torch.equal(disp.xe[r.inv_perm[:, 0].astype(np.int64)].cpu(), x)


# ----------------------------------------------------------------------------------------- experts
def _expert_case(dtype, rows_per_expert, d, f, seed):
    g = torch.Generator().manual_seed(seed)
    e = len(rows_per_expert)
    dt = TORCH_DTYPE[dtype]
    rnd = lambda *s: (torch.randn(*s, generator=g)).to(dt).float()
    counts = torch.tensor(rows_per_expert, dtype=torch.int32)
    tile_m = 16
    padded = (counts + tile_m - 1) // tile_m * tile_m
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.cumsum(padded, 0)
    rows = int(offsets[-1])
    xe = rnd(rows, d)
    wg, wu, wd = 0.05 * rnd(e * d, f), 0.05 * rnd(e * d, f), 0.05 * rnd(e * f, d)
    wg, wu, wd = (t.to(dt).float() for t in (wg, wu, wd))
    return counts, offsets, xe, wg, wu, wd


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize(
    "rows_per_expert,d,f",
    [
        ([5, 0, 130, 64, 1, 300], 128, 256),  # ragged, empty expert, several m-tiles
        ([40, 17], 72, 40),  # dims that are not multiples of the tile sizes
        ([128] * 4, 256, 128),  # exact tiles
        ([3] * 32, 64, 64),  # many tiny experts
        ([(5 * i) % 7 for i in range(256)], 64, 64),  # the largest expert count the library takes
        # more tiles than compute units (every persistent block walks several, heavy and light mixed)
        ([(37 * i * i + 11 * i) % 701 for i in range(72)], 128, 384),
    ],
)
def test_grouped_swiglu_matches_oracle(gpu_device, dtype, rows_per_expert, d, f):
    _say("grouped_swiglu", dtype, rows_per_expert[:6], d, f)
    counts, offsets, xe, wg, wu, wd = _expert_case(dtype, rows_per_expert, d, f, seed=d + f)
    e = len(rows_per_expert)
    dt = TORCH_DTYPE[dtype]
    dev = gpu_device
    ye, h = _abi.grouped_swiglu(
        xe.to(dt).to(dev), counts.to(dev), offsets.to(dev), wg.to(dt).to(dev), wu.to(dt).to(dev), wd.to(dt).to(dev), e
    )
    for ex in range(e):
        lo, n = int(offsets[ex]), int(counts[ex])
        if n == 0:
            continue
        u = xe[lo : lo + n].double()
        h_ref = torch.nn.functional.silu(u @ wg[ex * d : (ex + 1) * d].double()) * (u @ wu[ex * d : (ex + 1) * d].double())
        assert_output_close(h[lo : lo + n], h_ref, dtype, f"h of expert {ex}")
        # second GEMM checked from the device's own (rounded) h, so its error is isolated
        y_ref = h[lo : lo + n].double().cpu() @ wd[ex * f : (ex + 1) * f].double()
        assert_output_close(ye[lo : lo + n], y_ref, dtype, f"ye of expert {ex}")
        y_full = O.glu_expert(u, wg[ex * d : (ex + 1) * d].double(), wu[ex * d : (ex + 1) * d].double(), wd[ex * f : (ex + 1) * f].double())
        assert_output_close(ye[lo : lo + n], y_full, dtype, f"expert {ex}")


@pytest.mark.parametrize(
    "bound,rows_per_expert,d,f",
    [
        (1, [1, 0, 1, 1, 0, 0, 1, 1], 2048, 768),   # one decoding sequence at the Qwen3 shape
        (1, [1, 1], 72, 40),                          # K not a multiple of the 128 rows a step takes
        (2, [2, 0, 1, 2], 256, 136),
        (4, [3, 4, 0, 1, 4, 2], 128, 200),
        (8, [8, 5, 0, 7, 1, 8, 3], 320, 192),
        (8, [(3 * i) % 9 for i in range(128)], 64, 64),
        (4, [9, 4, 13, 0, 1], 128, 64),               # counts above the bound: walked again, still right
        (4, [4, 2], 8192, 64),
        (4, [4, 1], 18432, 64),                       # the longest K whose four rows fit LDS
        (1, [1, 0, 1], 128, 4096),                    # a long inner dimension: the second product keeps
        (2, [2, 1, 0, 2], 64, 4352),                  # eight steps of loads in flight (4352: 17 steps)
        # 5 to 16 rows: the same stream with the arithmetic on the matrix pipe
        (16, [16, 9, 0, 12, 1, 5], 2048, 768),       # the Qwen3 shape
        (12, [12, 3, 7], 72, 40),                     # K and N off the kernel's steps
        (5, [5, 0, 2, 5], 256, 136),
        (16, [16, 2], 5112, 64),                      # the longest K whose sixteen rows fit LDS
        (8, [8, 1], 8192, 64),                        # eight rows staged
        (16, [16, 2, 9], 8192, 64),                   # sixteen such rows do not fit: eight at a time
        (8, [20, 8, 9], 128, 136),                    # counts above the bound
        (16, [33, 16, 0, 17], 64, 200),
    ],
)
def test_grouped_swiglu_with_a_bound_on_the_rows_per_expert(gpu_device, bound, rows_per_expert, d, f):
    """``fs2moe_grouped_swiglu_rows``: with a bound of 1..4 rows per expert and bf16 weights the two
    products stream the weights through the vector ALUs, with 5..16 through the matrix pipe (larger
    bounds take the GEMM kernels).  Each expert against the oracle's SwiGLU in f64; rows read
    through a map give the same bits."""
    _say("grouped_swiglu_rows", bound, rows_per_expert[:8], d, f)
    counts, offsets, xe, wg, wu, wd = _expert_case("bf16", rows_per_expert, d, f, seed=bound + d + f)
    e = len(rows_per_expert)
    dev = gpu_device
    bf = torch.bfloat16
    args = (counts.to(dev), offsets.to(dev), wg.to(bf).to(dev), wu.to(bf).to(dev), wd.to(bf).to(dev), e)
    ye, h = _abi.grouped_swiglu(xe.to(bf).to(dev), *args, rows_per_expert=bound)
    for ex in range(e):
        lo, n = int(offsets[ex]), int(counts[ex])
        if n == 0:
            continue
        u = xe[lo : lo + n].double()
        h_ref = torch.nn.functional.silu(u @ wg[ex * d : (ex + 1) * d].double()) * (u @ wu[ex * d : (ex + 1) * d].double())
        assert_output_close(h[lo : lo + n], h_ref, "bf16", f"h of expert {ex}")
        y_ref = h[lo : lo + n].double().cpu() @ wd[ex * f : (ex + 1) * f].double()
        assert_output_close(ye[lo : lo + n], y_ref, "bf16", f"ye of expert {ex}")
        y_full = O.glu_expert(u, wg[ex * d : (ex + 1) * d].double(), wu[ex * d : (ex + 1) * d].double(), wd[ex * f : (ex + 1) * f].double())
        assert_output_close(ye[lo : lo + n], y_full, "bf16", f"expert {ex}")
    # through a row map: rows scattered over a larger matrix, same bits
    total = xe.shape[0]
    g = torch.Generator().manual_seed(5)
    src_rows = torch.randperm(total + 11, generator=g)[:total]
    src = torch.randn(total + 11, d, generator=g).to(bf)
    src[src_rows] = xe.to(bf)
    ye2, h2 = _abi.grouped_swiglu(src.to(dev), *args, row_map=src_rows.to(torch.int32).to(dev), rows_per_expert=bound)
    for ex in range(e):
        lo, n = int(offsets[ex]), int(counts[ex])
        assert torch.equal(ye2[lo : lo + n], ye[lo : lo + n]) and torch.equal(h2[lo : lo + n], h[lo : lo + n])
    # bounds outside 1..16 take the other kernels; a negative bound is refused
    ye3, _ = _abi.grouped_swiglu(xe.to(bf).to(dev), *args, rows_per_expert=17)
    ye4, _ = _abi.grouped_swiglu(xe.to(bf).to(dev), *args)
    for ex in range(e):
        lo, n = int(offsets[ex]), int(counts[ex])
        assert torch.equal(ye3[lo : lo + n], ye4[lo : lo + n])
    with pytest.raises(_abi.Fs2MoeError, match="rows_per_expert"):
        _abi.grouped_swiglu(xe.to(bf).to(dev), *args, rows_per_expert=-1)


def test_grouped_swiglu_row_map_equals_gathered_rows(gpu_device):
    """Reading the rows through dispatch's permutation gives bit for bit what the gathered copy gives."""
    _say("grouped_swiglu row_map")
    t, d, e, k, f = 1500, 128, 24, 4, 192
    spec = W.small_spec(tokens=t, model_dim=d, num_experts=e, top_k=k, inner_dim=f, dtype="bf16", zipf_s=1.2, seed=13)
    wl = W.make_workload_from_spec(spec)
    _, idx, w = oracle_routing(wl)
    dev = gpu_device
    assert _abi.fuses_gather(d, f, torch.bfloat16, torch.bfloat16)
    assert not _abi.fuses_gather(d, f, torch.float32, torch.float32)
    x = wl.x.reshape(-1, d).to(torch.bfloat16).to(dev)
    idx_d, w_d = idx.to(torch.int32).to(dev), w.float().to(dev)
    gathered = _abi.dispatch(idx_d, w_d, x, e, 16, False)
    bare = _abi.dispatch(idx_d, w_d, x, e, 16, False, gather=False)
    assert bare.xe is None and torch.equal(bare.perm, gathered.perm)
    weights = [v.to(torch.bfloat16).to(dev) for v in (wl.gate, wl.up, wl.down)]
    ye_a, h_a = _abi.grouped_swiglu(gathered.xe, gathered.counts, gathered.offsets, *weights, e)
    ye_b, h_b = _abi.grouped_swiglu(x, bare.counts, bare.offsets, *weights, e, row_map=bare.perm)
    valid = (gathered.perm >= 0)
    assert torch.equal(h_a[valid], h_b[valid])
    assert torch.equal(ye_a[valid], ye_b[valid])
    # where the library has no fused path it says so instead of reading garbage
    with pytest.raises(_abi.Fs2MoeError):
        _abi.grouped_swiglu(x.float(), bare.counts, bare.offsets, *(v.float() for v in weights), e, row_map=bare.perm)


def test_grouped_swiglu_beyond_4_gb_of_activations(gpu_device):
    """Rows whose byte offset does not fit 32 bits: the throughput kernel (32-bit offsets) steps
    aside for the general one, and a row map is refused rather than mis-read."""
    _say("grouped_swiglu > 4 GB")
    d, f, e = 2048, 128, 2
    far = 1_090_000  # rows; far * d * 2 bytes = 4.46 GB
    counts = torch.tensor([100, 60], dtype=torch.int32)
    offsets = torch.tensor([0, far, far + 64], dtype=torch.int32)
    g = torch.Generator().manual_seed(9)
    bf = lambda t: t.to(torch.bfloat16)  # noqa: E731
    wg, wu = bf(0.02 * torch.randn(e * d, f, generator=g)), bf(0.02 * torch.randn(e * d, f, generator=g))
    wd = bf(0.02 * torch.randn(e * f, d, generator=g))
    rows = {0: bf(torch.randn(100, d, generator=g)), 1: bf(torch.randn(60, d, generator=g))}
    dev = gpu_device
    xe = torch.empty((far + 64, d), dtype=torch.bfloat16, device=dev)
    xe[:100] = rows[0].to(dev)
    xe[far : far + 60] = rows[1].to(dev)
    ye, h = _abi.grouped_swiglu(xe, counts.to(dev), offsets.to(dev), wg.to(dev), wu.to(dev), wd.to(dev), e)
    for ex, lo in ((0, 0), (1, far)):
        u = rows[ex].double()
        ref = O.glu_expert(u, wg[ex * d : (ex + 1) * d].double(), wu[ex * d : (ex + 1) * d].double(), wd[ex * f : (ex + 1) * f].double())
        assert_output_close(ye[lo : lo + u.shape[0]], ref, "bf16", f"expert {ex}")
    row_map = torch.zeros(far + 64, dtype=torch.int32, device=dev)
    with pytest.raises(_abi.Fs2MoeError, match="4 GB"):
        _abi.grouped_swiglu(xe, counts.to(dev), offsets.to(dev), wg.to(dev), wu.to(dev), wd.to(dev), e, row_map=row_map)


@pytest.mark.parametrize("t,d,e,k,f", [(48, 128, 16, 4, 64), (700, 128, 4, 2, 192)])  # decode / throughput kernel
def test_grouped_swiglu_fp8_row_map_equals_gathered_rows(gpu_device, t, d, e, k, f):
    """The e4m3-weight kernels read rows through the permutation too, with identical results."""
    _say("grouped_swiglu fp8 row_map", t, d, e, k, f)
    spec = W.small_spec(tokens=t, model_dim=d, num_experts=e, top_k=k, inner_dim=f, dtype="bf16",
                        weight_dtype="fp8", zipf_s=1.2, seed=17)
    wl = W.make_workload_from_spec(spec)
    _, idx, w = oracle_routing(wl)
    dev = gpu_device
    assert _abi.fuses_gather(d, f, torch.bfloat16, torch.float8_e4m3fn)
    x = wl.x.reshape(-1, d).to(torch.bfloat16).to(dev)
    idx_d, w_d = idx.to(torch.int32).to(dev), w.float().to(dev)
    gathered = _abi.dispatch(idx_d, w_d, x, e, 16, False)
    bare = _abi.dispatch(idx_d, w_d, x, e, 16, False, gather=False)
    packed = [_abi.pack_fp8_weights(wl.fp8[n + "_q"], e).to(dev) for n in ("gate", "up", "down")]
    scales = tuple(wl.fp8[n + "_scale"].to(dev) for n in ("gate", "up", "down"))
    ye_a, h_a = _abi.grouped_swiglu(gathered.xe, gathered.counts, gathered.offsets, *packed, e, scales=scales)
    ye_b, h_b = _abi.grouped_swiglu(x, bare.counts, bare.offsets, *packed, e, scales=scales, row_map=bare.perm)
    valid = gathered.perm >= 0
    assert int(valid.sum()) == t * k
    assert torch.equal(h_a[valid], h_b[valid])
    assert torch.equal(ye_a[valid], ye_b[valid])


@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize(
    "t,d,f",
    [
        (200, 128, 256), (37, 72, 40), (1, 64, 64), (600, 192, 320),
        # up to 16 bf16 rows stream the weights (K off the 32-wide steps, N off the 16-channel blocks)
        (1, 5120, 1024), (3, 72, 40), (8, 2048, 768), (16, 1000, 200), (16, 8, 8), (17, 256, 128),
    ],
)
def test_dense_swiglu_matches_oracle(gpu_device, dtype, t, d, f):
    _say("dense_swiglu", dtype, t, d, f)
    g = torch.Generator().manual_seed(t)
    dt = TORCH_DTYPE[dtype]
    x = torch.randn(t, d, generator=g).to(dt).float()
    wg, wu, wd = (0.05 * torch.randn(*s, generator=g) for s in ((f, d), (f, d), (d, f)))
    wg, wu, wd = (w.to(dt).float() for w in (wg, wu, wd))
    y = _abi.dense_swiglu(*(v.to(dt).to(gpu_device) for v in (x, wg, wu, wd)))
    ref = O.shared_glu(x.double(), wg.double(), wu.double(), wd.double())
    assert_output_close(y, ref, dtype, "shared expert")


@pytest.mark.parametrize(
    "rows,d,f,experts",
    [
        # tiles of 256 rows x 256 channels on 256 blocks.  Down projection (1 channel tile): 258 row
        # tiles, the last of 208 rows: the two left over by the one whole round go out as halves,
        # the second half of the last one 80 rows; gate/up (2 channel tiles): 516 tiles, 4 left over
        (66000, 256, 256, 1),
        # two experts of 198 + 99 row tiles (the last of each partly filled): 41 left over, as halves
        (76000, 256, 128, 2),
        # 384 + 1 tiles: 129 left over would be 258 halves, one too many: dealt whole
        (98560, 256, 128, 1),
    ],
)
def test_tiles_around_the_last_round_of_the_deal(gpu_device, rows, d, f, experts):
    """The throughput kernel deals its tiles round-robin to one block per CU and splits the heavy
    tiles that do not fill a round into halves when they then fit one round: shapes on both sides of
    that rule, the grouped experts reading their rows through a map and the dense network, checked
    on sampled rows (every row depends on its own tile only)."""
    _say("last round of the deal", rows, d, f, experts)
    g = torch.Generator().manual_seed(rows)
    dev = gpu_device
    tokens = 4096
    x = torch.randn(tokens, d, generator=g).to(torch.bfloat16)
    row_map = torch.randint(0, tokens, (rows,), generator=g, dtype=torch.int32)
    first = rows * 2 // 3 if experts == 2 else rows
    counts = torch.tensor([first, rows - first][:experts], dtype=torch.int32)
    offsets = torch.tensor([0, first, rows][: experts + 1], dtype=torch.int32)
    wg, wu = (0.05 * torch.randn(experts * d, f, generator=g) for _ in range(2))
    wd = 0.05 * torch.randn(experts * f, d, generator=g)
    wg, wu, wd = (w.to(torch.bfloat16) for w in (wg, wu, wd))
    ye, _ = _abi.grouped_swiglu(x.to(dev), counts.to(dev), offsets.to(dev), wg.to(dev), wu.to(dev), wd.to(dev),
                                experts, row_map=row_map.to(dev))
    torch.cuda.synchronize()
    # the first and last rows of every tile boundary region, and a random sample
    pick = torch.cat([torch.arange(0, 3), torch.arange(rows - 400, rows), torch.arange(first - 200, min(first + 200, rows)),
                      torch.randint(0, rows, (300,), generator=g)]).unique()
    got = ye[pick.to(dev)]
    for e in range(experts):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        sel = (pick >= lo) & (pick < hi)
        if not bool(sel.any()):
            continue
        xr = x[row_map[pick[sel]].long()].double()
        ref = O.glu_expert(xr, wg[e * d : (e + 1) * d].double(), wu[e * d : (e + 1) * d].double(),
                           wd[e * f : (e + 1) * f].double())
        assert_output_close(got[sel.to(dev)], ref, "bf16", f"expert {e}")
    if experts == 1:
        # the same rows through the dense network (nn.Linear-oriented weights, no map)
        xs = x[row_map.long()].contiguous()
        y = _abi.dense_swiglu(xs.to(dev), wg.t().contiguous().to(dev), wu.t().contiguous().to(dev),
                              wd.t().contiguous().to(dev))
        ref = O.shared_glu(xs[pick].double(), wg.t().double(), wu.t().double(), wd.t().double())
        assert_output_close(y[pick.to(dev)], ref, "bf16", "dense network")


# ----------------------------------------------------------------------------------------- combine
@pytest.mark.parametrize("dtype", ["bf16", "fp32"])
@pytest.mark.parametrize("weight_output", [False, True])
@pytest.mark.parametrize("with_base", [False, True])
@pytest.mark.parametrize("k", [4, 3, 7, 12])  # also values below the kernel's compile-time bounds 4, 8, 16
def test_combine_matches_oracle(gpu_device, dtype, weight_output, with_base, k):
    _say("combine", dtype, weight_output, with_base, k)
    g = torch.Generator().manual_seed(21)
    t, d, e = 777, 128, 12
    dt = TORCH_DTYPE[dtype]
    logits = torch.randn(t, e, generator=g)
    idx = O.topk_lowest_index(logits, k)
    w = O.combine_weights(logits, idx, "softmax", True).float()
    r = O.route(idx, e, 16)
    ye = torch.randn(r.num_rows, d, generator=g).to(dt).float()
    base = torch.randn(t, d, generator=g).to(dt).float() if with_base else None
    dev = gpu_device
    out = _abi.combine(
        ye.to(dt).to(dev), torch.from_numpy(r.inv_perm).to(dev), idx.to(torch.int32).to(dev), w.to(dev),
        None if base is None else base.to(dt).to(dev), weight_output,
    )
    # f32 accumulation in ascending expert id from the base, one rounding at the end
    acc = base.clone() if with_base else torch.zeros(t, d)
    order = torch.argsort(idx, dim=1)
    rows = torch.from_numpy(r.inv_perm.astype(np.int64))
    for j in range(k):
        slot = order[:, j]
        y = ye[rows[torch.arange(t), slot]]
        if weight_output:
            acc = torch.addcmul(acc, y, w[torch.arange(t), slot][:, None]) if False else acc + w[torch.arange(t), slot][:, None] * y
        else:
            acc = acc + y
    want = acc.to(dt).float()
    got = out.float().cpu()
    if not weight_output:
        assert torch.equal(got, want), "unweighted combine must be bit-exact"
    else:
        # the device may fuse the multiply-add; allow one ulp of the output type
        assert_output_close(out, acc, dtype)
        assert float((got - want).abs().max()) <= float(want.abs().max()) * (2**-7 if dtype == "bf16" else 2**-22)


# ------------------------------------------------------------------------ experts, fp8 weights
@pytest.mark.parametrize(
    "rows_per_expert,d,f",
    [
        ([5, 0, 17, 64, 1, 11, 0, 33], 128, 192),  # decode-like: few rows, empty experts
        ([100, 3], 64, 64),  # more than 64 rows: weights re-streamed per 64-row chunk
        # 64 or more rows per expert on average: the throughput kernel (codes turned into bf16 on
        # the way to LDS, scales in its epilogue); ragged last tiles, an empty expert, F and D that
        # leave the last channel tile partly (192 = 128 + 64) or mostly (128 of 256) empty
        ([300, 0, 70, 513, 1, 129, 256, 40], 128, 192),
        ([700, 260], 64, 64),
        ([257, 255, 31, 1000], 320, 448),
    ],
)
def test_grouped_swiglu_fp8_weights_match_oracle(gpu_device, rows_per_expert, d, f):
    _say("grouped_swiglu fp8", rows_per_expert, d, f)
    counts, offsets, xe, wg, wu, wd = _expert_case("bf16", rows_per_expert, d, f, seed=3 * d + f)
    e = len(rows_per_expert)
    qs = [W.quantize_fp8_per_channel(w, e) for w in (wg, wu, wd)]
    deq = [W.dequantize_fp8_per_channel(q, s) for q, s in qs]
    dev = gpu_device

    def kernel_layout(q, k, n):  # (E*k, n) -> 1 KB tiles (E, n/16, k/64, 16, 64)
        packed = _abi.pack_fp8_weights(q, e)
        assert packed.shape == (e, n // 16, k // 64, 16, 64)
        # tile [t, c, b] row i, byte j is weight (in = 64 b + j, out = 16 c + i) of expert t
        ref = q.view(torch.uint8).view(e, k, n)
        pk = packed.view(torch.uint8)
        assert int(pk[e - 1, 1, 0, 3, 5]) == int(ref[e - 1, 5, 16 + 3])
        return packed.to(dev)

    ye, h = _abi.grouped_swiglu(
        xe.to(torch.bfloat16).to(dev), counts.to(dev), offsets.to(dev),
        kernel_layout(qs[0][0], d, f), kernel_layout(qs[1][0], d, f), kernel_layout(qs[2][0], f, d), e,
        scales=tuple(s.to(dev) for _, s in qs),
    )
    for ex in range(e):
        lo, n = int(offsets[ex]), int(counts[ex])
        if n == 0:
            continue
        u = xe[lo : lo + n].double()
        g_, u_, d_ = (deq[0][ex * d : (ex + 1) * d].double(), deq[1][ex * d : (ex + 1) * d].double(), deq[2][ex * f : (ex + 1) * f].double())
        h_ref = torch.nn.functional.silu(u @ g_) * (u @ u_)
        assert_output_close(h[lo : lo + n], h_ref, "bf16", f"h of expert {ex}")
        assert_output_close(ye[lo : lo + n], O.glu_expert(u, g_, u_, d_), "bf16", f"expert {ex}")

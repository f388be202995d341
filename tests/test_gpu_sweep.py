"""Seeded sweep over shapes, modes and options of the layer, against the oracle.

The hand-picked cases of the other GPU tests use round numbers; this one draws top-k values that
are not powers of two, expert counts off the fragment sizes, token counts either side of the block
sizes, every routing mode, the shared expert, e4m3 weights, tile sizes and the residual input, and
checks every case three ways: the single-call entry point equals the staged path bit for bit, the
routing artefacts equal the oracle's, and the output is within the dtype's tolerance.  A third of the
cases also run with the RMS normalisation in front: the normalised rows against the oracle's, and the
one-call form bit for bit against the layer run on those rows.
"""

import random

import pytest
import torch

from fairseq2_amd import _abi
import workloads as W
from oracle import moe_oracle as O
from tests._util import (
    TORCH_DTYPE, assert_output_close, assert_routing_equal, build_module, emulate_device_rounding, oracle_forward,
    oracle_routing, output_bound,
)

pytestmark = pytest.mark.gpu

MODES = [
    W.RoutingMode("sigmoid", False, "input"), W.RoutingMode("softmax", True, "output"),
    W.RoutingMode("softmax", False, "output"), W.RoutingMode("sigmoid", True, "input"),
]


def _draw(rng):
    dtype = rng.choice(["bf16", "bf16", "fp32"])
    wdt = "fp8" if (dtype == "bf16" and rng.random() < 0.3) else None
    e = rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 24, 32, 40, 64, 72, 128, 136, 200, 256, 264, 384, 500, 512])
    k = rng.randint(1, min(e, 32 if rng.random() < 0.25 else 16))
    t = rng.choice([1, 2, 7, 16, 17, 31, 32, 33, 64, 100, 255, 256, 257, 511, 600, 1100])
    aligned = wdt is not None or rng.random() < 0.7
    d = rng.choice([64, 128, 192, 256, 512]) if aligned else rng.choice([72, 136, 200])
    f = rng.choice([64, 128, 192, 320]) if aligned else rng.choice([40, 88, 264])
    return dict(
        dtype=dtype, wdt=wdt, e=e, k=k, t=t, d=d, f=f, mode=rng.choice(MODES), shared=rng.random() < 0.3,
        zipf=rng.choice([None, 1.0, 1.5]), tile_m=rng.choice([1, 3, 16, 100, 128, 1024]), res=rng.random() < 0.4,
    )


# Cases a draw is unlikely to produce, run in front of every seed's draws: every expert selected with
# sixteen scaled input rows per token and e4m3 weights (the most bf16 roundings per output element),
# and many experts with a top-k that is not a power of two at a tile size that pads heavily.
FIXED = [
    dict(dtype="bf16", wdt="fp8", e=16, k=16, t=1100, d=512, f=320, mode=MODES[0], shared=False, zipf=1.5,
         tile_m=1024, res=False),
    dict(dtype="fp32", wdt=None, e=128, k=8, t=1100, d=136, f=128, mode=MODES[1], shared=False, zipf=None,
         tile_m=3, res=False),
    dict(dtype="bf16", wdt=None, e=200, k=11, t=600, d=192, f=64, mode=MODES[3], shared=True, zipf=1.0,
         tile_m=100, res=True),
    # more experts and a larger top-k than any published layer (the reference takes any, moe.py:35-48):
    # past 256 experts the router runs on the vector ALUs and the stream kernels stand aside
    dict(dtype="bf16", wdt=None, e=384, k=24, t=600, d=256, f=128, mode=MODES[1], shared=False, zipf=1.0,
         tile_m=16, res=False),
    dict(dtype="bf16", wdt="fp8", e=512, k=32, t=257, d=128, f=192, mode=MODES[0], shared=True, zipf=None,
         tile_m=3, res=True),
    dict(dtype="fp32", wdt=None, e=300, k=17, t=7, d=72, f=40, mode=MODES[2], shared=False, zipf=1.5,
         tile_m=1, res=False),
    dict(dtype="bf16", wdt=None, e=500, k=20, t=9, d=256, f=128, mode=MODES[1], shared=False, zipf=None,
         tile_m=16, res=False),
]


class _RMSNorm:
    def __init__(self, weight, eps, dim):
        self.weight, self.bias, self.eps, self.normalized_shape = weight, None, eps, (dim,)


def _check_norm_in_front(m, c, dt, res, device, it):
    g = torch.Generator().manual_seed(7 * it + 1)
    raw = (2.0 * torch.randn(c["t"], c["d"], generator=g)).to(dt)
    gamma = (1.0 + 0.2 * torch.randn(c["d"], generator=g)).to(dt)
    norm = _RMSNorm(gamma.to(device), 1e-5, c["d"])
    raw_d = raw.to(device)
    with torch.no_grad():
        fused = m(raw_d, residual=res.view(raw.shape) if res is not None else None, norm=norm)
        xn = _abi.router_topk_norm(raw_d, norm.weight, norm.eps, m.router.detach(), m.router_bias, m.top_k)[0]
        two = m(xn, residual=res.view(raw.shape) if res is not None else None)
    torch.cuda.synchronize()
    assert torch.equal(fused, two), f"case {it}: norm in front differs from the layer on normalised rows"
    want = O.rms_norm(raw, gamma, 1e-5).double()
    step = 2.0 ** -7 if c["dtype"] == "bf16" else 2.0 ** -20
    assert bool(((xn.cpu().double() - want).abs() <= step * want.abs()).all()), f"case {it}: normalised rows"


# The k + 1 largest logits of a token are "well separated" when their gaps exceed the rounding of
# the device's f32 logits by a wide margin: then the ordered selection has one right answer and the
# device must give the oracle's.  Closer than that, the order (or the k-th expert) depends on the
# summation order of the matmul; the device's answer is then checked against ITS OWN logits through
# the host mirror of its selection rule, and against the oracle's logits up to this margin.
SEPARATION = 2e-5


def _check_routing(c, wl, x2d, m, gi, it):
    """Device indices: always the host mirror's on the device's logits, bit for bit; the oracle's own
    where the logits are well separated, else a valid top-k of the oracle's logits within SEPARATION.
    Returns the indices the expected output is evaluated with (the device's)."""
    score = _abi.SCORE_SOFTMAX if c["mode"].score_fn == "softmax" else _abi.SCORE_SIGMOID
    di, dw, dl = _abi.router_topk(x2d, m.router.detach(), m.router_bias, c["k"], score, c["mode"].renormalize,
                                  want_logits=True)
    torch.cuda.synchronize()
    assert torch.equal(di, gi.view(di.shape)), f"case {it}: the layer's routing differs from the router stage's"
    mi, mw = _abi.cpu_router_select(dl, c["k"], score, c["mode"].renormalize)
    assert torch.equal(mi, di.cpu()), f"case {it}: device selection differs from the host mirror on the device's logits"
    torch.testing.assert_close(dw.cpu(), mw, rtol=5e-5, atol=1e-6)
    logits, idx, _ = oracle_routing(wl)
    scale = max(1.0, float(logits.abs().max()))
    torch.testing.assert_close(dl.cpu().double(), logits, rtol=0, atol=(2e-5 if c["dtype"] == "fp32" else 2e-6) * scale)
    top = torch.sort(logits, dim=1, descending=True).values[:, : c["k"] + 1]
    separated = top.shape[1] < 2 or float((top[:, :-1] - top[:, 1:]).min()) >= SEPARATION
    dev_idx = di.cpu().long()
    if separated:
        assert torch.equal(dev_idx, idx), f"case {it}: selected experts differ from the oracle"
    else:
        # a valid ordered top-k up to the margin: descending, and nothing left out that is larger
        chosen = torch.gather(logits, 1, dev_idx)
        assert bool((chosen[:, :-1] - chosen[:, 1:] >= -SEPARATION).all()), f"case {it}: order"
        rest = logits.scatter(1, dev_idx, float("-inf")).max(dim=1).values
        assert bool((chosen[:, -1] >= rest - SEPARATION).all()), f"case {it}: a larger logit was left out"
        assert bool((torch.sort(dev_idx, dim=1).values[:, 1:] != torch.sort(dev_idx, dim=1).values[:, :-1]).all())
    return dev_idx, separated


def _explained_by_the_rounding_points(wl, c, idx, gw, res_c, single, want, atol_scale, it):
    """An element outside the element-wise bound is the kernel's doing or the number format's.  The
    same arithmetic on the CPU, in f32 with a bf16 rounding wherever the device (and the reference
    module run in bf16) rounds, tells which: a heavy-tailed gated product rounds with an absolute
    error that a pair of cancelling terms does not shrink, and an output element can then sit at
    1.0-1.1 of the bound in that evaluation as well (about one case in a thousand, all seen in the
    mode that scales the rows on the way in).  Accepted only if the device agrees with that
    evaluation everywhere, the elements over the bound are a handful, none beyond 1.25, and the
    CPU evaluation is out (or at the edge) at each of them too.  bf16 cases without a shared
    expert; anything else stays a failure."""
    emu = emulate_device_rounding(wl, idx, gw.cpu(), residual=res_c).double().reshape(want.shape)
    got = single.detach().double().cpu().reshape(want.shape)
    bound = output_bound(want, c["dtype"], atol_scale)
    over = (got - want).abs() > bound
    assert_output_close(single, emu, c["dtype"], f"case {it}: against the CPU evaluation with the device's roundings")
    assert int(over.sum()) <= max(1, over.numel() // 10000), f"case {it}: {int(over.sum())} elements over the bound"
    assert float(((got - want).abs() / bound).max()) <= 1.25, f"case {it}: beyond what the roundings explain"
    assert bool((((emu - want).abs() / bound)[over] >= 0.9).all()), (
        f"case {it}: over the bound where the CPU evaluation with the same roundings is inside it")
    print(f"  case {it}: {int(over.sum())} element(s) at up to {float(((got - want).abs() / bound).max()):.3f} of the "
          "bound, as in the CPU evaluation with the device's rounding points", flush=True)


# (seed 52 holds a case of the kind _explained_by_the_rounding_points is for)
@pytest.mark.parametrize("seed", [11, 12, 13, 52])
def test_seeded_sweep(gpu_device, seed):
    rng = random.Random(seed)
    near_ties = 0
    cases = list(FIXED) + [_draw(rng) for _ in range(40)]
    for it, c in enumerate(cases):
        print(f"sweep seed={seed} case={it} {c}", flush=True)
        spec = W.small_spec(
            tokens=c["t"], model_dim=c["d"], num_experts=c["e"], top_k=c["k"], inner_dim=c["f"], dtype=c["dtype"],
            weight_dtype=c["wdt"], zipf_s=c["zipf"], shared=c["shared"], mode=c["mode"], seed=100 * seed + it,
        )
        wl = W.make_workload_from_spec(spec)
        m = build_module(wl, gpu_device, c["tile_m"])
        dt = TORCH_DTYPE[c["dtype"]]
        x = wl.x.to(dt).to(gpu_device)
        res, res_c = None, None
        if c["res"]:
            g = torch.Generator().manual_seed(it)
            res_c = torch.randn(wl.x.shape, generator=g).to(dt)
            res = res_c.to(gpu_device)
        with torch.no_grad():
            single = m(x, residual=res)
            staged, gi, gw, disp = m.forward_with_routing(x)
            if res is not None:
                staged = m._stages(x.reshape(-1, c["d"]), res.reshape(-1, c["d"]))[0].view(x.shape)
        torch.cuda.synchronize()
        assert torch.equal(single, staged), f"case {it}: single call differs from the staged path"
        idx, separated = _check_routing(c, wl, x.reshape(-1, c["d"]), m, gi, it)
        near_ties += not separated
        ref = oracle_forward(wl, idx, c["tile_m"], dtype=torch.float64)
        want = ref.out if res_c is None else ref.out + res_c.double()
        assert_routing_equal(gi, disp, ref.routing, f"case {it}")
        # many terms, each rounded a fourth time on the way in: see tests/_util.py
        many_roundings = c["k"] >= 8 and c["mode"].scale_on == "input"
        atol_scale = 2.0 if many_roundings else 1.0
        try:
            assert_output_close(single, want, c["dtype"], f"case {it}", atol_scale=atol_scale)
        except AssertionError:
            if c["dtype"] != "bf16" or c["shared"]:
                raise
            _explained_by_the_rounding_points(wl, c, idx, gw, res_c, single, want, atol_scale, it)
        if random.Random(1000 * seed + it).random() < 0.35:
            _check_norm_in_front(m, c, dt, res, gpu_device, it)
    print(f"sweep seed={seed}: {len(cases)} cases, {near_ties} with near-ties resolved through the host mirror", flush=True)

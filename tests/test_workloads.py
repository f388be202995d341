"""The seeded workload generator: draw order, routing statistics, fp8 quantiser."""

import numpy as np
import pytest
import torch

import workloads as W
from oracle import moe_oracle as O


def _counts(name):
    wl = W.make_workload(name, with_weights=False)
    logits = O.router_logits(wl.x.double(), wl.router.double(), None if wl.router_bias is None else wl.router_bias.double())
    idx = O.topk_lowest_index(logits, wl.spec.top_k)
    srt, _ = torch.sort(logits, dim=1, descending=True)
    margin = float((srt[:, wl.spec.top_k - 1] - srt[:, wl.spec.top_k]).min())
    return O.route(idx, wl.spec.num_experts).counts, margin


# Five largest per-expert token counts and the smallest top-k margin of each seeded shape.  These
# depend on the draw order (x, router, perm, ...) and on the bias rule, so they fix both.
@pytest.mark.parametrize(
    "name,top5,extra",
    [
        ("small_fp32", [1068, 1067, 1031, 1029, 1025], dict(min=954)),
        ("mixtral_8x7b", [5481, 3412, 2257, 1664, 1309], dict(min=574)),
        ("qwen3_30b_a3b", [8138, 7691, 6939, 6074, 5198], dict(median=11, empty=17, le8=59)),
        ("llama4_scout", [552, 546, 538, 536, 534], dict(min=486)),
        ("qwen3_decode_fp8", [64, 60, 55, 47, 46], dict(active=44)),
        ("qwen3_decode_bf16_1", [1, 1, 1, 1, 1], dict(active=8)),
        ("qwen3_decode_bf16_8", [8, 8, 8, 6, 5], dict(active=20)),
    ],
)
def test_routing_statistics(name, top5, extra):
    counts, margin = _counts(name)
    spec = W.SPECS[name]
    assert int(counts.sum()) == spec.num_tokens * spec.top_k
    assert sorted(counts.tolist(), reverse=True)[:5] == top5
    if "min" in extra:
        assert int(counts.min()) == extra["min"]
    if "median" in extra:
        assert sorted(counts.tolist())[(len(counts) - 1) // 2] == extra["median"]  # lower median
    if "empty" in extra:
        assert int((counts == 0).sum()) == extra["empty"]
    if "le8" in extra:
        assert int((counts <= 8).sum()) == extra["le8"]
    if "active" in extra:
        assert int((counts > 0).sum()) == extra["active"]
    # far above the fp32 accumulation error of a D-term dot product of unit-scale values
    assert margin > 1e-5


def test_values_are_representable_in_the_declared_dtype():
    wl = W.make_workload_from_spec(W.small_spec(dtype="bf16", shared=True))
    for t in (wl.x, wl.router, wl.gate, wl.up, wl.down, wl.shared_gate, wl.shared_up, wl.shared_down):
        assert torch.equal(t, t.to(torch.bfloat16).float())
    assert wl.gate.shape == (8 * 64, 96) and wl.down.shape == (8 * 96, 64)
    assert wl.shared_gate.shape == (96, 64) and wl.shared_down.shape == (64, 96)


def test_zipf_bias_rule():
    perm = torch.tensor([2, 0, 3, 1])
    b = W.zipf_router_bias(4, 1.2, perm)
    want = np.zeros(4)
    for r, e in enumerate(perm.tolist()):
        want[e] = -1.2 * np.log(r + 1)
    np.testing.assert_allclose(b.numpy(), want, rtol=1e-6)
    assert b[2] == 0.0


def test_fp8_quantiser_per_output_channel():
    g = torch.Generator().manual_seed(0)
    e, k, n = 3, 32, 20
    w = 0.02 * torch.randn(e * k, n, generator=g)
    q, s = W.quantize_fp8_per_channel(w, e)
    assert q.dtype == torch.float8_e4m3fn and s.shape == (e, n)
    deq = W.dequantize_fp8_per_channel(q, s)
    assert torch.isfinite(deq).all()
    # the column maximum maps onto +-448 exactly
    assert torch.equal(q.view(e, k, n).float().abs().amax(1), torch.full((e, n), 448.0))
    # e4m3 has a 3-bit mantissa: relative error <= 2^-4 for normal values
    rel = (deq - w).abs() / w.abs().clamp_min(1e-12)
    big = w.view(e, k, n).abs() > s[:, None, :] * 2.0**-6  # normal range after scaling
    assert float(rel.view(e, k, n)[big].max()) <= 2.0**-4 + 1e-6
    assert float((deq - w).norm() / w.norm()) < 0.04


def test_fp8_workload_uses_dequantised_weights():
    wl = W.make_workload_from_spec(W.small_spec(weight_dtype="fp8"))
    assert set(wl.fp8) == {"gate_q", "gate_scale", "up_q", "up_scale", "down_q", "down_scale"}
    assert torch.equal(wl.gate, W.dequantize_fp8_per_channel(wl.fp8["gate_q"], wl.fp8["gate_scale"]))
    assert wl.fp8["down_scale"].shape == (8, 64)

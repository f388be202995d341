"""Writes the golden vectors of the MoE forward path (``tests/golden/*.npz``).

The reference holds no fixture for this path (its tests never call
``fairseq2.models.llama4.moe.MoE``), so the vectors come from this build's own
restatement of the reference: for every case the expected output is evaluated
in float64 with ``oracle.moe_oracle.ref_dense_forward``, which follows
``src/fairseq2/models/llama4/moe.py:102-157`` op for op (dense score matrix,
E-fold gather, three ``bmm``, ``scatter_add_``).  The tests then check two other
evaluations against the stored numbers: the per-expert formulation of the
oracle (CPU) and the HIP kernels (GPU).

Run from the repository root:  ``python tests/golden/make_fixtures.py``.
Files hold plain arrays only (``numpy.load`` with ``allow_pickle=False``):
fp32 inputs as float32, bf16 inputs as their 16-bit patterns (uint16), e4m3
weights as their codes (uint8) with float32 scales, expert selections as int32,
expected outputs as float64.  ``load_case`` below is the one reader.  The pre-norm case also
stores the raw rows and the norm's weight: its ``x`` is their RMS normalisation as the oracle
computes it, and its expected output includes the raw rows as the residual.
"""

from __future__ import annotations

import json
import sys
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))

import workloads as W  # noqa: E402
from oracle import moe_oracle as O  # noqa: E402

# name -> (spec keywords, number of leading tokens whose input row is zeroed: all their logits tie)
CASES = {
    # the reference's own mode: sigmoid of the selected logits, applied to the expert input
    "reference_mode_fp32": (dict(tokens=40, model_dim=64, num_experts=4, top_k=2, inner_dim=64,
                                 dtype="fp32", seed=101), 0),
    # bf16, every expert GEMM on the throughput kernel (D and F multiples of 64), exact ties
    "reference_mode_bf16_ties": (dict(tokens=48, model_dim=64, num_experts=8, top_k=2, inner_dim=128,
                                      dtype="bf16", seed=102), 3),
    # softmax over all experts, top-k renormalised, weights applied to the expert output, skewed
    # router bias (some experts receive no token)
    "softmax_renorm_bias_bf16": (dict(tokens=40, model_dim=64, num_experts=16, top_k=4, inner_dim=64,
                                      dtype="bf16", seed=103, zipf_s=1.2,
                                      mode=W.RoutingMode("softmax", True, "output")), 0),
    # one routed expert per token plus the shared expert (the Llama-4 arrangement)
    "shared_expert_top1_bf16": (dict(tokens=32, model_dim=64, num_experts=4, top_k=1, inner_dim=64,
                                     dtype="bf16", seed=104, shared=True), 0),
    # e4m3 expert weights with per-channel scales, a decode-sized batch
    "fp8_weights_decode": (dict(tokens=8, model_dim=128, num_experts=8, top_k=2, inner_dim=64,
                                dtype="bf16", weight_dtype="fp8", seed=105, zipf_s=1.2,
                                mode=W.RoutingMode("softmax", True, "output")), 0),
    # the whole feed-forward step of a pre-norm decoder layer: x + layer(rms_norm(x))
    "pre_norm_residual_bf16": (dict(tokens=32, model_dim=64, num_experts=8, top_k=2, inner_dim=64,
                                    dtype="bf16", seed=111,
                                    mode=W.RoutingMode("softmax", True, "output")), 0),
}
# cases whose layer input is the RMS normalisation (this epsilon) of stored raw rows, and whose
# expected output includes those raw rows as the residual
PRE_NORM = {"pre_norm_residual_bf16": 1e-5}


def build_case(name: str) -> W.Workload:
    kw, zero_rows = CASES[name]
    wl = W.make_workload_from_spec(W.small_spec(**kw))
    if zero_rows:
        wl.x[:, :zero_rows] = 0.0
    if name in PRE_NORM:
        # raw rows of varying scale and an elementwise weight, both exact in the activation type;
        # the layer's input is their normalisation (nn/normalization.py:234-236), rounded to that type
        dt = torch.bfloat16 if wl.spec.dtype == "bf16" else torch.float32
        g = torch.Generator().manual_seed(7)
        raw = 3.0 * torch.randn(wl.x.shape, generator=g) * (0.25 + torch.rand(wl.x.shape[:-1] + (1,), generator=g))
        gamma = 1.0 + 0.2 * torch.randn(wl.x.shape[-1], generator=g)
        wl.raw, wl.gamma, wl.norm_eps = raw.to(dt).float(), gamma.to(dt).float(), PRE_NORM[name]
        wl.x = O.rms_norm(wl.raw.to(dt), wl.gamma.to(dt), wl.norm_eps).float()
    return wl


def evaluate(wl: W.Workload) -> dict[str, np.ndarray]:
    s = wl.spec
    d = lambda t: None if t is None else t.double()  # noqa: E731
    shared = (d(wl.shared_gate), d(wl.shared_up), d(wl.shared_down)) if s.shared else None
    logits = O.router_logits(d(wl.x), d(wl.router), d(wl.router_bias))
    idx = O.topk_lowest_index(logits, s.top_k)
    out = O.ref_dense_forward(
        d(wl.x), d(wl.router), d(wl.gate), d(wl.up), d(wl.down), s.top_k, shared=shared,
        router_bias=d(wl.router_bias), score_fn=s.mode.score_fn, renormalize=s.mode.renormalize,
        scale_on=s.mode.scale_on,
    )
    if getattr(wl, "raw", None) is not None:
        out = out + wl.raw.double()
        # the selection must not hinge on the last bit of a normalised value
        top = torch.sort(logits, dim=1, descending=True).values[:, : s.top_k + 1]
        # (one rounding step of a normalised value moves a logit by about 1e-4 here)
        assert float((top[:, :-1] - top[:, 1:]).min()) > 2e-3, "choose another seed: near-tied logits"
    return {"topk_idx": idx.numpy().astype(np.int32), "out": out.numpy()}


def _pack(t: torch.Tensor, dtype: str) -> np.ndarray:
    """float32 values exactly representable in ``dtype`` -> the stored array."""
    if dtype == "bf16":
        bits = t.contiguous().view(torch.int32).numpy()
        assert not (bits & 0xFFFF).any(), "value is not a bf16 number"
        return (bits >> 16).astype(np.uint16)
    return t.numpy()


def _unpack(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint16:
        return torch.from_numpy(a.astype(np.int32) << 16).view(torch.float32)
    return torch.from_numpy(a)


def main() -> None:
    for name in CASES:
        wl = build_case(name)
        s = wl.spec
        fp8 = s.weight_dtype == "fp8"
        arrays = {"x": _pack(wl.x, s.dtype), "router": _pack(wl.router, s.dtype)}
        if fp8:
            # the de-quantised weights are a function of codes and scales: not stored
            for key, t in wl.fp8.items():
                arrays["fp8_" + key] = t.numpy() if t.dtype == torch.float32 else t.view(torch.uint8).numpy()
        else:
            arrays.update(gate=_pack(wl.gate, s.dtype), up=_pack(wl.up, s.dtype), down=_pack(wl.down, s.dtype))
        if wl.router_bias is not None:
            arrays["router_bias"] = wl.router_bias.numpy()
        if s.shared:
            arrays.update(shared_gate=_pack(wl.shared_gate, s.dtype), shared_up=_pack(wl.shared_up, s.dtype),
                          shared_down=_pack(wl.shared_down, s.dtype))
        if name in PRE_NORM:
            arrays.update(raw=_pack(wl.raw, s.dtype), gamma=_pack(wl.gamma, s.dtype))
        arrays.update({"expected_" + k: v for k, v in evaluate(wl).items()})
        meta = dict(
            tokens=s.num_tokens, model_dim=s.model_dim, num_experts=s.num_experts, top_k=s.top_k,
            inner_dim=s.inner_dim, dtype=s.dtype, weight_dtype=s.weight_dtype, shared=s.shared,
            score_fn=s.mode.score_fn, renormalize=s.mode.renormalize, scale_on=s.mode.scale_on,
        )
        if name in PRE_NORM:
            meta["norm_eps"] = PRE_NORM[name]
        arrays["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
        np.savez_compressed(HERE / f"{name}.npz", **arrays)
        print(f"{name}: {(HERE / f'{name}.npz').stat().st_size / 1024:.0f} KiB")


def load_case(name: str) -> tuple[W.Workload, dict[str, np.ndarray]]:
    """A stored case as a workload (CPU tensors) and its expected results."""
    with np.load(HERE / f"{name}.npz", allow_pickle=False) as z:
        a = {k: z[k] for k in z.files}
    m = json.loads(a["meta"].tobytes().decode())
    spec = W.small_spec(
        tokens=m["tokens"], model_dim=m["model_dim"], num_experts=m["num_experts"], top_k=m["top_k"],
        inner_dim=m["inner_dim"], dtype=m["dtype"], weight_dtype=m["weight_dtype"], shared=m["shared"],
        mode=W.RoutingMode(m["score_fn"], m["renormalize"], m["scale_on"]),
    )
    get = lambda k: _unpack(a[k]) if k in a else None  # noqa: E731
    wl = W.Workload(spec, get("x"), get("router"), get("router_bias"))
    if m["weight_dtype"] == "fp8":
        for key in ("gate", "up", "down"):
            q = torch.from_numpy(a[f"fp8_{key}_q"]).view(torch.float8_e4m3fn)
            scale = torch.from_numpy(a[f"fp8_{key}_scale"])
            wl.fp8[key + "_q"], wl.fp8[key + "_scale"] = q, scale
            setattr(wl, key, W.dequantize_fp8_per_channel(q, scale))
    else:
        wl.gate, wl.up, wl.down = get("gate"), get("up"), get("down")
    wl.shared_gate, wl.shared_up, wl.shared_down = get("shared_gate"), get("shared_up"), get("shared_down")
    if "norm_eps" in m:
        wl.raw, wl.gamma, wl.norm_eps = get("raw"), get("gamma"), m["norm_eps"]
    return wl, {"topk_idx": a["expected_topk_idx"], "out": a["expected_out"]}


if __name__ == "__main__":
    main()

"""Seeded synthetic workloads for the MoE feed-forward path.

Six named layer shapes are defined: one small fp32 case that the CPU reference
formulation runs comfortably, three bf16 prefill shapes (Mixtral-8x7B,
Qwen3-30B-A3B, Llama-4-Scout), the Qwen3 prefill shape with fp8 weights and one
fp8-weight decode shape.  Every tensor is
drawn from one CPU generator in a fixed order, so the same seed gives the same
layer on any machine:

    x, router, perm, gate, up, down[, shared gate, shared up, shared down]

The reference layer (fairseq2 ``models/llama4/moe.py:94-157``) has no router
bias, scores with a sigmoid and scales the expert *input*.  The Mixtral and
Qwen3 shapes use the softmax / output-weighted conventions instead; those are
expressed through :class:`RoutingMode` and are extensions of the reference.

Router bias: "a per-expert bias drawn from Zipf(s)" is read as a popularity
law, ``bias[perm[r]] = -s * ln(r + 1)`` for rank r, so that expert r's share of
tokens falls off like a power law.  Adding raw Zipf integer samples (infinite
mean for s <= 2) to logits of unit scale would send every token to the same K
experts, which measures nothing.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
from torch import Tensor


@dataclass(frozen=True)
class RoutingMode:
    """How router logits become combine weights.

    ``score_fn="sigmoid"``, ``renormalize=False``, ``scale_on="input"`` is the
    reference behaviour (``moe.py:113-133``).
    """

    score_fn: str = "sigmoid"  # "sigmoid" | "softmax"
    renormalize: bool = False
    scale_on: str = "input"  # "input" | "output"


@dataclass(frozen=True)
class WorkloadSpec:
    name: str
    seed: int
    batch: int
    seq_len: int
    model_dim: int
    num_experts: int
    top_k: int
    inner_dim: int
    dtype: str  # "fp32" | "bf16"
    weight_dtype: str  # "fp32" | "bf16" | "fp8"
    zipf_s: float | None
    shared: bool
    mode: RoutingMode
    act_quant: str | None = None  # "mxfp8": the experts' inputs in block-scaled e4m3 (W8A8)

    @property
    def num_tokens(self) -> int:
        return self.batch * self.seq_len

    @property
    def sparse_flops(self) -> int:
        """Algorithmic flops of the routed experts (6*T*K*D*F) plus the shared expert."""
        f = 6 * self.num_tokens * self.top_k * self.model_dim * self.inner_dim
        if self.shared:
            f += 6 * self.num_tokens * self.model_dim * self.inner_dim
        return f

    @property
    def dense_flops(self) -> int:
        """Flops of the reference's dense formulation (every expert sees every token)."""
        f = 6 * self.num_tokens * self.num_experts * self.model_dim * self.inner_dim
        if self.shared:
            f += 6 * self.num_tokens * self.model_dim * self.inner_dim
        return f


_REFERENCE_MODE = RoutingMode("sigmoid", False, "input")

SPECS: dict[str, WorkloadSpec] = {
    "small_fp32": WorkloadSpec(
        "small_fp32", 0, 8, 512, 512, 8, 2, 1408, "fp32", "fp32", None, False, _REFERENCE_MODE
    ),
    "mixtral_8x7b": WorkloadSpec(
        "mixtral_8x7b", 1, 16, 512, 4096, 8, 2, 14336, "bf16", "bf16", 1.1, False,
        RoutingMode("softmax", True, "output"),
    ),
    "qwen3_30b_a3b": WorkloadSpec(
        "qwen3_30b_a3b", 2, 8, 1024, 2048, 128, 8, 768, "bf16", "bf16", 1.2, False,
        RoutingMode("softmax", True, "output"),
    ),
    "llama4_scout": WorkloadSpec(
        "llama4_scout", 3, 8, 1024, 5120, 16, 1, 8192, "bf16", "bf16", None, True, _REFERENCE_MODE
    ),
    # the Qwen3 prefill shape with the decode case's weight format: e4m3 weights in the GEMM regime
    "qwen3_30b_a3b_fp8": WorkloadSpec(
        "qwen3_30b_a3b_fp8", 2, 8, 1024, 2048, 128, 8, 768, "bf16", "fp8", 1.2, False,
        RoutingMode("softmax", True, "output"),
    ),
    # and with the experts' inputs quantised as well: both products on the fp8 matrix pipe
    "qwen3_30b_a3b_w8a8": WorkloadSpec(
        "qwen3_30b_a3b_w8a8", 2, 8, 1024, 2048, 128, 8, 768, "bf16", "fp8", 1.2, False,
        RoutingMode("softmax", True, "output"), "mxfp8",
    ),
    "qwen3_decode_fp8": WorkloadSpec(
        "qwen3_decode_fp8", 4, 64, 1, 2048, 128, 8, 768, "bf16", "fp8", 1.2, False,
        RoutingMode("softmax", True, "output"),
    ),
    # decode steps of one and of eight sequences with the weights as the reference holds them
    "qwen3_decode_bf16_1": WorkloadSpec(
        "qwen3_decode_bf16_1", 5, 1, 1, 2048, 128, 8, 768, "bf16", "bf16", 1.2, False,
        RoutingMode("softmax", True, "output"),
    ),
    "qwen3_decode_bf16_8": WorkloadSpec(
        "qwen3_decode_bf16_8", 6, 8, 1, 2048, 128, 8, 768, "bf16", "bf16", 1.2, False,
        RoutingMode("softmax", True, "output"),
    ),
}

FP8_MAX = 448.0  # largest finite OCP e4m3fn value


@dataclass
class Workload:
    """Tensors of one layer, all on the CPU.

    ``x``, ``router`` and the weights hold values that are exactly representable
    in ``spec.dtype`` but are stored as fp32, so that an fp32/fp64 evaluation
    and the device kernels consume identical numbers.  For fp8 workloads the
    ``*_q`` tensors hold the e4m3 codes, ``*_scale`` the per-output-channel fp32
    scales, and ``gate/up/down`` the de-quantised values.
    """

    spec: WorkloadSpec
    x: Tensor  # (B, S, D)
    router: Tensor  # (D, E)
    router_bias: Tensor | None  # (E,)
    gate: Tensor | None = None  # (E*D, F)
    up: Tensor | None = None  # (E*D, F)
    down: Tensor | None = None  # (E*F, D)
    shared_gate: Tensor | None = None  # (F, D)
    shared_up: Tensor | None = None  # (F, D)
    shared_down: Tensor | None = None  # (D, F)
    fp8: dict[str, Tensor] = field(default_factory=dict)


def _round_to(t: Tensor, dtype: str) -> Tensor:
    if dtype == "bf16":
        return t.to(torch.bfloat16).to(torch.float32)
    return t


def zipf_router_bias(num_experts: int, s: float, perm: Tensor) -> Tensor:
    """``bias[perm[r]] = -s * ln(r + 1)``: expert popularity follows rank^-s."""
    ranks = torch.arange(num_experts, dtype=torch.float64)
    bias = torch.empty(num_experts, dtype=torch.float32)
    bias[perm] = (-s * torch.log(ranks + 1.0)).to(torch.float32)
    return bias


def quantize_fp8_per_channel(w: Tensor, num_experts: int) -> tuple[Tensor, Tensor]:
    """Quantises folded expert weights ``(E*K, N)`` to e4m3 with one fp32 scale
    per expert and output channel: ``scale[e, n] = max_k |w[e, k, n]| / 448``.

    torch's fp32 -> float8_e4m3fn cast does not saturate, so the weights are
    scaled so the column maximum lands exactly on 448 before the cast.
    """
    rows, n = w.shape
    k = rows // num_experts
    w3 = w.view(num_experts, k, n)
    amax = w3.abs().amax(dim=1)  # (E, N)
    scale = (amax / FP8_MAX).clamp_min(torch.finfo(torch.float32).tiny)
    q = (w3 / scale[:, None, :]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q.view(rows, n), scale.to(torch.float32)


def dequantize_fp8_per_channel(q: Tensor, scale: Tensor) -> Tensor:
    e, n = scale.shape
    k = q.shape[0] // e
    return (q.view(e, k, n).to(torch.float32) * scale[:, None, :]).view(e * k, n)


def make_workload(
    name: str,
    *,
    with_weights: bool = True,
    batch: int | None = None,
    seq_len: int | None = None,
) -> Workload:
    """Draws the named workload.  ``with_weights=False`` stops after the router
    tensors (enough for routing statistics at the large shapes)."""
    spec = SPECS[name]
    if batch is not None or seq_len is not None:
        spec = WorkloadSpec(
            **{**spec.__dict__, "batch": batch or spec.batch, "seq_len": seq_len or spec.seq_len}
        )
    return make_workload_from_spec(spec, with_weights=with_weights)


def make_workload_from_spec(spec: WorkloadSpec, *, with_weights: bool = True) -> Workload:
    g = torch.Generator("cpu").manual_seed(spec.seed)
    d, e, f = spec.model_dim, spec.num_experts, spec.inner_dim

    x = _round_to(torch.randn(spec.batch, spec.seq_len, d, generator=g), spec.dtype)
    router = _round_to(0.02 * torch.randn(d, e, generator=g), spec.dtype)
    perm = torch.randperm(e, generator=g)
    bias = zipf_router_bias(e, spec.zipf_s, perm) if spec.zipf_s is not None else None

    wl = Workload(spec, x, router, bias)
    if not with_weights:
        return wl

    wdt = "bf16" if spec.weight_dtype == "fp8" else spec.weight_dtype
    wl.gate = _round_to(0.02 * torch.randn(e * d, f, generator=g), wdt)
    wl.up = _round_to(0.02 * torch.randn(e * d, f, generator=g), wdt)
    wl.down = _round_to(0.02 * torch.randn(e * f, d, generator=g), wdt)
    if spec.shared:
        wl.shared_gate = _round_to(0.02 * torch.randn(f, d, generator=g), wdt)
        wl.shared_up = _round_to(0.02 * torch.randn(f, d, generator=g), wdt)
        wl.shared_down = _round_to(0.02 * torch.randn(d, f, generator=g), wdt)

    if spec.weight_dtype == "fp8":
        for key in ("gate", "up", "down"):
            q, s = quantize_fp8_per_channel(getattr(wl, key), e)
            wl.fp8[key + "_q"] = q
            wl.fp8[key + "_scale"] = s
            setattr(wl, key, dequantize_fp8_per_channel(q, s))
    return wl


def small_spec(
    *,
    tokens: int = 96,
    model_dim: int = 64,
    num_experts: int = 8,
    top_k: int = 2,
    inner_dim: int = 96,
    dtype: str = "bf16",
    weight_dtype: str | None = None,
    seed: int = 7,
    zipf_s: float | None = None,
    shared: bool = False,
    mode: RoutingMode = _REFERENCE_MODE,
    act_quant: str | None = None,
) -> WorkloadSpec:
    """A free-form spec for tests at sizes the CPU evaluates in milliseconds."""
    return WorkloadSpec(
        "custom", seed, 1, tokens, model_dim, num_experts, top_k, inner_dim, dtype,
        weight_dtype or dtype, zipf_s, shared, mode, act_quant,
    )


def describe_bias_rule(spec: WorkloadSpec) -> str:
    if spec.zipf_s is None:
        return "none (reference behaviour)"
    return f"bias[perm[r]] = -{spec.zipf_s} * ln(r + 1)"


def log2_ceil(n: int) -> int:
    return max(0, math.ceil(math.log2(max(1, n))))


_TORCH_DTYPE = {"fp32": torch.float32, "bf16": torch.bfloat16}


def build_module(wl: Workload, device, tile_m: int = 16):
    """Constructs the drop-in module for a workload and loads its weights through the
    reference's state-dict names."""
    from fairseq2_amd.moe import MoE

    s = wl.spec
    dt = _TORCH_DTYPE[s.dtype]
    prev = torch.get_default_dtype()
    torch.set_default_dtype(dt)
    try:
        m = MoE(
            s.model_dim, s.inner_dim, s.shared, s.num_experts, 1.0, s.top_k,
            inner_dim_scale=1.0, auto_scale=False,
            score_fn=s.mode.score_fn, renormalize=s.mode.renormalize, scale_on=s.mode.scale_on,
            router_bias=wl.router_bias is not None, tile_m=tile_m, act_quant=s.act_quant,
        )
    finally:
        torch.set_default_dtype(prev)
    sd = {
        "router": wl.router.to(dt),
        "experts.gate_proj": wl.gate.to(dt),
        "experts.inner_proj": wl.up.to(dt),
        "experts.output_proj": wl.down.to(dt),
    }
    if s.shared:
        sd["shared_expert.gate_proj.weight"] = wl.shared_gate.to(dt)
        sd["shared_expert.inner_proj.weight"] = wl.shared_up.to(dt)
        sd["shared_expert.output_proj.weight"] = wl.shared_down.to(dt)
    if wl.router_bias is not None:
        sd["router_bias"] = wl.router_bias
    m.load_state_dict(sd, strict=True)
    m = m.to(device).requires_grad_(False).eval()
    if s.weight_dtype == "fp8":
        f8 = wl.fp8
        m.experts.load_fp8_weights(
            f8["gate_q"], f8["gate_scale"], f8["up_q"], f8["up_scale"], f8["down_q"], f8["down_scale"]
        )
    return m

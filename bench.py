#!/usr/bin/env python3
"""Benchmark of the MoE feed-forward forward path on one MI355X.

A step is one forward pass of the layer over one batch of synthetic tokens that
is already resident in HBM.  The default workload is the Qwen3-30B-A3B-shaped
layer (8192 tokens, d_model 2048, 128 experts, top-8, expert ffn 768, bf16).

Prints ONE JSON line: whole-layer tokens/s, the roofline of the dominant kernel
pair (the grouped SwiGLU GEMMs, MFMA-bound) measured with events on the launch
stream, per-stage times and HBM/MFMA fractions, and the reference's dense
formulation timed on this machine's host cores on a bounded sample.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3, "fp8": 5000.0}  # dense, published

# HBM bytes per launch of the dominant kernel pair, from `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` runs of this script (see profiles/); None until measured for a workload.
# The commit whose kernels the table below was measured on: a kernel change after it makes the
# figures stale until the counter runs are repeated (the roofline object carries the stamp).
MEASURED_TRAFFIC_AT = "06e32e2"
MEASURED_TRAFFIC_BYTES: dict[str, float | None] = {
    # profiles/bench_<workload>_all_kernels.md, the two launches of the grouped experts together
    # (FETCH_SIZE scaled by 2.0, WRITE_SIZE by 1.0 against a 256 MiB copy)
    "qwen3_30b_a3b": 2.653e9,     # gate/up 1566 + 101 MB, down 717 + 269 MB
    "mixtral_8x7b": 13.402e9,     # gate/up 8792 + 470 MB, down 4006 + 134 MB
    "llama4_scout": 6.677e9,      # routed experts only: gate/up 4103 + 135 MB, down 2355 + 84 MB
    "small_fp32": 0.866e9,        # gate/up 402 + 46 MB, down 401 + 17 MB
    "qwen3_decode_fp8": 0.222e9,  # gate/up 143 + 1 MB, down 76 + 2 MB
    "qwen3_30b_a3b_fp8": 1.886e9,  # gate/up 1033 + 101 MB, down 484 + 269 MB
    "qwen3_30b_a3b_w8a8": 1.475e9,  # gate/up 778 + 67 MB, down 362 + 269 MB
}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--settle-ms", type=float, default=150.0,
                   help="run the step untimed for this long before the warm-up steps: from idle the "
                        "GPU raises its clock over some 40 ms of sustained load, and a short run "
                        "would measure that ramp instead of the sustained rate")
    p.add_argument("--workload", default="qwen3_30b_a3b")
    p.add_argument("--tile-m", type=int, default=16)
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--cpu-seconds", type=float, default=15.0, help="target CPU-baseline time")
    p.add_argument("--stage-reps", type=int, default=20)
    p.add_argument("--graph", action="store_true",
                   help="time replays of one captured HIP graph of the layer instead of eager calls")
    p.add_argument("--training-step", action="store_true",
                   help="also time forward + backward of the module (reported beside the metric, "
                        "not part of it; bf16 / fp32 weights only)")
    p.add_argument("--no-vendor-gemm", action="store_true",
                   help="skip the yardstick that is otherwise reported beside the metric for bf16 "
                        "workloads: the expert GEMM shapes as three dense products in the vendor's "
                        "library (torch.matmul -> hipBLASLt) on normally distributed and on all-zero "
                        "operands, and this build's expert kernels on all-zero operands (what the "
                        "matrix pipes sustain depends on the operand data: the part is power-limited)")
    p.add_argument("--vendor-gemm", action="store_true", help="accepted for compatibility: the yardstick is on by default")
    p.add_argument("--no-pre-norm-step", action="store_true",
                   help="skip the pre-norm variant of the step (x + layer(rms_norm(x)) in one call) that is "
                        "otherwise timed beside the metric: a profiler run then sees the kernels of the "
                        "metric's own step only")
    p.add_argument("--calibration-copy", action="store_true",
                   help="also run a 256 MiB device copy (reference point for rocprofv3 byte counters)")
    return p.parse_args()


def elem_bytes(dtype: str) -> int:
    return 4 if dtype == "fp32" else 2


def stage_work(spec, active_experts: int) -> dict[str, dict]:
    """Algorithmic bytes / flops of each stage (padding rows and re-reads are not useful work)."""
    t, d, e, k, f = spec.num_tokens, spec.model_dim, spec.num_experts, spec.top_k, spec.inner_dim
    b = elem_bytes(spec.dtype)
    wb = 1 if spec.weight_dtype == "fp8" else b
    scales = active_experts * (2 * f + d) * 4 if spec.weight_dtype == "fp8" else 0
    work = {
        "router": {"bytes": t * d * b + d * e * b + t * k * 8, "flops": 2 * t * d * e},
        "dispatch": {"bytes": t * d * b + t * k * d * b + t * k * 12},
        "experts": {
            "flops": 6 * t * k * d * f,
            "bytes": 3 * active_experts * d * f * wb + scales + 2 * t * k * d * b + 2 * t * k * f * b,
        },
        "combine": {"bytes": t * k * d * b + t * d * b + (t * d * b if spec.shared else 0)},
    }
    if spec.shared:
        work["shared"] = {"flops": 6 * t * d * f}
    return work


def time_stages(module, x, reps: int):
    """Average milliseconds of each stage, from events on the stream the kernels run on."""
    import torch

    from fairseq2_amd import _abi
    from fairseq2_amd.moe import _SCORE_FNS

    ex = module.experts
    scale_input = module.scale_on == "input"
    # as in MoE._stages: unscaled rows are read through the permutation by the first GEMM
    fused = (not scale_input) and hasattr(ex, "fuses_gather") and ex.fuses_gather(x.dtype)
    names = ["router", "dispatch", "experts"] + (["shared"] if module.shared_expert else []) + ["combine"]
    # as in MoE._stages: a token takes an expert at most once, a bound the expert stage uses when small
    bound = x.shape[0] if x.shape[0] <= 16 else 0
    tot = {n: 0.0 for n in names}
    tot["dispatch_with_gather"] = 0.0
    ev = lambda: torch.cuda.Event(enable_timing=True)
    def timed(fn):
        e0, e1 = ev(), ev()
        e0.record()
        r = fn()
        e1.record()
        return r, (e0, e1)

    # All repetitions are enqueued back to back and read after one synchronisation at the end: a
    # synchronisation per repetition would let the GPU idle (and its clock drop) between them.
    recorded = []
    for rep in range(reps + 2):
        spans = {}
        (idx, w, _), spans["router"] = timed(lambda: _abi.router_topk(
            x, module.router, module.router_bias, module.top_k, _SCORE_FNS[module.score_fn], module.renormalize,
            router_t=module._router_expert_major(),  # as the module's own calls pass it
        ))
        # the row copy that the fused path skips, timed on its own (at the place in the sequence
        # where it would be the real thing): the HBM-bound part of dispatch, with its own roofline
        _, spans["dispatch_with_gather"] = timed(lambda: _abi.dispatch(
            idx, w, x, ex.num_local_experts, module.tile_m, scale_input, gather=True
        ))
        disp, spans["dispatch"] = timed(lambda: _abi.dispatch(
            idx, w, x, ex.num_local_experts, module.tile_m, scale_input, gather=not fused
        ))
        if fused:
            ye, spans["experts"] = timed(lambda: ex.forward_rows(x, disp.counts, disp.offsets, row_map=disp.perm,
                                                                 rows_per_expert=bound))
        else:
            ye, spans["experts"] = timed(lambda: ex.forward_rows(disp.xe, disp.counts, disp.offsets,
                                                                 rows_per_expert=bound))
        base = None
        if module.shared_expert is not None:
            base, spans["shared"] = timed(lambda: module.shared_expert(x))
        _, spans["combine"] = timed(lambda: _abi.combine(ye, disp.inv_perm, idx, w, base, not scale_input, out=base))
        if rep >= 2:
            recorded.append(spans)
    torch.cuda.synchronize()
    for spans in recorded:
        for n, (e0, e1) in spans.items():
            tot[n] += e0.elapsed_time(e1)
    out = {n: v / reps for n, v in tot.items()}
    out["fused_gather"] = fused
    return out


def experts_back_to_back(module, x, reps: int) -> float:
    """Milliseconds per call of the expert stage alone, `reps` calls enqueued back to back between
    two events.  At decode sizes the stage is two kernels of a few tens of microseconds: between the
    events of time_stages the GPU also waits for the host to launch them (the span reads 75 us where
    the kernels take 47), while a queue of calls keeps the GPU busy, so this is the kernels' time plus
    the gap between them."""
    import torch

    from fairseq2_amd import _abi
    from fairseq2_amd.moe import _SCORE_FNS

    ex = module.experts
    scale_input = module.scale_on == "input"
    fused = (not scale_input) and hasattr(ex, "fuses_gather") and ex.fuses_gather(x.dtype)
    bound = x.shape[0] if x.shape[0] <= 16 else 0
    idx, w, _ = _abi.router_topk(x, module.router, module.router_bias, module.top_k,
                                 _SCORE_FNS[module.score_fn], module.renormalize)
    disp = _abi.dispatch(idx, w, x, ex.num_local_experts, module.tile_m, scale_input, gather=not fused)
    if fused:
        run = lambda: ex.forward_rows(x, disp.counts, disp.offsets, row_map=disp.perm, rows_per_expert=bound)  # noqa: E731
    else:
        run = lambda: ex.forward_rows(disp.xe, disp.counts, disp.offsets, rows_per_expert=bound)  # noqa: E731
    for _ in range(10):
        run()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        run()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def cpu_baseline(wl, seconds: float) -> dict:
    """The reference's dense formulation (every expert over every token) on the host cores, on the
    first tokens of the same workload; its cost is linear in the token count and independent of the
    routing, so tokens/s carries over to the full batch."""
    import torch

    from oracle import moe_oracle as O

    spec = wl.spec
    dt = torch.float32 if spec.dtype == "fp32" else torch.bfloat16
    kw = O.dense_cpu_baseline_inputs(wl, dt)
    flat = kw["seqs"].reshape(-1, spec.model_dim)

    def run(n):
        args = dict(kw)
        args["seqs"] = flat[:n].reshape(1, n, spec.model_dim)
        t0 = time.perf_counter()
        with torch.no_grad():
            O.ref_dense_forward(**args)
        return time.perf_counter() - t0

    probe_n = min(64, spec.num_tokens)
    run(probe_n)  # warm-up (thread pool, kernels selection)
    # Grow the sample until one pass takes about `seconds`: small samples run at a lower rate (the
    # per-expert matrix products are too small to use the cores), so a size extrapolated from the
    # probe alone would fall well short of the target time.
    n, dt_s = probe_n, run(probe_n)
    for _ in range(3):
        if dt_s >= 0.6 * seconds or n >= spec.num_tokens:
            break
        want = int(n * min(16.0, 0.9 * seconds / max(dt_s, 1e-9)))
        n = min(spec.num_tokens, max(n + 64, want // 64 * 64))
        dt_s = run(n)
    # the whole workload in less than the target time: repeat the pass and report the mean
    passes = 1
    if dt_s < 0.6 * seconds:
        passes = int(min(10, max(2, 0.9 * seconds / max(dt_s, 1e-9))))
        t0 = time.perf_counter()
        for _ in range(passes):
            run(n)
        dt_s = (time.perf_counter() - t0) / passes
    return {
        "value": n / dt_s,
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"dense reference formulation in {str(dt).replace('torch.', '')} on the first {n} of "
                  f"{spec.num_tokens} tokens, mean of {passes} timed pass(es) of {dt_s:.2f} s each "
                  f"(after shorter passes that sized the sample)",
    }


def vendor_gemm(spec, dev, fp8: bool = False) -> dict:
    """The routed rows as ONE group through the vendor's dense bf16 GEMM: (T K, D) x (D, F) twice and
    (T K, F) x (F, D).  No grouping, no skew, no gather, no gate: what the same flops cost in the
    library AMD ships, on this box.  Timed twice: on data drawn like the workload's, and on all-zero
    operands, which toggle no bits in the matrix pipes and so show what the same instruction stream
    reaches when the clock is not held down by power.
    ``fp8``: both operands e4m3 with one scale per tensor (torch._scaled_mm, bf16 result): the
    library's counterpart of the W8A8 workload's products, without that path's block scales, channel
    scales or the quantisation of the gated product."""
    import torch

    rows, d, f = spec.num_tokens * spec.top_k, spec.model_dim, spec.inner_dim
    if fp8:
        one = torch.ones((), device=dev)
        mm = lambda a, b: torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)  # noqa: E731
        cast = lambda t: t.to(torch.float8_e4m3fn)  # noqa: E731
    else:
        mm = lambda a, b: torch.matmul(a, b)  # noqa: E731
        cast = lambda t: t.to(torch.bfloat16)  # noqa: E731
    # weights as (in, out) for the bf16 product (the reference's layout); the e4m3 product wants its
    # second operand column-major, i.e. stored (out, in)
    wshape = (lambda i, o: (o, i)) if fp8 else (lambda i, o: (i, o))

    def timed(fn, reps=20):
        for _ in range(10):
            fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = float("inf")
        for _ in range(3):
            a.record()
            for _ in range(reps):
                fn()
            b.record()
            torch.cuda.synchronize()
            best = min(best, a.elapsed_time(b) / reps)
        return best

    flops = 6.0 * rows * d * f
    out = {"what": ("torch._scaled_mm (hipBLASLt, e4m3 x e4m3, per-tensor scales)" if fp8 else "torch.matmul (hipBLASLt)")
                   + " on the routed rows as one dense group: gate, up and down products"}
    for name in ("normal", "zeros"):
        if name == "normal":
            g = torch.Generator(device=dev).manual_seed(1)
            x = cast(torch.randn(rows, d, device=dev, generator=g))
            h = cast(torch.randn(rows, f, device=dev, generator=g))
            w1 = cast((1.0 if fp8 else 0.02) * torch.randn(*wshape(d, f), device=dev, generator=g))
            w2 = cast((1.0 if fp8 else 0.02) * torch.randn(*wshape(f, d), device=dev, generator=g))
        else:
            x, h = cast(torch.zeros(rows, d, device=dev)), cast(torch.zeros(rows, f, device=dev))
            w1, w2 = cast(torch.zeros(*wshape(d, f), device=dev)), cast(torch.zeros(*wshape(f, d), device=dev))
        with torch.no_grad():
            up_ms = timed(lambda: mm(x, w1))
            down_ms = timed(lambda: mm(h, w2))
        total = 2 * up_ms + down_ms
        ent = {"ms": round(total, 4), "gate_or_up_ms": round(up_ms, 4), "down_ms": round(down_ms, 4),
               "achieved_tflops": round(flops / (total * 1e-3) / 1e12, 1)}
        if name == "normal":
            out.update(ent)
        else:
            out["zero_operands"] = ent
        del x, h, w1, w2
    return out


def experts_on_zero_operands(module, x2, reps: int) -> dict:
    """This build's expert kernels on the workload's routing with every operand zero (weights and
    rows): same launches, same tiles, same memory traffic, no bits toggling in the matrix pipes.
    Zeroes the module's expert weights, so it runs after everything else that uses the module."""
    import torch

    from fairseq2_amd import _abi
    from fairseq2_amd.moe import _SCORE_FNS

    ex = module.experts
    if not (module.scale_on != "input" and hasattr(ex, "fuses_gather") and ex.fuses_gather(x2.dtype)):
        return {}
    idx, w, _ = _abi.router_topk(x2, module.router, module.router_bias, module.top_k,
                                 _SCORE_FNS[module.score_fn], module.renormalize)
    disp = _abi.dispatch(idx, w, x2, ex.num_local_experts, module.tile_m, False, gather=False)
    for p in ex.parameters():
        p.zero_()
    zx = torch.zeros_like(x2)
    run = lambda: ex.forward_rows(zx, disp.counts, disp.offsets, row_map=disp.perm)  # noqa: E731
    for _ in range(10):
        run()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        run()
    b.record()
    torch.cuda.synchronize()
    return {"ms": round(a.elapsed_time(b) / reps, 4)}


def training_step(module, x3, steps: int) -> dict:
    """Forward + backward of the module with every parameter and the input requiring a gradient
    (the library's backward kernels): milliseconds per step and the peak memory torch saw."""
    import torch

    module.train().requires_grad_(True)
    x = x3.detach().clone().requires_grad_(True)
    grad = torch.randn_like(x)

    def step():
        for p in module.parameters():
            p.grad = None
        x.grad = None
        module(x).backward(grad)

    for _ in range(3):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    module.requires_grad_(False).eval()
    return {
        "ms": round(ms, 4), "steps": steps,
        "peak_memory_gib": round(torch.cuda.max_memory_allocated() / 2**30, 2),
        "what": "forward + backward of the module (gradients of the input and of every parameter)",
    }


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(
            "bench.py measures the single-GPU MoE forward path; this build has no multi-GPU path, "
            f"so --gpus {args.gpus} is not supported (use --gpus 1)",
            file=sys.stderr,
        )
        return 2

    import torch

    import workloads as W

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (no GPU visible)", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")

    wl = W.make_workload(args.workload)
    spec = wl.spec
    module = W.build_module(wl, dev, args.tile_m)
    dt = torch.float32 if spec.dtype == "fp32" else torch.bfloat16
    x3 = wl.x.to(dt).to(dev)
    x2 = x3.reshape(-1, spec.model_dim)

    with torch.no_grad():
        if args.graph:
            # the input already sits in the graph's input buffer: a step is one replay
            from fairseq2_amd import GraphedForward

            step = GraphedForward(module, x3).replay
        else:
            step = lambda: module(x3)  # noqa: E731
        # let the clock settle under this very load (untimed, like the warm-up steps)
        t_settle = time.perf_counter()
        while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
            for _ in range(8):
                step()
            torch.cuda.synchronize()
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        # the whole pre-norm feed-forward step in one call (not part of the metric): the rows
        # normalised by the router, the residual added by combine; timed like the step above
        class _Norm:
            weight, bias, eps, normalized_shape = torch.ones(spec.model_dim, dtype=dt, device=dev), None, 1e-5, (spec.model_dim,)

        fused_step = lambda: module(x3, residual=x3, norm=_Norm)  # noqa: E731
        fused_step_ms = None
        if not args.no_pre_norm_step:
            # settled like the step above: its first calls size buffers the plain step never asked for
            t_settle = time.perf_counter()
            while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
                for _ in range(8):
                    fused_step()
                torch.cuda.synchronize()
            for _ in range(args.warmup):
                fused_step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(args.steps):
                fused_step()
            torch.cuda.synchronize()
            fused_step_ms = (time.perf_counter() - t1) / args.steps * 1e3
        stage_ms = time_stages(module, x2, args.stage_reps)
        if args.calibration_copy:
            # A plain device copy of known size (256 MiB read + 256 MiB written), so that a counter
            # run of this script can scale FETCH_SIZE / WRITE_SIZE against a known byte count.
            src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            torch.cuda.synchronize()

    ms_per_step = elapsed / args.steps * 1e3
    tokens_per_s = spec.num_tokens * args.steps / elapsed

    with torch.no_grad():
        active = int((module.forward_with_routing(x3)[3].counts > 0).sum())
    work = stage_work(spec, active)
    # The expert GEMMs are MFMA-bound at prefill sizes and a weight stream (HBM-bound) at decode sizes:
    # the bound is whichever roofline gives the longer time for the algorithmic work.
    experts_hbm_bound = (
        work["experts"]["bytes"] / (HBM_PEAK_GBS * 1e9)
        > work["experts"]["flops"] / (MFMA_PEAK_TFLOPS[spec.dtype] * 1e12)
    )
    w8a8 = spec.act_quant == "mxfp8" and module.experts.runs_w8a8(dt, spec.num_tokens * spec.top_k)
    # the matrix pipe the expert products run on: fp8 only when both operands are e4m3 (W8A8);
    # e4m3 weights alone are turned into bf16 on the way to LDS
    peak_tf = MFMA_PEAK_TFLOPS["fp8" if w8a8 else spec.dtype]
    fused_gather = bool(stage_ms.pop("fused_gather", False))
    t, d, k, b = spec.num_tokens, spec.model_dim, spec.top_k, elem_bytes(spec.dtype)
    work["dispatch_with_gather"] = dict(work["dispatch"])
    if fused_gather:
        # no gathered copy exists: dispatch is bookkeeping, and the first GEMM reads the rows from x
        work["dispatch"] = {"bytes": t * k * 4 + t * k * 12}
        work["experts"]["bytes"] -= t * k * d * b - t * d * b
    stages = {}
    for name, ms in stage_ms.items():
        ent = {"ms": round(ms, 4)}
        w = work[name]
        if name == "shared" or (name == "experts" and not experts_hbm_bound):
            tf = w["flops"] / (ms * 1e-3) / 1e12
            pk = MFMA_PEAK_TFLOPS[spec.dtype] if name == "shared" else peak_tf
            ent.update(bound="mfma", achieved_tflops=round(tf, 2), frac=round(tf / pk, 4))
        else:
            gbs = w["bytes"] / (ms * 1e-3) / 1e9
            ent.update(bound="hbm", achieved_gbs=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 4))
        stages[name] = ent

    exp_ms = stage_ms["experts"]
    if w8a8:
        kernel = ("glu_gemm_mx_kernel<gate,up> + <down> (fs2moe_grouped_swiglu_w8a8; the launch time "
                  "includes mx_quantize_kernel over the token rows)")
    elif spec.weight_dtype == "fp8" and experts_hbm_bound:
        kernel = "glu_gemm_fp8w_kernel<gate,up> + <down> (fs2moe_grouped_swiglu)"
    elif spec.weight_dtype == "fp8":
        # e4m3 weights turned into bf16 on the way to LDS: the matrix pipe runs in bf16
        kernel = "glu_gemm_bf16_dma_kernel<gate,up> + <down>, e4m3 weights (fs2moe_grouped_swiglu)"
    else:
        kernel = "glu_gemm_%s_dma_kernel<gate,up> + <down> (fs2moe_grouped_swiglu)" % spec.dtype
    if spec.dtype == "fp32":
        kernel = "glu_gemm_f32_kernel<gate,up> + <down> (fs2moe_grouped_swiglu)"
    if spec.dtype == "bf16" and spec.weight_dtype == "bf16" and spec.num_tokens <= 16:
        # a few rows per expert: the weights are streamed without LDS tiles
        kernel = "%s<gate,up> + <down> (fs2moe_grouped_swiglu_rows)" % (
            "glu_gemv_bf16_kernel" if spec.num_tokens <= 4 else "glu_gemv16_bf16_kernel")
    if experts_hbm_bound:
        # (a weight stream of a few tens of microseconds: timed as a queue of calls, see there)
        with torch.no_grad():
            exp_ms = experts_back_to_back(module, x2, max(50, args.stage_reps))
        achieved = work["experts"]["bytes"] / (exp_ms * 1e-3) / 1e9
        roofline = {
            "kernel": kernel, "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
            "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload), "traffic_measured_at": MEASURED_TRAFFIC_AT,
            "launch_ms": round(exp_ms, 4), "launch_timing": "calls queued back to back",
            "bytes_per_launch": work["experts"]["bytes"], "active_experts": active,
        }
    else:
        achieved = work["experts"]["flops"] / (exp_ms * 1e-3) / 1e12
        roofline = {
            "kernel": kernel, "bound": "mfma", "achieved": round(achieved, 2), "peak": peak_tf,
            "unit": "TFLOP/s", "frac": round(achieved / peak_tf, 4),
            "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload), "traffic_measured_at": MEASURED_TRAFFIC_AT,
            "launch_ms": round(exp_ms, 4),
            "flops_per_launch": work["experts"]["flops"],
        }

    result = {
        "metric": "MoE layer forward tokens/sec on 1 MI355X",
        "value": round(tokens_per_s, 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("fp8 (e4m3) expert products: block-scaled activations, per-channel-scaled weights; bf16 elsewhere"
                  if w8a8 else spec.dtype if spec.weight_dtype != "fp8" else "bf16 activations, fp8 (e4m3) weights"),
        "data": "synthetic",
        "config": {
            "workload": spec.name,
            "launch": "one captured HIP graph per step" if args.graph else "eager",
            "clock_settle_ms": args.settle_ms,
            "gather": "fused into the first expert GEMM" if fused_gather else "separate copy in dispatch",
            "tokens": spec.num_tokens,
            "model_dim": spec.model_dim,
            "num_experts": spec.num_experts,
            "top_k": spec.top_k,
            "expert_inner_dim": spec.inner_dim,
            "shared_expert": spec.shared,
            "routing": f"{spec.mode.score_fn}, renormalize={spec.mode.renormalize}, scale_on={spec.mode.scale_on}",
            "router_bias": W.describe_bias_rule(spec),
            "tile_m": args.tile_m,
            "seed": spec.seed,
        },
        "roofline": roofline,
        "stages": stages,
    }
    if fused_step_ms is not None:
        result["pre_norm_step"] = {
            "ms": round(fused_step_ms, 4),
            "what": "x + layer(rms_norm(x)) in one call: norm in the router kernel, residual in combine",
        }
    if args.training_step and spec.weight_dtype != "fp8":
        result["training_step"] = training_step(module, x3, max(3, args.steps // 10))
    if not args.no_vendor_gemm and spec.dtype == "bf16" and not experts_hbm_bound:
        result["vendor_gemm"] = vendor_gemm(spec, dev, fp8=w8a8)
        if spec.weight_dtype == "bf16":
            with torch.no_grad():
                z = experts_on_zero_operands(module, x2, args.stage_reps)
            if z:
                z["achieved_tflops"] = round(work["experts"]["flops"] / (z["ms"] * 1e-3) / 1e12, 1)
                z["what"] = ("this build's two expert kernels, same routing, every operand zero: the same "
                             "instruction stream and memory traffic without the operands' switching power")
                result["experts_zero_operands"] = z
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(wl, args.cpu_seconds)
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())

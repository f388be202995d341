"""``fs2moe_forward_static``: the whole layer with the library's built-in scratch array in place of a
caller's workspace, for callers that cannot allocate.  Called through the C ABI and compared, bit for
bit, with ``fs2moe_forward`` on the same inputs: two calls in a row, the second on a smaller input (the
array then still holds the first call's intermediates), then the first input again.
"""

from __future__ import annotations

import pytest
import torch

from fairseq2_amd import _abi
import workloads as W
from fairseq2_amd.moe import _SCORE_FNS
from tests._util import TORCH_DTYPE, build_module


def _ptr(t):
    return None if t is None else t.data_ptr()


def _layer_args(m, wl, fp8: bool):
    ex = m.experts
    if fp8:
        w = (ex.gate_q, ex.inner_q, ex.output_q)
        s = (ex.gate_scale, ex.inner_scale, ex.output_scale)
    else:
        w = (ex.gate_proj.detach(), ex.inner_proj.detach(), ex.output_proj.detach())
        s = (None, None, None)
    sh = (None, None, None)
    f_shared = 0
    if wl.spec.shared:
        se = m.shared_expert
        sh = (se.gate_proj.weight.detach(), se.inner_proj.weight.detach(), se.output_proj.weight.detach())
        f_shared = sh[0].shape[0]
    return w, s, sh, f_shared


def _both_ways(lib, m, wl, x, residual, fp8: bool, tile_m: int):
    """(fs2moe_forward with a torch workspace, fs2moe_forward_static) on rows x."""
    spec = wl.spec
    w, s, sh, f_shared = _layer_args(m, wl, fp8)
    t, d = x.shape
    f = spec.inner_dim
    act = _abi.dtype_code(x.dtype)
    wdt = _abi.FP8_E4M3 if fp8 else act
    mode = spec.mode
    sizes = (t, d, spec.num_experts, spec.top_k, f, f_shared, tile_m, act)
    need = lib.fs2moe_forward_workspace_bytes(*sizes)
    assert 0 <= need <= lib.fs2moe_forward_static_capacity()
    ws = torch.empty(need, dtype=torch.uint8, device=x.device)
    want = torch.empty_like(x)
    got = torch.empty_like(x)
    stream = torch.cuda.current_stream().cuda_stream
    head = (_ptr(x), _ptr(residual), _ptr(m.router.detach()), _ptr(m.router_bias), *map(_ptr, w), *map(_ptr, s),
            *map(_ptr, sh))
    ints = (t, d, spec.num_experts, spec.top_k, f, f_shared, tile_m, act, wdt, _SCORE_FNS[mode.score_fn],
            int(mode.renormalize), int(mode.scale_on == "input"))
    rc = lib.fs2moe_forward(*head, *ints, _ptr(ws), ws.numel(), _ptr(want), stream)
    assert rc == 0, lib.fs2moe_last_error()
    rc = lib.fs2moe_forward_static(*head, *ints, _ptr(got), stream)
    assert rc == 0, lib.fs2moe_last_error()
    torch.cuda.synchronize()
    return want, got


CASES = [
    # dtype, fp8 weights, mode, shared, tokens (first call, second call), D, E, K, F
    ("bf16", True, W.RoutingMode("softmax", True, "output"), False, (64, 17), 256, 32, 4, 192),  # decode regime
    ("bf16", False, W.RoutingMode("softmax", True, "output"), False, (300, 64), 128, 8, 2, 192),  # fused gather
    ("bf16", False, W.RoutingMode("sigmoid", False, "input"), True, (200, 33), 128, 8, 2, 64),  # reference + shared
    ("fp32", False, W.RoutingMode("sigmoid", False, "input"), False, (77, 5), 64, 8, 3, 72),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,fp8,mode,shared,tokens,d,e,k,f", CASES)
def test_static_scratch_entry_point_equals_forward(gpu_device, dtype, fp8, mode, shared, tokens, d, e, k, f):
    print("forward_static", dtype, fp8, mode, shared, tokens, d, e, k, f, flush=True)
    lib = _abi.load()
    spec = W.small_spec(tokens=tokens[0], model_dim=d, num_experts=e, top_k=k, inner_dim=f, dtype=dtype,
                        weight_dtype="fp8" if fp8 else None, zipf_s=1.1, shared=shared, mode=mode, seed=61)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device, 16)
    big = wl.x.to(TORCH_DTYPE[dtype]).to(gpu_device).reshape(-1, d).contiguous()
    small = big[: tokens[1]].contiguous()
    res_big = torch.flip(big, dims=(0,)).contiguous()
    # first call, then a smaller one over the first call's leftovers, then the first again
    for x, residual in ((big, None), (small, None), (big, res_big), (small, res_big[: tokens[1]].contiguous())):
        want, got = _both_ways(lib, m, wl, x, residual, fp8, 16)
        assert torch.isfinite(got.float()).all()
        assert torch.equal(got, want), f"T={x.shape[0]} residual={residual is not None}"


@pytest.mark.gpu
def test_static_scratch_call_allocates_nothing_and_runs_up_to_its_capacity(gpu_device):
    """After one call on the device (which looks the array's address up and sets function
    attributes), a call changes neither the device's free memory nor torch's allocation count.
    Also the largest token count whose intermediates still fit the array, against fs2moe_forward."""
    print("forward_static at capacity", flush=True)
    lib = _abi.load()
    d, e, k, f, tile_m = 256, 16, 2, 128, 16
    cap = lib.fs2moe_forward_static_capacity()
    need = lambda t: lib.fs2moe_forward_workspace_bytes(t, d, e, k, f, 0, tile_m, _abi.BF16)  # noqa: E731
    lo, hi = 1, 1 << 20
    assert need(lo) <= cap < need(hi)
    while hi - lo > 1:  # need() grows with the token count
        mid = (lo + hi) // 2
        lo, hi = (mid, hi) if need(mid) <= cap else (lo, mid)
    t_max = lo
    assert need(t_max) <= cap < need(t_max + 1)
    spec = W.small_spec(tokens=t_max, model_dim=d, num_experts=e, top_k=k, inner_dim=f, dtype="bf16", zipf_s=1.1,
                        mode=W.RoutingMode("softmax", True, "output"), seed=62)
    wl = W.make_workload_from_spec(spec)
    m = build_module(wl, gpu_device, tile_m)
    x = wl.x.to(torch.bfloat16).to(gpu_device).reshape(-1, d).contiguous()
    want, got = _both_ways(lib, m, wl, x, None, False, tile_m)
    assert torch.equal(got, want), f"T={t_max}, {need(t_max)} of {cap} bytes"
    # one token more is refused
    w, s, sh, _ = _layer_args(m, wl, False)
    out = torch.empty((t_max + 1, d), dtype=torch.bfloat16, device=gpu_device)
    xx = torch.zeros((t_max + 1, d), dtype=torch.bfloat16, device=gpu_device)
    stream = torch.cuda.current_stream().cuda_stream
    args = lambda rows, dst: (  # noqa: E731
        _ptr(rows), None, _ptr(m.router.detach()), _ptr(m.router_bias), *map(_ptr, w), *map(_ptr, s), *map(_ptr, sh),
        rows.shape[0], d, e, k, f, 0, tile_m, _abi.BF16, _abi.BF16, _SCORE_FNS["softmax"], 1, 0, _ptr(dst), stream)
    assert lib.fs2moe_forward_static(*args(xx, out)) == -1
    # a warmed call allocates nothing
    got2 = torch.empty_like(x)
    torch.cuda.synchronize()
    free0, alloc0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    assert lib.fs2moe_forward_static(*args(x, got2)) == 0, lib.fs2moe_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == alloc0
    assert torch.equal(got2, want)


@pytest.mark.gpu
def test_static_scratch_rejects_what_does_not_fit(gpu_device):
    print("forward_static too large", flush=True)
    lib = _abi.load()
    # the prefill shape needs hundreds of megabytes: refused before anything is launched
    x = torch.zeros(16, device=gpu_device)
    p = x.data_ptr()
    rc = lib.fs2moe_forward_static(p, None, p, None, p, p, p, None, None, None, None, None, None, 8192, 2048, 128,
                                   8, 768, 0, 16, _abi.BF16, _abi.BF16, 1, 1, 0, p, None)
    assert rc == -1
    assert "scratch" in lib.fs2moe_last_error().decode()

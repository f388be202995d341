"""CPU-only checks of the C ABI library and the host-side module (no kernel is launched)."""

import ctypes
import os
import re

import pytest
import torch

from fairseq2_amd import _abi
from fairseq2_amd import moe as M
from oracle import moe_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fs2moe.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fs2moe_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_abi.LIB_PATH):
        from fairseq2_amd.build import build_library

        build_library(verbose=False)
    return _abi.load()


def test_library_exports_every_declared_symbol(lib):
    declared = _declared_symbols()
    assert declared, "no declarations found in the header"
    raw = ctypes.CDLL(_abi.LIB_PATH)
    for name in declared:
        assert hasattr(raw, name), f"{name} is declared in fs2moe.h but not exported"
    assert sorted(_abi.EXPORTED_SYMBOLS) == declared, "ctypes prototypes and header disagree"


def test_abi_version_and_limits(lib):
    assert lib.fs2moe_abi_version() == _abi.ABI_VERSION == 15
    assert re.search(rf"#define FS2MOE_ABI_VERSION {_abi.ABI_VERSION}\b", open(HEADER).read())
    text = open(HEADER).read()
    assert f"#define FS2MOE_MAX_EXPERTS {_abi.MAX_EXPERTS}" in text
    assert f"#define FS2MOE_MAX_TOP_K {_abi.MAX_TOP_K}" in text
    for name, val in (("FS2MOE_F32", _abi.F32), ("FS2MOE_BF16", _abi.BF16), ("FS2MOE_FP8_E4M3", _abi.FP8_E4M3)):
        assert re.search(rf"#define {name} {val}\b", text)


def test_header_and_wrapper_agree_on_the_w8a8_option():
    assert re.search(rf"#define FS2MOE_ACT_MXFP8 {hex(_abi.ACT_MXFP8)}\b", open(HEADER).read())
    # the option shares no bit with an element type
    assert _abi.ACT_MXFP8 & (_abi.F32 | _abi.BF16 | _abi.FP8_E4M3) == 0


def test_expert_major_router_is_taken_where_the_library_says_so(lib):
    """ROUTER_OUT_IN: the size rule of fs2moe_router_takes_out_in, the wrapper's choice between the two
    forms, its shape check, and the refusal of the flag elsewhere (host code only)."""
    assert re.search(rf"#define FS2MOE_ROUTER_OUT_IN {hex(_abi.ROUTER_OUT_IN)}\b", open(HEADER).read())
    takes = lib.fs2moe_router_takes_out_in
    assert takes(8192, 2048, 128, _abi.BF16) == 1 and takes(8192, 2048, 128, _abi.F32) == 0
    assert takes(8192, 2048 + 64, 128, _abi.BF16) == 0, "whole steps of 128 features"
    assert takes(8192, 2048, 132, _abi.BF16) == 0 and takes(8192, 2048, 264, _abi.BF16) == 0
    assert takes(32, 2048, 128, _abi.BF16) == 0 and takes(64, 2048, 128, _abi.BF16) == 0
    assert takes(4097, 2048, 128, _abi.BF16) == 1 and takes(33, 128, 8, _abi.BF16) == 1
    x = torch.zeros(8192, 256, dtype=torch.bfloat16)
    r = torch.zeros(256, 16, dtype=torch.bfloat16)
    rt = r.t().contiguous()
    assert _abi.router_operand(lib, x, r, None, _abi.SCORE_SOFTMAX) == (r, _abi.SCORE_SOFTMAX)
    mat, score = _abi.router_operand(lib, x, r, rt, _abi.SCORE_SOFTMAX)
    assert mat is rt and score == (_abi.SCORE_SOFTMAX | _abi.ROUTER_OUT_IN)
    mat, score = _abi.router_operand(lib, x[:16], r, rt, _abi.SCORE_SIGMOID)
    assert mat is r and score == _abi.SCORE_SIGMOID, "few tokens: the (D, E) form"
    with pytest.raises(ValueError, match="router_t"):
        _abi.router_operand(lib, x, r, r, _abi.SCORE_SOFTMAX)  # not transposed
    with pytest.raises(ValueError, match="router_t"):
        _abi.router_operand(lib, x, r, rt.float(), _abi.SCORE_SOFTMAX)
    fake = ctypes.c_void_p(0x1000)
    rc = lib.fs2moe_router_topk(fake, fake, None, 16, 256, 16, 2, _abi.BF16, _abi.SCORE_SIGMOID | _abi.ROUTER_OUT_IN,
                                0, fake, fake, None, None, 0, None)
    assert rc == -1 and b"fs2moe_router_takes_out_in" in lib.fs2moe_last_error()
    assert _abi.router_expert_major(torch.zeros(4, 4)) is None, "no copy of what is not a bf16 matrix on the GPU"


def test_argument_errors_are_reported_without_touching_the_gpu(lib):
    # null pointers
    rc = lib.fs2moe_router_topk(None, None, None, 4, 8, 4, 2, _abi.BF16, 0, 0, None, None, None, None, 0, None)
    assert rc == -1 and b"null" in lib.fs2moe_last_error()
    # E beyond the limit (pointers only need to be non-null: validation comes first)
    fake = ctypes.c_void_p(0x1000)
    rc = lib.fs2moe_router_topk(fake, fake, None, 4, 8, 1000, 2, _abi.BF16, 0, 0, fake, fake, None, None, 0, None)
    assert rc == -1 and b"E=1000" in lib.fs2moe_last_error()
    rc = lib.fs2moe_router_topk(fake, fake, None, 4, 8, 4, 5, _abi.BF16, 0, 0, fake, fake, None, None, 0, None)
    assert rc == -1 and b"K=5" in lib.fs2moe_last_error()
    # dispatch: max_rows below the bound
    rc = lib.fs2moe_dispatch(fake, None, fake, 100, 2, 8, 64, 16, _abi.BF16, 0, 10, fake, fake, fake, fake, fake, fake, 1 << 20, None)
    assert rc == -1 and b"max_rows" in lib.fs2moe_last_error()
    # experts: dims not multiples of 8
    rc = lib.fs2moe_grouped_swiglu(fake, None, fake, fake, fake, fake, fake, None, None, None, 4, 60, 64, 128, _abi.BF16, _abi.BF16, fake, fake, None)
    assert rc == -1 and b"multiples of 8" in lib.fs2moe_last_error()
    # the variant with a bound on the rows per expert checks the same things, and the bound
    rc = lib.fs2moe_grouped_swiglu_rows(fake, None, fake, fake, fake, fake, fake, None, None, None, 4, 60, 64, 128, _abi.BF16, _abi.BF16, fake, fake, 2, None)
    assert rc == -1 and b"multiples of 8" in lib.fs2moe_last_error()
    rc = lib.fs2moe_grouped_swiglu_rows(fake, None, fake, fake, fake, fake, fake, None, None, None, 4, 64, 64, 128, _abi.BF16, _abi.BF16, fake, fake, -1, None)
    assert rc == -1 and b"rows_per_expert" in lib.fs2moe_last_error()
    assert lib.fs2moe_grouped_swiglu_rows(fake, None, fake, fake, fake, fake, fake, None, None, None, 4, 64, 64, 0, _abi.BF16, _abi.BF16, fake, fake, 2, None) == 0
    # the fused gather exists for bf16 activations with D and F multiples of 64 (bf16 or e4m3
    # weights), and nowhere else
    assert lib.fs2moe_grouped_swiglu_fuses_gather(2048, 768, _abi.BF16, _abi.BF16) == 1
    assert lib.fs2moe_grouped_swiglu_fuses_gather(2048, 760, _abi.BF16, _abi.BF16) == 0
    assert lib.fs2moe_grouped_swiglu_fuses_gather(2048, 768, _abi.F32, _abi.F32) == 0
    assert lib.fs2moe_grouped_swiglu_fuses_gather(2048, 768, _abi.BF16, _abi.FP8_E4M3) == 1
    assert lib.fs2moe_grouped_swiglu_fuses_gather(2048, 768, _abi.F32, _abi.FP8_E4M3) == 0
    assert lib.fs2moe_grouped_swiglu_fuses_gather(2048, 0, _abi.BF16, _abi.FP8_E4M3) == 0
    rc = lib.fs2moe_grouped_swiglu(fake, fake, fake, fake, fake, fake, fake, None, None, None, 4, 64, 64, 128, _abi.F32, _abi.F32, fake, fake, None)
    assert rc == -2 and b"fused gather" in lib.fs2moe_last_error()
    # combine: misaligned buffer
    rc = lib.fs2moe_combine(ctypes.c_void_p(0x1004), fake, fake, None, None, 4, 2, 64, _abi.BF16, 0, fake, None)
    assert rc == -1 and b"aligned" in lib.fs2moe_last_error()
    # the whole-layer call: workspace size grows with every dimension, too small a workspace and
    # a half-given shared expert are refused
    need = lib.fs2moe_forward_workspace_bytes(64, 128, 8, 2, 256, 0, 16, _abi.BF16)
    assert need > 0 and need % 256 == 0
    assert lib.fs2moe_forward_workspace_bytes(64, 128, 8, 2, 256, 256, 16, _abi.BF16) > need
    assert lib.fs2moe_forward_workspace_bytes(128, 128, 8, 2, 256, 0, 16, _abi.BF16) > need
    assert lib.fs2moe_forward_workspace_bytes(64, 128, 8, 2, 256, 0, 16, _abi.F32) > need
    assert lib.fs2moe_forward_workspace_bytes(-1, 128, 8, 2, 256, 0, 16, _abi.BF16) == -1
    ws = ctypes.c_void_p(0x10000)
    args = [fake, None] + [fake] * 2 + [fake] * 3 + [None] * 3  # x, residual, router, bias, weights, scales
    tail = [64, 128, 8, 2, 256, 0, 16, _abi.BF16, _abi.BF16, 0, 0, 1]
    out = ctypes.c_void_p(0x2000)
    rc = lib.fs2moe_forward(*args, None, None, None, *tail, ws, need - 1, out, None)
    assert rc == -1 and b"workspace" in lib.fs2moe_last_error()
    rc = lib.fs2moe_forward(*args, fake, None, None, *tail, ws, need, out, None)
    assert rc == -1 and b"shared expert" in lib.fs2moe_last_error()
    rc = lib.fs2moe_forward(*args, None, None, None, *tail, ws, need, fake, None)
    assert rc == -1 and b"alias" in lib.fs2moe_last_error()
    # with a shared expert the output may not overwrite the residual
    args_res = [fake, out] + args[2:]
    tail_sh = [64, 128, 8, 2, 256, 256, 16, _abi.BF16, _abi.BF16, 0, 0, 1]
    need_sh = lib.fs2moe_forward_workspace_bytes(64, 128, 8, 2, 256, 256, 16, _abi.BF16)
    rc = lib.fs2moe_forward(*args_res, fake, fake, fake, *tail_sh, ws, need_sh, out, None)
    assert rc == -1 and b"residual" in lib.fs2moe_last_error()
    rc = lib.fs2moe_combine_residual(fake, fake, fake, None, None, None, 4, 2, 64, _abi.BF16, 0, fake, None)
    assert rc == -1 and b"residual" in lib.fs2moe_last_error()
    rc = lib.fs2moe_forward(*args, None, None, None, *tail, ctypes.c_void_p(0x10010), need, ctypes.c_void_p(0x2000), None)
    assert rc == -1 and b"aligned" in lib.fs2moe_last_error()
    # the variant with the normalisation in front: a larger workspace (the normalised rows), the
    # output may overwrite the input, the router refuses xn == x
    need_n = lib.fs2moe_forward_norm_workspace_bytes(64, 128, 8, 2, 256, 0, 16, _abi.BF16)
    assert need_n >= need + 64 * 128 * 2 and need_n % 256 == 0
    assert lib.fs2moe_forward_norm_workspace_bytes(64, 0, 8, 2, 256, 0, 16, _abi.BF16) == -1
    nargs = [fake, fake, 1e-5, None] + [fake] * 2 + [fake] * 3 + [None] * 3
    rc = lib.fs2moe_forward_norm(*nargs, None, None, None, *tail, ws, need, out, None)
    assert rc == -1 and b"workspace" in lib.fs2moe_last_error()
    tail0 = [0] + tail[1:]  # no tokens: every check passes, nothing is launched
    assert lib.fs2moe_forward_norm(*nargs, None, None, None, *tail0, ws, need_n, fake, None) == 0
    rc = lib.fs2moe_router_topk_norm(fake, fake, 1e-5, fake, fake, None, 4, 8, 4, 2, _abi.BF16, 0, 0, fake, fake, None, None, 0, None)
    assert rc == -1 and b"alias" in lib.fs2moe_last_error()
    rc = lib.fs2moe_router_topk_norm(fake, fake, 1e-5, None, fake, None, 4, 8, 4, 2, _abi.BF16, 0, 0, fake, fake, None, None, 0, None)
    assert rc == -1 and b"xn" in lib.fs2moe_last_error()
    rc = lib.fs2moe_router_topk_norm(fake, fake, -1.0, out, fake, None, 4, 8, 4, 2, _abi.BF16, 0, 0, fake, fake, None, None, 0, None)
    assert rc == -1 and b"norm_eps" in lib.fs2moe_last_error()
    # router scratch: only where several blocks can share a token tile (few tokens, bf16, D >= 512)
    assert lib.fs2moe_router_workspace_bytes(64, 2048, 128, _abi.BF16) == 8 * 64 * 128 * 4
    assert lib.fs2moe_router_workspace_bytes(2048, 2048, 128, _abi.BF16) == 4 * 2048 * 128 * 4
    assert lib.fs2moe_router_workspace_bytes(8192, 2048, 128, _abi.BF16) == 0
    assert lib.fs2moe_router_workspace_bytes(64, 256, 128, _abi.BF16) == 0
    assert lib.fs2moe_router_workspace_bytes(64, 2048, 128, _abi.F32) == 0
    assert lib.fs2moe_router_workspace_bytes(64, 2048, 0, _abi.BF16) == -1
    rc = lib.fs2moe_router_topk(fake, fake, None, 4, 8, 4, 2, _abi.BF16, 0, 0, fake, fake, None, ctypes.c_void_p(0x1004), 64, None)
    assert rc == -1 and b"workspace" in lib.fs2moe_last_error()
    # sizes of zero are a no-op, not an error
    assert lib.fs2moe_router_topk(fake, fake, None, 0, 8, 4, 2, _abi.BF16, 0, 0, fake, fake, None, None, 0, None) == 0
    assert lib.fs2moe_dispatch_workspace_bytes(8192, 8, 128) >= (32 * 128 + 8192 * 8) * 4
    assert lib.fs2moe_dispatch_workspace_bytes(-1, 8, 128) == -1


def test_backward_entry_points_report_argument_errors_without_touching_the_gpu(lib):
    fake, other = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x2000)
    err = lib.fs2moe_last_error
    # plain grouped product: layout, sizes, groups
    rc = lib.fs2moe_grouped_gemm(fake, None, fake, fake, fake, 7, 4, 64, 64, 128, _abi.BF16, fake, None)
    assert rc == -1 and b"layout" in err()
    rc = lib.fs2moe_grouped_gemm(fake, None, fake, fake, fake, _abi.W_IN_OUT, 4, 60, 64, 128, _abi.BF16, fake, None)
    assert rc == -1 and b"multiples of 8" in err()
    rc = lib.fs2moe_grouped_gemm(fake, None, fake, None, fake, _abi.W_IN_OUT, 4, 64, 64, 128, _abi.BF16, fake, None)
    assert rc == -1 and b"counts without offsets" in err()
    rc = lib.fs2moe_grouped_gemm(fake, None, None, None, fake, _abi.W_IN_OUT, 4, 64, 64, 128, _abi.BF16, fake, None)
    assert rc == -1 and b"E=4" in err()  # one matrix without groups
    assert lib.fs2moe_grouped_gemm(fake, None, fake, fake, fake, _abi.W_IN_OUT, 4, 64, 64, 0, _abi.BF16, fake, None) == 0
    # two-source product: only where the throughput kernel runs
    assert lib.fs2moe_grouped_gemm_sum_supported(768, 2048, 65536, _abi.BF16) == 1
    assert lib.fs2moe_grouped_gemm_sum_supported(768, 2048, 65536, _abi.F32) == 0
    assert lib.fs2moe_grouped_gemm_sum_supported(760, 2048, 65536, _abi.BF16) == 0
    rc = lib.fs2moe_grouped_gemm_sum(fake, fake, fake, fake, fake, fake, 4, 760, 2048, 1024, _abi.BF16, fake, None)
    assert rc != 0 and b"grouped_gemm_sum" in err()
    # kept products: bf16 with the throughput kernel's sizes only
    assert lib.fs2moe_grouped_swiglu_keeps(2048, 768, 65536, _abi.BF16) == 1
    assert lib.fs2moe_grouped_swiglu_keeps(2048, 768, 65536, _abi.F32) == 0
    assert lib.fs2moe_grouped_swiglu_keeps(2048, 760, 65536, _abi.BF16) == 0
    # weight gradient
    rc = lib.fs2moe_grouped_wgrad(fake, None, fake, fake, fake, 4, 60, 64, 128, _abi.BF16, fake, None, 0, None)
    assert rc == -1 and b"multiples of 8" in err()
    rc = lib.fs2moe_grouped_wgrad(fake, None, fake, fake, fake, 4, 64, 64, 128, 9, fake, None, 0, None)
    assert rc == -1 and b"dtype 9" in err()
    assert lib.fs2moe_grouped_wgrad_workspace_bytes(1, 2048, 128, 8192) == 0
    assert lib.fs2moe_grouped_wgrad_workspace_bytes(0, 2048, 128, 8192) > 0  # the router's gradient: segments
    assert lib.fs2moe_grouped_wgrad_workspace_bytes(0, 0, 128, 8192) == -1
    # element-wise and per-token steps
    rc = lib.fs2moe_swiglu_backward(fake, fake, fake, 10, 60, _abi.BF16, fake, fake, fake, None)
    assert rc == -1 and b"F=60" in err()
    rc = lib.fs2moe_pair_dot(fake, None, fake, fake, 4, 33, 64, _abi.BF16, fake, None)
    assert rc == -1 and b"K=33" in err()
    rc = lib.fs2moe_router_backward(fake, fake, fake, fake, 4, 1000, 2, 0, 0, _abi.BF16, fake, None)
    assert rc == -1 and b"E=1000" in err()
    rc = lib.fs2moe_router_backward(fake, fake, fake, fake, 4, 8, 2, 5, 0, _abi.BF16, fake, None)
    assert rc == -1 and b"score_fn 5" in err()
    # the normalisation's backward: no aliasing, the weight's gradient needs the weight and scratch
    need = lib.fs2moe_rms_norm_backward_workspace_bytes(100, 64)
    assert need >= 100 * 4 + 3 * 64 * 4 and lib.fs2moe_rms_norm_backward_workspace_bytes(100, 0) == -1
    rc = lib.fs2moe_rms_norm_backward(fake, None, 1e-5, other, 100, 64, _abi.BF16, other, None, None, 0, None)
    assert rc == -1 and b"alias" in err()
    out = ctypes.c_void_p(0x3000)
    rc = lib.fs2moe_rms_norm_backward(fake, None, 1e-5, other, 100, 64, _abi.BF16, out, fake, fake, need, None)
    assert rc == -1 and b"without a weight" in err()
    rc = lib.fs2moe_rms_norm_backward(fake, fake, 1e-5, other, 100, 64, _abi.BF16, out, fake, fake, need - 1, None)
    assert rc == -1 and b"workspace" in err()
    rc = lib.fs2moe_rms_norm_backward(fake, fake, 1e-5, other, 100, 64, 9, out, None, None, 0, None)
    assert rc == -1 and b"dtype 9" in err()
    # no rows and no weight gradient: nothing to launch
    assert lib.fs2moe_rms_norm_backward(fake, fake, 1e-5, other, 0, 64, _abi.BF16, out, None, None, 0, None) == 0


def test_max_rows_matches_the_header_macro():
    # FS2MOE_MAX_ROWS(T, K, E, tile_m) = T*K + E*(tile_m - 1)
    assert _abi.max_rows(8192, 8, 128, 16) == 8192 * 8 + 128 * 15
    assert _abi.max_rows(7, 2, 4, 1) == 14


# ------------------------------------------------------------------------------------ the module
def test_constructor_follows_the_reference_inner_dim_rule():
    # llama4 scout: MoE(5120, int(5120*4*1.2), True, 16, 1.0, 1, inner_dim_scale=2/3, inner_dim_to_multiple=2048)
    with torch.device("meta"):
        m = M.MoE(5120, 24576, True, 16, 1.0, 1, inner_dim_scale=2 / 3, inner_dim_to_multiple=2048)
    assert m.experts.inner_dim == 8192
    assert m.shared_expert.gate_proj.weight.shape == (8192, 5120)
    with torch.device("meta"):
        m = M.MoE(64, 3000, False, 4, 2.0, 2, inner_dim_to_multiple=8)
    assert m.experts.inner_dim == 1000  # int(int(3000*2/3) / 2.0) = 1000, already a multiple of 8
    assert m.shared_expert is None


def test_state_dict_names_and_shapes_match_the_reference_layout():
    with torch.device("meta"):
        m = M.MoE(64, 96, True, 8, 1.0, 2, inner_dim_scale=1.0, auto_scale=False)
    sd = m.state_dict()
    want = {
        "router": (64, 8),
        "experts.gate_proj": (8 * 64, 96),
        "experts.inner_proj": (8 * 64, 96),
        "experts.output_proj": (8 * 96, 64),
        "shared_expert.gate_proj.weight": (96, 64),
        "shared_expert.inner_proj.weight": (96, 64),
        "shared_expert.output_proj.weight": (64, 96),
    }
    assert {k: tuple(v.shape) for k, v in sd.items()} == want
    assert m.top_k == 2 and m.tp_gang is None
    assert m.inner_dim_scale == 1.0 and m.inner_dim_to_multiple == 1
    assert m.experts.num_local_experts == 8


def test_ambient_dtype_and_device_are_honoured():
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("meta"):
            m = M.MoE(64, 64, True, 4, 1.0, 1, inner_dim_scale=1.0, auto_scale=False)
    finally:
        torch.set_default_dtype(prev)
    assert all(p.dtype == torch.bfloat16 and p.is_meta for p in m.parameters())


def test_extension_options_are_validated():
    kw = dict(inner_dim_scale=1.0, auto_scale=False)
    with torch.device("meta"):
        with pytest.raises(ValueError, match="score_fn"):
            M.MoE(64, 64, False, 4, 1.0, 1, score_fn="tanh", **kw)
        with pytest.raises(ValueError, match="scale_on"):
            M.MoE(64, 64, False, 4, 1.0, 1, scale_on="both", **kw)
        with pytest.raises(ValueError, match="top_k"):
            M.MoE(64, 64, False, 4, 1.0, 5, **kw)
        with pytest.raises(ValueError, match="num_experts"):
            M.MoE(64, 64, False, 1000, 1.0, 1, **kw)
        with pytest.raises(ValueError, match="multiples of 8"):
            M.MoE(60, 64, False, 4, 1.0, 1, **kw)
        # any activation module is accepted, as in the reference (experts.py:84-87); only the SiLU
        # gate runs fused
        g = M.MoE(64, 64, False, 4, 1.0, 1, moe_activation=torch.nn.GELU(), **kw)
        assert isinstance(g.experts.activation, torch.nn.GELU) and not g.experts.has_fused_gate
        assert M.MoE(64, 64, False, 4, 1.0, 1, **kw).experts.has_fused_gate
        m = M.MoE(64, 64, False, 4, 1.0, 1, router_bias=True, **kw)
    assert "router_bias" in m.state_dict()


def test_stage_wrappers_check_their_tensors_before_calling_the_library():
    """A tensor of the wrong shape or type must raise on the host: the library takes raw pointers
    and would read it as what it expects.  (Host tensors: every check below fails before a pointer
    is taken.)"""
    e, d, f, t, k = 4, 64, 64, 6, 2
    bf = torch.bfloat16
    xe = torch.zeros(16, d, dtype=bf)
    counts, offsets = torch.zeros(e, dtype=torch.int32), torch.zeros(e + 1, dtype=torch.int32)
    wg, wu, wd = torch.zeros(e * d, f, dtype=bf), torch.zeros(e * d, f, dtype=bf), torch.zeros(e * f, d, dtype=bf)
    idx, w = torch.zeros(t, k, dtype=torch.int32), torch.zeros(t, k)
    inv = torch.zeros(t, k, dtype=torch.int32)
    for fn in (_abi.grouped_swiglu, _abi.grouped_swiglu_keep):
        with pytest.raises(ValueError, match="counts"):
            fn(xe, counts.long(), offsets, wg, wu, wd, e)
        with pytest.raises(ValueError, match="offsets"):
            fn(xe, counts, offsets[:-1], wg, wu, wd, e)
        with pytest.raises(ValueError, match="w_up"):
            fn(xe, counts, offsets, wg, wu.float(), wd, e)
        with pytest.raises(ValueError, match="down weights"):
            fn(xe, counts, offsets, wg, wu, torch.zeros(e * f, d + 8, dtype=bf), e)
        with pytest.raises(ValueError, match="row_map"):
            fn(xe, counts, offsets, wg, wu, wd, e, row_map=torch.zeros(16, dtype=torch.int64))
    for fn in (_abi.dense_swiglu, _abi.dense_swiglu_keep):
        with pytest.raises(ValueError, match="w_gate"):
            fn(xe, torch.zeros(f, d), torch.zeros(f, d, dtype=bf), torch.zeros(d, f, dtype=bf))
        with pytest.raises(ValueError, match="shared-expert weights"):
            fn(xe, torch.zeros(f, d, dtype=bf), torch.zeros(f, d, dtype=bf), torch.zeros(d, f + 8, dtype=bf))
    x = torch.zeros(t, d, dtype=bf)
    with pytest.raises(ValueError, match="topk_idx"):
        _abi.dispatch(idx.long(), w, x, e, 1, False)
    with pytest.raises(ValueError, match="topk_w"):
        _abi.dispatch(idx, w.double(), x, e, 1, False)
    with pytest.raises(ValueError, match="one row per row"):
        _abi.dispatch(idx, w, x[:-1], e, 1, False)
    with pytest.raises(ValueError, match="needs topk_w"):
        _abi.dispatch(idx, None, x, e, 1, True)
    ye = torch.zeros(t * k, d, dtype=bf)
    with pytest.raises(ValueError, match="inv_perm"):
        _abi.combine(ye, inv[:, :1], idx, w, None, True)
    with pytest.raises(ValueError, match="base"):
        _abi.combine(ye, inv, idx, w, x.float(), True)
    with pytest.raises(ValueError, match="out"):
        _abi.combine(ye, inv, idx, w, None, True, out=torch.zeros(t, d + 8, dtype=bf))
    with pytest.raises(ValueError, match="residual"):
        _abi.combine(ye, inv, idx, w, None, True, residual=x[:-1])
    with pytest.raises(ValueError, match="needs topk_w"):
        _abi.combine(ye, inv, idx, None, None, True)
    with pytest.raises(ValueError, match="a2"):
        _abi.grouped_gemm_sum(xe, wg.view(e * f, d), xe.float(), wg.view(e * f, d), counts, offsets, e)
    with pytest.raises(ValueError, match="same number of rows"):
        _abi.grouped_wgrad(xe, xe[:-1].contiguous(), counts, offsets, e)
    with pytest.raises(ValueError, match="dh"):
        _abi.swiglu_backward(xe, xe.clone(), xe.float())


def test_no_cpu_fallback_and_forward_only():
    m = M.MoE(64, 64, False, 4, 1.0, 1, inner_dim_scale=1.0, auto_scale=False)
    x = torch.zeros(2, 3, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        m.requires_grad_(False)(x)
    assert issubclass(M.MoE, M.FeedForwardNetwork)


def test_norm_argument_is_validated_before_anything_runs():
    class Norm:
        def __init__(self, weight, bias, eps, shape):
            self.weight, self.bias, self.eps, self.normalized_shape = weight, bias, eps, shape

    x = torch.zeros(4, 64)
    assert M.MoE._norm_args(None, x) is None
    with pytest.raises(ValueError, match="without bias"):
        M.MoE._norm_args(Norm(None, torch.zeros(64), 1e-5, (64,)), x)
    with pytest.raises(ValueError, match="normalises over"):
        M.MoE._norm_args(Norm(None, None, 1e-5, (32,)), x)
    # no elementwise weight: only eps travels
    assert M.MoE._norm_args(Norm(None, None, 1e-6, (64,)), x) == (None, 1e-6)
    # a weight must live on the GPU like everything else (no CPU fallback)
    with pytest.raises(RuntimeError, match="GPU only"):
        M.MoE._norm_args(Norm(torch.ones(64), None, 1e-5, (64,)), x)


def test_host_mirror_of_the_selection_matches_the_oracle(lib):
    """fs2moe_cpu_router_select on the CPU: the oracle's ordered top-k (ties to the lower expert,
    NaN highest, -0 = +0, -inf selectable last) and weights in all four score modes."""
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(400, 24, generator=g)
    logits[0] = 0.0  # all equal: experts 0..K-1
    logits[1, 3] = float("nan")
    logits[2, 5] = float("inf")
    logits[3, :4] = 1.0
    logits[4, 7] = -0.0
    logits[4, 2] = 0.0
    logits[5, 6:] = float("-inf")
    logits[6] = torch.round(logits[6] * 2) / 2  # many exact ties
    for k in (1, 6, 16):
        for score_fn, renorm, name in ((0, False, "sigmoid"), (0, True, "sigmoid"), (1, False, "softmax"), (1, True, "softmax")):
            idx, w = _abi.cpu_router_select(logits, k, score_fn, renorm)
            ref = O.topk_lowest_index(logits.double(), k)
            assert torch.equal(idx.long(), ref), (k, name, renorm)
            wr = O.combine_weights(logits.double(), ref, name, renorm)
            ok = ~torch.isnan(wr)
            assert torch.allclose(w.double()[ok], wr[ok], rtol=2e-6, atol=1e-7), (k, name, renorm)
            assert bool(torch.isnan(w.double()[~ok]).all())
    # argument errors
    rc = lib.fs2moe_cpu_router_select(logits.data_ptr(), 4, 24, 25, 0, 0, logits.data_ptr(), logits.data_ptr())
    assert rc == -1


def test_fp8_buffers_follow_the_parameters():
    """The e4m3 codes and scales are derived from the Parameters: loading new Parameters drops them,
    clear_fp8_weights() drops them, and Module.to(dtype), which casts floating-point buffers, cannot
    touch them (they are stored as integers and viewed at call time)."""
    m = M.MoE(64, 64, False, 4, 1.0, 2, inner_dim_scale=1.0, auto_scale=False)
    g = torch.Generator().manual_seed(0)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(0.1 * torch.randn(p.shape, generator=g))
    ex = m.experts
    assert not ex.has_fp8_weights
    ex.quantize_fp8_()
    assert ex.has_fp8_weights
    assert ex.gate_q.dtype == torch.float8_e4m3fn and ex.gate_q.shape == (4, 64 // 16, 64 // 64, 16, 64)
    assert ex.output_scale.dtype == torch.float32 and ex.output_scale.shape == (4, 64)
    codes = ex.gate_q.view(torch.uint8).clone()
    m.to(torch.bfloat16)
    assert ex.has_fp8_weights and ex.gate_q.dtype == torch.float8_e4m3fn
    assert torch.equal(ex.gate_q.view(torch.uint8), codes)
    assert ex.gate_scale.dtype == torch.float32
    m.float()
    assert torch.equal(ex.gate_q.view(torch.uint8), codes)
    assert "gate_q" not in m.state_dict() and not any("bits" in k for k in m.state_dict())
    m.load_state_dict(m.state_dict())
    assert not ex.has_fp8_weights, "new Parameters make the derived codes stale"
    ex.quantize_fp8_()
    ex.clear_fp8_weights()
    assert not ex.has_fp8_weights
    with pytest.raises(AttributeError):
        ex.gate_q


def test_fp8_tile_packing_round_trip():
    g = torch.Generator().manual_seed(1)
    q = (50 * torch.randn(3 * 128, 80, generator=g)).to(torch.float8_e4m3fn)
    tiled = _abi.pack_fp8_weights(q, 3)
    assert tiled.shape == (3, 5, 2, 16, 64)
    # tile (e, c, k) holds channels 16 c .. 16 c + 15 (rows) x input features 64 k .. 64 k + 63
    assert tiled.view(torch.uint8)[1, 2, 1, 3, 5] == q.view(torch.uint8)[1 * 128 + 64 + 5, 2 * 16 + 3]
    assert torch.equal(_abi.unpack_fp8_weights(tiled, 3).view(torch.uint8), q.view(torch.uint8))

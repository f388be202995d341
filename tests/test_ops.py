"""The registered torch operator: what a tracing compiler sees of it, without a GPU."""

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

import fairseq2_amd  # noqa: F401  (registers the operator)


def _args(device, dtype=torch.bfloat16, t=5, d=64, e=8, f=32):
    x = torch.empty(t, d, device=device, dtype=dtype)
    router = torch.empty(d, e, device=device, dtype=dtype)
    w_in = torch.empty(e * d, f, device=device, dtype=dtype)
    w_out = torch.empty(e * f, d, device=device, dtype=dtype)
    return (x, router, None, w_in, w_in, w_out) + (None,) * 8 + (e, 2, 16, 0, False, True, False, 0.0)


def test_operator_is_registered_with_a_shape_only_implementation():
    op = torch.ops.fairseq2_amd.moe_forward
    with FakeTensorMode():
        for dtype in (torch.bfloat16, torch.float32):
            out = op(*_args("cuda", dtype))
            assert out.shape == (5, 64) and out.dtype == dtype and out.device.type == "cuda"
    schema = str(op.default._schema)
    assert "Tensor? residual" in schema and "Tensor? norm_weight" in schema and "-> Tensor" in schema


def test_operator_has_no_cpu_implementation():
    with pytest.raises(NotImplementedError):
        torch.ops.fairseq2_amd.moe_forward(*[a.zero_() if isinstance(a, torch.Tensor) else a for a in _args("cpu")])


def test_backward_operator_is_registered_with_a_shape_only_implementation():
    op = torch.ops.fairseq2_amd.moe_backward
    with FakeTensorMode():
        a = _args("cuda")
        x, router, _, w_in, _, w_out = a[:6]
        grads = op(torch.empty_like(x), x, router, None, w_in, w_in, w_out, None, None, None, 8, 2, 16, 0, False, True, None, False, 0.0)
        assert [g.shape for g in grads] == [x.shape, router.shape, w_in.shape, w_in.shape, w_out.shape]
        sg = torch.empty(32, 64, device="cuda", dtype=torch.bfloat16)
        sd = torch.empty(64, 32, device="cuda", dtype=torch.bfloat16)
        grads = op(torch.empty_like(x), x, router, None, w_in, w_in, w_out, sg, sg, sd, 8, 2, 16, 0, False, True,
                   None, False, 0.0)
        assert len(grads) == 8 and grads[7].shape == sd.shape
        nw = torch.empty(64, device="cuda", dtype=torch.bfloat16)
        grads = op(torch.empty_like(x), x, router, None, w_in, w_in, w_out, sg, sg, sd, 8, 2, 16, 0, False, True,
                   nw, True, 1e-5)
        assert len(grads) == 9 and grads[8].shape == nw.shape

"""The dispatcher registration (``torch.ops.ssm_amd.*``): every backend function is declared with the reference's
argument names and defaults and answers shape queries on meta tensors, which is all that tracing needs (no GPU)."""

import torch

from ssm_amd import torch_library as TL


def test_every_backend_function_is_declared():
    assert set(TL.OPERATORS) == {"selective_scan", "selective_scan_backward", "selective_state_step",
                                 "selective_state_step_backward", "ssd_chunk_scan", "ssd_chunk_scan_backward",
                                 "dw_causal_conv", "dw_causal_conv_backward", "fused_layer_norm",
                                 "fused_layer_norm_backward"}
    for name in TL.OPERATORS:
        schema = getattr(torch.ops.ssm_amd, name).default._schema
        assert schema.name == f"ssm_amd::{name}"
    s = torch.ops.ssm_amd.selective_scan.default._schema
    assert [a.name for a in s.arguments] == ["u", "delta", "A", "B", "C", "D", "z", "dt_bias", "softplus",
                                             "return_last_state"]
    step = torch.ops.ssm_amd.selective_state_step.default._schema
    assert step.arguments[0].alias_info is not None and step.arguments[0].alias_info.is_write   # state is updated in place
    assert step.arguments[9].default_value is True                                                # softplus=True


def test_meta_tensors_give_the_shapes_and_dtypes():
    m = lambda *s, dtype=torch.bfloat16: torch.empty(*s, dtype=dtype, device="meta")
    f = lambda *s: torch.empty(*s, dtype=torch.float32, device="meta")
    y, last = torch.ops.ssm_amd.selective_scan(m(2, 8, 64), m(2, 8, 64), f(8, 16), m(2, 1, 16, 64), m(2, 1, 16, 64),
                                               f(8), m(2, 8, 64), f(8), True, True)
    assert y.shape == (2, 8, 64) and y.dtype == torch.bfloat16 and last.shape == (2, 8, 16)
    y, last = torch.ops.ssm_amd.selective_scan(m(2, 8, 64), m(2, 8, 64), f(8, 16), m(2, 1, 16, 64), m(2, 1, 16, 64))
    assert last.numel() == 0
    grads = torch.ops.ssm_amd.selective_scan_backward(m(2, 8, 64), None, m(2, 8, 64), m(2, 8, 64), f(8, 16),
                                                      m(2, 1, 16, 64), m(2, 1, 16, 64), None, m(2, 8, 64), None, True)
    assert [None if g is None else tuple(g.shape) for g in grads] == [(2, 8, 64), (2, 8, 64), (8, 16), (2, 1, 16, 64),
                                                                      (2, 1, 16, 64), None, (2, 8, 64), None]
    assert torch.ops.ssm_amd.selective_state_step(f(2, 8, 16), m(2, 8), m(2, 8), f(8, 16), m(2, 1, 16),
                                                  m(2, 1, 16)).shape == (2, 8)
    Y = torch.ops.ssm_amd.ssd_chunk_scan(m(2, 32, 4, 64), f(2, 32, 4), f(4), m(2, 32, 4, 64), m(2, 32, 4, 64), 16)
    assert Y.shape == (2, 32, 4, 64) and Y.dtype == torch.bfloat16
    assert torch.ops.ssm_amd.dw_causal_conv(m(2, 8, 64), f(8, 4), f(8), "silu").shape == (2, 8, 64)
    dx, dw, db = torch.ops.ssm_amd.dw_causal_conv_backward(m(2, 8, 64), m(2, 8, 64), f(8, 4), None, "silu")
    assert dx.shape == (2, 8, 64) and dw.shape == (8, 4) and db is None
    assert torch.ops.ssm_amd.fused_layer_norm(m(4, 6, 32), f(32), None, f(4, 6, 32), True).shape == (4, 6, 32)
    dx, dw, db, dres = torch.ops.ssm_amd.fused_layer_norm_backward(m(4, 6, 32), m(4, 6, 32), f(32), f(32), None)
    assert dx.shape == (4, 6, 32) and dw.shape == (32,) and db.shape == (32,) and dres is None

"""CPU-only checks of the operator façade: signatures equal the reference's,
docstrings carry Args/Returns, contract violations raise ValueError before any
device is touched, and CPU tensors are refused (there is no CPU compute path)."""

import inspect

import pytest
import torch

from ssm_amd import ops
from ssm_amd.ops import ssd

REFERENCE_SIGNATURES = {
    # src/ssm/ops/__init__.py:1255-1266, :1361-1372, :1484-1495, :1580-1585, :1613-1622
    "selective_scan": ["u", "delta", "A", "B", "C", "D", "z", "dt_bias", "softplus", "return_last_state"],
    "selective_state_step": ["state", "x", "dt", "A", "B", "C", "D", "z", "dt_bias", "softplus"],
    "ssd_chunk_scan": ["X", "dt", "A", "B", "C", "chunk_size", "D", "z", "seq_meta", "initial_states"],
    "dw_causal_conv": ["x", "weight", "bias", "activation"],
    "fused_layer_norm": ["x", "weight", "bias", "residual", "is_rms", "eps", "prenorm", "residual_in_fp32"],
}
REFERENCE_DEFAULTS = {
    "selective_scan": dict(D=None, z=None, dt_bias=None, softplus=False, return_last_state=False),
    "selective_state_step": dict(D=None, z=None, dt_bias=None, softplus=True),
    "ssd_chunk_scan": dict(D=None, z=None, seq_meta=None, initial_states=None),
    "dw_causal_conv": dict(bias=None, activation="silu"),
    "fused_layer_norm": dict(residual=None, is_rms=False, eps=1e-5, prenorm=True, residual_in_fp32=True),
}


@pytest.mark.parametrize("name", sorted(REFERENCE_SIGNATURES))
def test_signatures_match_the_reference(name):
    sig = inspect.signature(getattr(ops, name))
    assert list(sig.parameters) == REFERENCE_SIGNATURES[name]
    for k, v in REFERENCE_DEFAULTS[name].items():
        assert sig.parameters[k].default == v, (name, k)


@pytest.mark.parametrize("fn", [ops.selective_scan, ops.selective_state_step, ops.ssd_chunk_scan, ops.dw_causal_conv,
                                ops.fused_layer_norm, ops.fused_layer_norm_with_residual, ssd.chunk_cumsum,
                                ssd.bmm_chunk, ssd.chunk_state, ssd.state_passing, ssd.chunk_scan, ssd.ssd_combined])
def test_docstrings_have_args_and_returns(fn):
    doc = fn.__doc__ or ""
    assert "Args:" in doc and "Returns:" in doc, fn.__name__


def test_backend_status_records():
    assert ops._cpu_backend_status().available is False
    st = ops._cuda_backend_status()
    assert st.name == "cuda" and isinstance(st.available, bool)
    assert ops._hip_backend_status().name == "hip"


def test_cpu_tensors_are_refused_not_computed():
    u = torch.randn(1, 2, 4)
    A = -torch.rand(2, 3)
    Bm = torch.randn(2, 3)
    with pytest.raises(ops.DeviceError):
        ops.selective_scan(u, u, A, Bm, Bm)
    with pytest.raises(ops.DeviceError):
        ops.dw_causal_conv(u, torch.randn(2, 3))
    with pytest.raises(ops.DeviceError):
        ops.fused_layer_norm(u, torch.ones(4), None)
    with pytest.raises(ops.DeviceError):
        ops.selective_state_step(torch.zeros(1, 2, 3), u[:, :, 0], u[:, :, 0], A, Bm, Bm)
    with pytest.raises(ops.DeviceError):
        ops.ssd_chunk_scan(torch.randn(1, 4, 2, 3), torch.rand(1, 4, 2), A, Bm, Bm, 2)


def test_selective_scan_contract_errors():
    u = torch.randn(2, 4, 8)
    A = -torch.rand(4, 3)
    Bm = torch.randn(4, 3)
    with pytest.raises(ValueError):
        ops.selective_scan(u[0], u[0], A, Bm, Bm)                       # rank
    with pytest.raises(ValueError):
        ops.selective_scan(u, u[:, :, :4], A, Bm, Bm)                  # delta shape
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A[:3], Bm, Bm)                        # A shape
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A, Bm[:, :2], Bm)                     # B shape
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A, torch.randn(2, 3, 3, 8), Bm)       # groups do not divide D
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A, torch.randn(2, 2, 3, 7), Bm)       # L mismatch
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A, Bm, Bm, D=torch.ones(3))
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A, Bm, Bm, z=u[:, :, :4])
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, A, Bm, Bm, dt_bias=torch.ones(5))
    with pytest.raises(ValueError):
        ops.selective_scan(u, u, torch.complex(A, A), Bm, Bm)         # complex tensors: not supported
    with pytest.raises(ValueError):
        ops.selective_scan(u.to(torch.int32), u, A, Bm, Bm)           # not a floating type


def test_compute_type_follows_the_reference():
    """reference.py:9-19, :135-137: the primary tensor's type, 16-bit widened to float32, promoted with A's when
    A is not float32; every other operand is cast to it."""
    from ssm_amd.ops import _contract as K
    f16, bf, f32, f64 = torch.float16, torch.bfloat16, torch.float32, torch.float64
    t = lambda dt: torch.zeros(1, dtype=dt)
    assert not K.f64_compute(t(f32)) and not K.f64_compute(t(bf), t(f32)) and not K.f64_compute(t(f16), t(f16))
    assert K.f64_compute(t(f64)) and K.f64_compute(t(f64), t(f32))
    assert K.f64_compute(t(f32), t(f64)) and K.f64_compute(t(bf), t(f64))
    a, b, c = K.narrow(t(f64), None, t(bf))
    assert a.dtype == f32 and b is None and c.dtype == bf


def test_state_step_contract_errors():
    st = torch.zeros(2, 4, 3)
    x = torch.randn(2, 4)
    A = -torch.rand(4, 3)
    Bm = torch.randn(4, 3)
    with pytest.raises(ValueError):
        ops.selective_state_step(st[0], x, x, A, Bm, Bm)
    with pytest.raises(ValueError):
        ops.selective_state_step(st, x[:, :2], x, A, Bm, Bm)
    with pytest.raises(ValueError):
        ops.selective_state_step(st, x, x, A[:2], Bm, Bm)
    with pytest.raises(ValueError):
        ops.selective_state_step(st, x, x, A, torch.randn(2, 3, 3), Bm)   # 3 groups do not divide 4
    with pytest.raises(ValueError):
        ops.selective_state_step(st, x, x, A, Bm, Bm, z=x[:, :1])


def test_chunk_scan_contract_errors():
    X = torch.randn(2, 6, 2, 3)
    dt = torch.rand(2, 6, 2)
    A = -torch.rand(2, 3)
    Bm = torch.randn(2, 3)
    with pytest.raises(ValueError):
        ops.ssd_chunk_scan(X[0], dt, A, Bm, Bm, 2)
    with pytest.raises(ValueError):
        ops.ssd_chunk_scan(X, dt[:, :3], A, Bm, Bm, 2)
    with pytest.raises(ValueError):
        ops.ssd_chunk_scan(X, dt, torch.rand(3), Bm, Bm, 2)
    with pytest.raises(ValueError):
        ops.ssd_chunk_scan(X, dt, A, Bm[:1], Bm, 2)
    with pytest.raises(ValueError):
        ops.ssd_chunk_scan(X, dt, A, Bm, Bm, 0)
    with pytest.raises(ValueError):
        ops.ssd_chunk_scan(X, dt, A, Bm, Bm, 2, initial_states=torch.zeros(2, 2))


def test_conv_contract_errors():
    x = torch.randn(2, 4, 8)
    with pytest.raises(ValueError):
        ops.dw_causal_conv(x[0], torch.randn(4, 3))
    with pytest.raises(ValueError):
        ops.dw_causal_conv(x, torch.randn(5, 3))                      # channels match neither axis
    with pytest.raises(ValueError):
        ops.dw_causal_conv(x, torch.randn(4, 2, 3))                   # not depthwise
    with pytest.raises(ValueError):
        ops.dw_causal_conv(x, torch.randn(4, 3), bias=torch.zeros(3))
    with pytest.raises(ValueError):
        ops.dw_causal_conv(x, torch.randn(4, 3), activation="relu")


def test_norm_contract_errors():
    x = torch.randn(2, 3, 8)
    with pytest.raises(ValueError):
        ops.fused_layer_norm(x[0], torch.ones(8), None)
    with pytest.raises(ValueError):
        ops.fused_layer_norm(x, torch.ones(7), None)
    with pytest.raises(ValueError):
        ops.fused_layer_norm(x, torch.ones(8), torch.ones(7))
    with pytest.raises(ValueError):
        ops.fused_layer_norm(x, torch.ones(8), None, residual=x[:, :2])


def test_ssd_contract_errors():
    x = torch.randn(2, 6, 4, 3)
    Bm = torch.randn(2, 6, 3, 5)
    with pytest.raises(ValueError):
        ssd.ssd_combined(x, torch.rand(2, 6, 4), -torch.rand(4), Bm, Bm, 3)       # 3 groups do not divide 4 heads
    with pytest.raises(ValueError):
        ssd.chunk_cumsum(torch.rand(2, 6), -torch.rand(4), 3)
    with pytest.raises(ValueError):
        ssd.bmm_chunk(torch.randn(2, 6, 4), torch.randn(2, 6, 5), 3)


def test_sequence_length_metadata():
    from ssm_amd.ops import _contract as K
    dev = torch.device("cpu")
    assert K.sequence_lengths(None, 2, dev) is None
    assert K.sequence_lengths({"seq_lens": [4, 2]}, 2, dev).tolist() == [4, 2]
    assert K.sequence_lengths({"cu_seqlens": torch.tensor([0, 3, 5]), "seq_lens": [9, 9]}, 2, dev).tolist() == [3, 2]
    with pytest.raises(ValueError):
        K.sequence_lengths({"cu_seqlens": torch.tensor([0, 3])}, 2, dev)
    with pytest.raises(ValueError):
        K.sequence_lengths({"seq_lens": [1]}, 2, dev)
    with pytest.raises(ValueError):
        K.sequence_lengths({"other": 1}, 2, dev)

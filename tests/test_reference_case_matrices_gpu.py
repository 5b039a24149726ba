"""The reference's own compiled-backend test, case by case, pointed at this backend.

``/root/reference/tests/ops/test_backend_gradients.py`` compares a compiled backend with the Python reference
path over five option matrices (``_SELECTIVE_SCAN_CPU_CASES``, ``_SELECTIVE_STATE_STEP_CPU_CASES``,
``_SSD_CHUNK_SCAN_CPU_CASES``, ``_DW_CONV_CPU_CASES``, ``_FUSED_LAYER_NORM_CPU_CASES``; :190-351) in float32
and float16, values and every gradient, with its own tolerances (:134-147).  The matrices, shapes (:366, :534,
:686, :863, :962), seeds, element types of every operand (``A`` float32, everything else in the case's type,
``A`` of random sign), the loss (sum of the outputs) and the tolerances are restated here as data; the compiled
backend is the HIP library and the Python path is its restatement in ``oracle/``.
"""

import pytest
import torch

from oracle import ops_oracle as O

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.float16]


def _ops():
    from ssm_amd import ops
    return ops


def _value_tol(dtype):          # _output_tolerances
    return dict(atol=2e-3, rtol=3e-3) if dtype == torch.float16 else dict(atol=1e-4, rtol=1e-4)


def _grad_tol(dtype):           # _grad_tolerances
    return dict(atol=5e-3, rtol=5e-3) if dtype == torch.float16 else dict(atol=1e-4, rtol=1e-4)


def _leaf(t, where):
    if t is None:
        return None
    t = t.detach().clone()
    if where == "gpu":
        t = t.cuda()
    return t.requires_grad_(t.is_floating_point())


def _compare_grads(gpu, cpu, names, dtype):
    for name, a, b in zip(names, gpu, cpu):
        if b is None:
            assert a is None, name
            continue
        assert a.grad is not None and b.grad is not None, name
        assert a.grad.dtype == a.dtype and a.grad.shape == a.shape, name
        torch.testing.assert_close(a.grad.cpu(), b.grad.to(a.grad.dtype), msg=lambda m, n=name: f"grad {n}: {m}",
                                   **_grad_tol(dtype))


SCAN_CASES = {
    "full": dict(return_last_state=True, softplus=True, with_D=True, with_z=True, with_dt_bias=True),
    "minimal": dict(return_last_state=False, softplus=False, with_D=False, with_z=False, with_dt_bias=False),
    "partial": dict(return_last_state=True, softplus=False, with_D=True, with_z=False, with_dt_bias=True),
    "gate-only": dict(return_last_state=False, softplus=True, with_D=False, with_z=True, with_dt_bias=False),
}


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "float16"])
@pytest.mark.parametrize("case", list(SCAN_CASES))
def test_selective_scan_matrix(dtype, case):
    c = SCAN_CASES[case]
    torch.manual_seed(101)
    batch, dim, nstate, length = 2, 3, 4, 5
    u = torch.randn(batch, dim, length).to(dtype)
    delta = torch.randn(batch, dim, length).to(dtype)
    A = torch.randn(dim, nstate)
    Bm, Cm = torch.randn(dim, nstate).to(dtype), torch.randn(dim, nstate).to(dtype)
    D = torch.randn(dim).to(dtype) if c["with_D"] else None
    z = torch.randn(batch, dim, length).to(dtype) if c["with_z"] else None
    bias = torch.randn(dim).to(dtype) if c["with_dt_bias"] else None
    base = (u, delta, A, Bm, Cm, D, z, bias)
    names = ("u", "delta", "A", "B", "C", "D", "z", "dt_bias")
    g = [_leaf(t, "gpu") for t in base]
    r = [_leaf(t, "cpu") for t in base]
    kw = dict(softplus=c["softplus"], return_last_state=c["return_last_state"])
    got = _ops().selective_scan(*g[:5], D=g[5], z=g[6], dt_bias=g[7], **kw)
    want = O.selective_scan(*r[:5], D=r[5], z=r[6], dt_bias=r[7], **kw)
    if not c["return_last_state"]:
        got, want = (got,), (want,)
    for a, b in zip(got, want):
        assert a.dtype == dtype
        torch.testing.assert_close(a.cpu(), b.to(a.dtype), **_value_tol(dtype))
    sum(t.sum() for t in got).backward()
    sum(t.sum() for t in want).backward()
    _compare_grads(g, r, names, dtype)


STEP_CASES = {
    "full": dict(softplus=True, with_D=True, with_z=True, with_dt_bias=True),
    "minimal": dict(softplus=False, with_D=False, with_z=False, with_dt_bias=False),
    "skip-z": dict(softplus=True, with_D=True, with_z=False, with_dt_bias=True),
}


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "float16"])
@pytest.mark.parametrize("case", list(STEP_CASES))
def test_selective_state_step_matrix(dtype, case):
    c = STEP_CASES[case]
    torch.manual_seed(102)
    batch, dim, nstate = 2, 3, 4
    state = torch.randn(batch, dim, nstate).to(dtype)
    x = torch.randn(batch, dim).to(dtype)
    dt = torch.randn(batch, dim).to(dtype)
    A = torch.randn(dim, nstate)
    Bm, Cm = torch.randn(dim, nstate).to(dtype), torch.randn(dim, nstate).to(dtype)
    D = torch.randn(dim).to(dtype) if c["with_D"] else None
    z = torch.randn(batch, dim).to(dtype) if c["with_z"] else None
    bias = torch.randn(dim).to(dtype) if c["with_dt_bias"] else None
    base = (x, dt, A, Bm, Cm, D, z, bias)
    names = ("x", "dt", "A", "B", "C", "D", "z", "dt_bias")
    g = [_leaf(t, "gpu") for t in base]
    r = [_leaf(t, "cpu") for t in base]
    sg, sr = state.clone().cuda(), state.clone()
    got = _ops().selective_state_step(sg, *g[:5], D=g[5], z=g[6], dt_bias=g[7], softplus=c["softplus"])
    # (the oracle's functional form: its in-place form overwrites a float32 state that autograd still needs)
    want, sr = O.selective_state_step_functional(sr, *r[:5], D=r[5], z=r[6], dt_bias=r[7], softplus=c["softplus"])
    torch.testing.assert_close(got.cpu(), want.to(got.dtype), **_value_tol(dtype))
    torch.testing.assert_close(sg.cpu(), sr.to(sg.dtype), **_value_tol(dtype))
    got.sum().backward()
    want.sum().backward()
    _compare_grads(g, r, names, dtype)


CHUNK_CASES = {
    "full": dict(with_D=True, with_z=True, with_seq_meta=True, with_initial_state=True),
    "minimal": dict(with_D=False, with_z=False, with_seq_meta=False, with_initial_state=False),
    "ragged": dict(with_D=False, with_z=True, with_seq_meta=True, with_initial_state=False),
}


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "float16"])
@pytest.mark.parametrize("case", list(CHUNK_CASES))
def test_ssd_chunk_scan_matrix(dtype, case):
    c = CHUNK_CASES[case]
    torch.manual_seed(103)
    batch, seqlen, heads, proj, chunk = 2, 4, 3, 2, 2
    X = torch.randn(batch, seqlen, heads, proj).to(dtype)
    dt = torch.randn(batch, seqlen, heads).to(dtype)
    A = torch.randn(heads, proj)
    Bm, Cm = torch.randn(heads, proj).to(dtype), torch.randn(heads, proj).to(dtype)
    D = torch.randn(heads).to(dtype) if c["with_D"] else None
    z = None
    if c["with_z"]:
        z = torch.randn(*((batch, seqlen, heads, proj) if case == "ragged" else (batch, seqlen, heads))).to(dtype)
    lens = torch.tensor([seqlen, seqlen - 1], dtype=torch.int64) if c["with_seq_meta"] else None
    init = torch.randn(batch, heads, proj).to(dtype) if c["with_initial_state"] else None
    base = (X, dt, A, Bm, Cm, D, z)
    names = ("X", "dt", "A", "B", "C", "D", "z")
    g = [_leaf(t, "gpu") for t in base]
    r = [_leaf(t, "cpu") for t in base]
    got = _ops().ssd_chunk_scan(*g[:5], chunk_size=chunk, D=g[5], z=g[6],
                                seq_meta=None if lens is None else {"seq_lens": lens.cuda()},
                                initial_states=None if init is None else init.cuda())
    want = O.ssd_chunk_scan(*r[:5], chunk, D=r[5], z=r[6], seq_meta=None if lens is None else {"seq_lens": lens},
                            initial_states=init)
    assert got.dtype == dtype
    torch.testing.assert_close(got.cpu(), want.to(got.dtype), **_value_tol(dtype))
    got.sum().backward()
    want.sum().backward()
    _compare_grads(g, r, names, dtype)


CONV_CASES = {"identity-bias": dict(with_bias=True, activation="identity"),
              "silu-no-bias": dict(with_bias=False, activation="silu")}


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "float16"])
@pytest.mark.parametrize("case", list(CONV_CASES))
def test_dw_causal_conv_matrix(dtype, case):
    c = CONV_CASES[case]
    torch.manual_seed(104)
    batch, channels, length, width = 2, 3, 6, 3
    x = torch.randn(batch, channels, length).to(dtype)
    w = torch.randn(channels, width).to(dtype)
    bias = torch.randn(channels).to(dtype) if c["with_bias"] else None
    g = [_leaf(t, "gpu") for t in (x, w, bias)]
    r = [_leaf(t, "cpu") for t in (x, w, bias)]
    got = _ops().dw_causal_conv(g[0], g[1], bias=g[2], activation=c["activation"])
    want = O.dw_causal_conv(r[0], r[1], r[2], activation=c["activation"])
    torch.testing.assert_close(got.cpu(), want.to(got.dtype), **_value_tol(dtype))
    got.sum().backward()
    want.sum().backward()
    _compare_grads(g, r, ("x", "weight", "bias"), dtype)


NORM_CASES = {
    "prenorm-full": dict(with_bias=True, with_residual=True, is_rms=False, prenorm=True, residual_in_fp32=True),
    "postnorm-rms": dict(with_bias=False, with_residual=True, is_rms=True, prenorm=False, residual_in_fp32=False),
    "no-residual": dict(with_bias=True, with_residual=False, is_rms=False, prenorm=False, residual_in_fp32=True),
}


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "float16"])
@pytest.mark.parametrize("case", list(NORM_CASES))
def test_fused_layer_norm_matrix(dtype, case):
    c = NORM_CASES[case]
    torch.manual_seed(105)
    batch, length, hidden = 2, 3, 4
    x = torch.randn(batch, length, hidden).to(dtype)
    w = torch.randn(hidden).to(dtype)
    bias = torch.randn(hidden).to(dtype) if c["with_bias"] else None
    res = torch.randn(batch, length, hidden).to(dtype) if c["with_residual"] else None
    g = [_leaf(t, "gpu") for t in (x, w, bias, res)]
    r = [_leaf(t, "cpu") for t in (x, w, bias, res)]
    kw = dict(is_rms=c["is_rms"], prenorm=c["prenorm"], residual_in_fp32=c["residual_in_fp32"])
    got = _ops().fused_layer_norm(g[0], g[1], g[2], residual=g[3], **kw)
    want = O.fused_layer_norm(r[0], r[1], r[2], residual=r[3], **kw)
    torch.testing.assert_close(got.cpu(), want.to(got.dtype), **_value_tol(dtype))
    got.sum().backward()
    want.sum().backward()
    _compare_grads(g, r, ("x", "weight", "bias", "residual"), dtype)

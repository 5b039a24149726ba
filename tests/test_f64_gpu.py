"""Calls whose compute type is float64 (csrc/f64_ops.hip through ``ops/_f64.py``).

Two kinds of checks.  (1) The reference's own float64 tests of a compiled backend on the device, restated as
data: ``torch.autograd.gradcheck`` on each of the five operators with the seeds, shapes, options and thresholds of
``/root/reference/tests/ops/test_backend_gradients.py:1172-1201`` (selective_scan), ``:1291-1321``
(selective_state_step), ``:1416-1447`` (ssd_chunk_scan), ``:1497-1517`` (dw_causal_conv), ``:1578-1612``
(fused_layer_norm, four variants).  (2) Values and every gradient against the oracle run in float64 on the same
inputs, over the options and broadcast forms each operator accepts, to 1e-10: double precision leaves no room
for a formula that is only nearly right.
"""

import itertools

import pytest
import torch

from oracle import ops_oracle as O

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = dict(rtol=1e-10, atol=1e-10)


def _ops():
    from ssm_amd import ops
    return ops


def _leaf(t, where):
    if t is None:
        return None
    t = t.detach().clone()
    if where == "gpu":
        t = t.cuda()
    return t.requires_grad_(t.is_floating_point())


def _same_grads(gpu, cpu, names):
    for name, a, b in zip(names, gpu, cpu):
        if b is None:
            continue
        assert a.grad is not None, name
        assert a.grad.dtype == a.dtype and a.grad.shape == a.shape, name
        want = b.grad if b.grad is not None else torch.zeros_like(b)
        torch.testing.assert_close(a.grad.cpu(), want.to(a.grad.dtype), msg=lambda m, n=name: f"grad {n}: {m}", **TOL)


# ------------------------------------------------------------------ the reference's gradcheck tests, on the device

def test_selective_scan_gradcheck():
    torch.manual_seed(1)
    batch, dim, nstate, length = 1, 2, 2, 3
    u = torch.randn(batch, dim, length, dtype=F64).cuda().requires_grad_()
    delta = torch.randn(batch, dim, length, dtype=F64).cuda().requires_grad_()
    A, B, C = (torch.randn(dim, nstate, dtype=F64).cuda().requires_grad_() for _ in range(3))

    def func(u, delta, A, B, C):
        out, _ = _ops().selective_scan(u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False,
                                       return_last_state=True)
        return out

    assert torch.autograd.gradcheck(func, (u, delta, A, B, C), eps=1e-4, atol=1e-4)


def test_selective_state_step_gradcheck():
    torch.manual_seed(3)
    batch, dim, nstate = 1, 2, 3
    base_state = torch.zeros(batch, dim, nstate, dtype=F64).cuda()
    x = torch.randn(batch, dim, dtype=F64).cuda().requires_grad_()
    dt = torch.randn(batch, dim, dtype=F64).cuda().requires_grad_()
    A, B, C = (torch.randn(dim, nstate, dtype=F64).cuda().requires_grad_() for _ in range(3))

    def func(x, dt, A, B, C):
        return _ops().selective_state_step(base_state.clone(), x, dt, A, B, C, D=None, z=None, dt_bias=None,
                                           softplus=False)

    assert torch.autograd.gradcheck(func, (x, dt, A, B, C), eps=1e-4, atol=1e-4)


def test_ssd_chunk_scan_gradcheck():
    torch.manual_seed(5)
    batch, seqlen, heads, proj = 1, 3, 1, 2
    X = torch.randn(batch, seqlen, heads, proj, dtype=F64).cuda().requires_grad_()
    dt = torch.randn(batch, seqlen, heads, dtype=F64).cuda().requires_grad_()
    A, B, C = (torch.randn(heads, proj, dtype=F64).cuda().requires_grad_() for _ in range(3))

    def func(X, dt, A, B, C):
        return _ops().ssd_chunk_scan(X, dt, A, B, C, chunk_size=2, D=None, z=None, seq_meta=None, initial_states=None)

    assert torch.autograd.gradcheck(func, (X, dt, A, B, C), eps=1e-4, atol=1e-4)


def test_dw_causal_conv_gradcheck():
    torch.manual_seed(7)
    batch, channels, length, width = 1, 2, 4, 3
    x = torch.randn(batch, channels, length, dtype=F64).cuda().requires_grad_()
    weight = torch.randn(channels, width, dtype=F64).cuda().requires_grad_()
    bias = torch.randn(channels, dtype=F64).cuda().requires_grad_()

    def func(x, weight, bias):
        return _ops().dw_causal_conv(x, weight, bias=bias, activation="identity")

    assert torch.autograd.gradcheck(func, (x, weight, bias), eps=1e-4, atol=1e-4)


@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("prenorm", [False, True])
def test_fused_layer_norm_gradcheck(is_rms, prenorm):
    torch.manual_seed(9)
    batch, length, hidden = 1, 2, 3
    x = torch.randn(batch, length, hidden, dtype=F64).cuda().requires_grad_()
    weight = torch.randn(hidden, dtype=F64).cuda().requires_grad_()
    bias = torch.randn(hidden, dtype=F64).cuda().requires_grad_()
    residual = torch.randn(batch, length, hidden, dtype=F64).cuda().requires_grad_()

    def func(x, weight, bias, residual):
        return _ops().fused_layer_norm(x, weight, bias, residual=residual, is_rms=is_rms, prenorm=prenorm)

    assert torch.autograd.gradcheck(func, (x, weight, bias, residual), eps=1e-4, atol=1e-4)


# ---------------------------------------------------------------------------- against the oracle in float64

SCAN_FORMS = ["DN", "BDN", "BGNL", "BDNL"]


@pytest.mark.parametrize("bform,cform", [("DN", "DN"), ("BDN", "BGNL"), ("BGNL", "BDN"), ("BDNL", "DN"), ("BGNL", "BGNL")])
@pytest.mark.parametrize("full", [True, False])
def test_selective_scan_matches_the_oracle(bform, cform, full):
    torch.manual_seed(11)
    batch, dim, nstate, length = 3, 4, 5, 37

    def proj(form):
        shape = {"DN": (dim, nstate), "BDN": (batch, dim, nstate), "BGNL": (batch, 2, nstate, length),
                 "BDNL": (batch, dim, nstate, length)}[form]
        return torch.randn(shape, dtype=F64)

    u, delta = torch.randn(batch, dim, length, dtype=F64), 0.5 * torch.randn(batch, dim, length, dtype=F64)
    A = -torch.rand(dim, nstate, dtype=F64) - 0.1
    Bm, Cm = proj(bform), proj(cform)
    D = torch.randn(dim, dtype=F64) if full else None
    z = torch.randn(batch, dim, length, dtype=F64) if full else None
    bias = torch.randn(dim, dtype=F64) if full else None
    base = (u, delta, A, Bm, Cm, D, z, bias)
    g = [_leaf(t, "gpu") for t in base]
    r = [_leaf(t, "cpu") for t in base]
    kw = dict(softplus=full, return_last_state=True)
    y, last = _ops().selective_scan(*g[:5], D=g[5], z=g[6], dt_bias=g[7], **kw)
    yr, lastr = O.selective_scan(*r[:5], D=r[5], z=r[6], dt_bias=r[7], **kw)
    assert y.dtype == F64 and last.dtype == F64
    torch.testing.assert_close(y.cpu(), yr, **TOL)
    torch.testing.assert_close(last.cpu(), lastr, **TOL)
    wy, wl = torch.randn(y.shape, dtype=F64), torch.randn(last.shape, dtype=F64)
    ((y * wy.cuda()).sum() + (last * wl.cuda()).sum()).backward()
    ((yr * wy).sum() + (lastr * wl).sum()).backward()
    _same_grads(g, r, ("u", "delta", "A", "B", "C", "D", "z", "dt_bias"))


@pytest.mark.parametrize("bform,cform", [("DN", "DN"), ("BDN", "BGN"), ("BGN", "BDN")])
@pytest.mark.parametrize("full", [True, False])
def test_selective_state_step_matches_the_oracle(bform, cform, full):
    torch.manual_seed(12)
    batch, dim, nstate = 3, 6, 5

    def proj(form):
        return torch.randn({"DN": (dim, nstate), "BDN": (batch, dim, nstate), "BGN": (batch, 2, nstate)}[form], dtype=F64)

    state = torch.randn(batch, dim, nstate, dtype=F64)
    x, dt = torch.randn(batch, dim, dtype=F64), 0.5 * torch.randn(batch, dim, dtype=F64)
    A = -torch.rand(dim, nstate, dtype=F64) - 0.1
    Bm, Cm = proj(bform), proj(cform)
    D = torch.randn(dim, dtype=F64) if full else None
    z = torch.randn(batch, dim, dtype=F64) if full else None
    bias = torch.randn(dim, dtype=F64) if full else None
    base = (state, x, dt, A, Bm, Cm, D, z, bias)
    g = [_leaf(t, "gpu") for t in base]
    r = [_leaf(t, "cpu") for t in base]
    # two steps in a row on the same state tensor: the second differentiates through the first
    sg = g[0].clone()
    y1 = _ops().selective_state_step(sg, *g[1:6], D=g[6], z=g[7], dt_bias=g[8], softplus=full)
    y2 = _ops().selective_state_step(sg, *g[1:6], D=g[6], z=g[7], dt_bias=g[8], softplus=full)
    yr1, s1 = O.selective_state_step_functional(r[0], *r[1:6], D=r[6], z=r[7], dt_bias=r[8], softplus=full)
    yr2, s2 = O.selective_state_step_functional(s1, *r[1:6], D=r[6], z=r[7], dt_bias=r[8], softplus=full)
    torch.testing.assert_close(y1.cpu(), yr1, **TOL)
    torch.testing.assert_close(y2.cpu(), yr2, **TOL)
    torch.testing.assert_close(sg.detach().cpu(), s2.detach(), **TOL)
    w1, w2, ws = torch.randn(y1.shape, dtype=F64), torch.randn(y1.shape, dtype=F64), torch.randn(state.shape, dtype=F64)
    ((y1 * w1.cuda()).sum() + (y2 * w2.cuda()).sum() + (sg * ws.cuda()).sum()).backward()
    ((yr1 * w1).sum() + (yr2 * w2).sum() + (s2 * ws).sum()).backward()
    _same_grads(g, r, ("state", "x", "dt", "A", "B", "C", "D", "z", "dt_bias"))


@pytest.mark.parametrize("aform,bform,cform,dform,zform", [
    ("HP", "HP", "HP", None, None), ("H", "BHP", "BLHP", "H", "BLH"), ("HP", "BLHP", "BHP", "HP", "BLHP"),
    ("H", "BLHP", "BLHP", "H", "BLHP")])
@pytest.mark.parametrize("ragged", [False, True])
def test_ssd_chunk_scan_matches_the_oracle(aform, bform, cform, dform, zform, ragged):
    torch.manual_seed(13)
    batch, seqlen, heads, proj = 3, 29, 2, 4
    shapes = {"H": (heads,), "HP": (heads, proj), "BHP": (batch, heads, proj), "BLHP": (batch, seqlen, heads, proj),
              "BLH": (batch, seqlen, heads)}
    X, dt = torch.randn(shapes["BLHP"], dtype=F64), 0.5 * torch.randn(shapes["BLH"], dtype=F64)
    A = -torch.rand(shapes[aform], dtype=F64) - 0.1
    Bm, Cm = torch.randn(shapes[bform], dtype=F64), torch.randn(shapes[cform], dtype=F64)
    D = torch.randn(shapes[dform], dtype=F64) if dform else None
    z = torch.randn(shapes[zform], dtype=F64) if zform else None
    init = torch.randn(shapes["BHP"], dtype=F64) if ragged else None
    lens = [seqlen, 0, 17] if ragged else None
    base = (X, dt, A, Bm, Cm, D, z, init)
    g = [_leaf(t, "gpu") for t in base]
    r = [_leaf(t, "cpu") for t in base]
    meta = None if lens is None else {"seq_lens": lens}
    y = _ops().ssd_chunk_scan(*g[:5], chunk_size=8, D=g[5], z=g[6], seq_meta=meta, initial_states=g[7])
    yr = O.ssd_chunk_scan(*r[:5], 8, D=r[5], z=r[6], seq_meta=meta, initial_states=r[7])
    assert y.dtype == F64
    torch.testing.assert_close(y.cpu(), yr, **TOL)
    w = torch.randn(y.shape, dtype=F64)
    (y * w.cuda()).sum().backward()
    (yr * w).sum().backward()
    _same_grads(g, r, ("X", "dt", "A", "B", "C", "D", "z", "initial_states"))


@pytest.mark.parametrize("channels_first,width,activation,with_bias,w3", list(itertools.product(
    [True, False], [1, 3, 5], ["silu", "identity"], [True, False], [False])) + [(True, 4, "swish", True, True),
                                                                             (False, 2, "none", False, True)])
def test_dw_causal_conv_matches_the_oracle(channels_first, width, activation, with_bias, w3):
    # the reference's CPU-backend test runs the same grid in float64 (tests/ops/test_cpu_ops.py:89-135)
    torch.manual_seed(14)
    batch, channels, length = 2, 3, 11
    x = torch.randn(batch, channels, length, dtype=F64)
    if not channels_first:
        x = x.permute(0, 2, 1).contiguous()
    w = torch.randn(channels, width, dtype=F64)
    if w3:
        w = w.unsqueeze(1)
    bias = torch.randn(channels, dtype=F64) if with_bias else None
    g = [_leaf(t, "gpu") for t in (x, w, bias)]
    r = [_leaf(t, "cpu") for t in (x, w, bias)]
    y = _ops().dw_causal_conv(g[0], g[1], g[2], activation=activation)
    yr = O.dw_causal_conv(r[0], r[1], r[2], activation=activation)
    assert y.dtype == F64 and y.shape == x.shape
    torch.testing.assert_close(y.cpu(), yr, **TOL)
    wy = torch.randn(y.shape, dtype=F64)
    (y * wy.cuda()).sum().backward()
    (yr * wy).sum().backward()
    _same_grads(g, r, ("x", "weight", "bias"))


@pytest.mark.parametrize("is_rms,prenorm,with_bias,with_res", [
    (False, True, True, True), (True, True, False, True), (False, False, True, True), (True, False, True, True),
    (False, True, True, False), (True, True, False, False)])
def test_fused_layer_norm_matches_the_oracle(is_rms, prenorm, with_bias, with_res):
    torch.manual_seed(15)
    batch, length, hidden = 2, 5, 70
    x = torch.randn(batch, length, hidden, dtype=F64)
    w = torch.randn(hidden, dtype=F64)
    bias = torch.randn(hidden, dtype=F64) if with_bias else None
    res = torch.randn(batch, length, hidden, dtype=F64) if with_res else None
    g = [_leaf(t, "gpu") for t in (x, w, bias, res)]
    r = [_leaf(t, "cpu") for t in (x, w, bias, res)]
    kw = dict(is_rms=is_rms, prenorm=prenorm, eps=1e-6)
    y, ro = _ops().fused_layer_norm_with_residual(g[0], g[1], g[2], residual=g[3], **kw)
    yr, ror = O.fused_layer_norm_with_residual(r[0], r[1], r[2], residual=r[3], acc=F64, **kw)
    assert y.dtype == F64 and ro.dtype == F64
    torch.testing.assert_close(y.cpu(), yr, **TOL)
    torch.testing.assert_close(ro.cpu(), ror, **TOL)
    wy, wr = torch.randn(y.shape, dtype=F64), torch.randn(y.shape, dtype=F64)
    ((y * wy.cuda()).sum() + (ro * wr.cuda()).sum()).backward()
    ((yr * wy).sum() + (ror * wr).sum()).backward()
    _same_grads(g, r, ("x", "weight", "bias", "residual"))
    y1 = _ops().fused_layer_norm(g[0].detach(), g[1].detach(), None if g[2] is None else g[2].detach(),
                                 residual=None if g[3] is None else g[3].detach(), **kw)
    torch.testing.assert_close(y1, y.detach(), rtol=0, atol=0)


# ------------------------------------------------------------------------------------------- mixed types

def test_float64_A_promotes_a_float32_call():
    """reference.py:135-137: a non-float32 ``A`` promotes the compute type; the result keeps ``u``'s type."""
    torch.manual_seed(16)
    batch, dim, nstate, length = 2, 3, 4, 50
    u, delta = torch.randn(batch, dim, length), 0.5 * torch.randn(batch, dim, length)
    A = -torch.rand(dim, nstate, dtype=F64) - 0.1
    Bm, Cm = torch.randn(batch, 1, nstate, length), torch.randn(batch, 1, nstate, length)
    y = _ops().selective_scan(u.cuda(), delta.cuda(), A.cuda(), Bm.cuda(), Cm.cuda(), softplus=True)
    want = O.selective_scan(u, delta, A, Bm, Cm, softplus=True)          # the oracle promotes the same way
    assert y.dtype == torch.float32 and want.dtype == torch.float32
    torch.testing.assert_close(y.cpu(), want, rtol=0, atol=0)            # float64 arithmetic, one rounding at the end


def test_float64_operands_of_a_float32_call_are_narrowed():
    """reference.py:139-160: every operand is cast to the compute type, here float32 (``u`` and ``A`` decide)."""
    torch.manual_seed(17)
    batch, dim, nstate, length = 2, 3, 4, 50
    u, delta = torch.randn(batch, dim, length), 0.5 * torch.randn(batch, dim, length, dtype=F64)
    A = -torch.rand(dim, nstate) - 0.1
    Bm, Cm = torch.randn(dim, nstate, dtype=F64), torch.randn(dim, nstate)
    g = [_leaf(t, "gpu") for t in (u, delta, A, Bm, Cm)]
    y = _ops().selective_scan(*g)
    want = O.selective_scan(u, delta.float(), A, Bm.float(), Cm)
    assert y.dtype == torch.float32
    torch.testing.assert_close(y.cpu(), want, rtol=1e-5, atol=1e-5)
    y.sum().backward()
    assert g[1].grad.dtype == F64 and g[3].grad.dtype == F64 and g[0].grad.dtype == torch.float32


def test_backend_module_functions_take_float64():
    from ssm_amd import backend_module
    be = backend_module.load()
    torch.manual_seed(18)
    batch, dim, nstate, length = 2, 3, 4, 9
    u, delta = torch.randn(batch, dim, length, dtype=F64), 0.5 * torch.randn(batch, dim, length, dtype=F64)
    A = -torch.rand(dim, nstate, dtype=F64) - 0.1
    Bm, Cm = torch.randn(dim, nstate, dtype=F64), torch.randn(dim, nstate, dtype=F64)
    r = [_leaf(t, "cpu") for t in (u, delta, A, Bm, Cm)]
    yr = O.selective_scan(*r)
    go = torch.randn(yr.shape, dtype=F64)
    (yr * go).sum().backward()
    dev = [t.cuda() for t in (u, delta, A, Bm, Cm)]
    y = be.selective_scan(*dev)[0]
    torch.testing.assert_close(y.cpu(), yr.detach(), **TOL)
    grads = be.selective_scan_backward(go.cuda(), None, *dev)
    for name, got, ref in zip(("u", "delta", "A", "B", "C"), grads, r):
        torch.testing.assert_close(got.cpu(), ref.grad, msg=lambda m, n=name: f"grad {n}: {m}", **TOL)

"""GPU parity of ``fused_layer_norm`` forward and backward against the CPU
oracle (autograd through it) and the upstream layer-norm vectors."""

import pytest
import torch

from oracle import ops_oracle as O
from tests import fixtures as fx

pytestmark = pytest.mark.gpu

FP32_TOL = dict(rtol=1e-5, atol=1e-5)
HALF_TOL = dict(rtol=2e-2, atol=2e-2)


def _ops():
    from ssm_amd import ops
    return ops


def cuda(t, grad=False):
    if t is None:
        return None
    t = t.clone().cuda()
    return t.requires_grad_(True) if grad else t


def run_pair(x, w, b, r, **kw):
    g = torch.Generator().manual_seed(17)
    go = torch.randn(x.shape, generator=g).to(x.dtype)
    out = []
    for where in ("gpu", "cpu"):
        if where == "gpu":
            xx, ww, bb, rr, gg = cuda(x, True), cuda(w, True), cuda(b, True), cuda(r, True), go.cuda()
            fn = _ops().fused_layer_norm
        else:
            xx, ww = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
            bb = b.clone().requires_grad_(True) if b is not None else None
            rr = r.clone().requires_grad_(True) if r is not None else None
            gg = go
            fn = O.fused_layer_norm
        y = fn(xx, ww, bb, residual=rr, **kw)
        y.backward(gg)
        out.append(dict(y=y.detach().cpu(), dx=xx.grad.cpu(), dw=ww.grad.cpu(),
                        db=bb.grad.cpu() if bb is not None else None,
                        dr=rr.grad.cpu() if rr is not None else None))
    return out


def check(pair, tol, ptol=None):
    got, want = pair
    for k in ("y", "dx", "dr"):
        if want[k] is not None:
            torch.testing.assert_close(got[k].float(), want[k].float(), **tol)
    for k in ("dw", "db"):
        if want[k] is not None:
            torch.testing.assert_close(got[k].float(), want[k].float(), **(ptol or tol))


def test_upstream_layer_norm_prenorm():
    rec = fx.upstream("layer_norms", "layer_norm_prenorm")
    i = rec["inputs"]
    x, w, b, r = cuda(i["x"], True), cuda(i["w"], True), cuda(i["b"], True), cuda(i["residual"], True)
    y, res_out = _ops().fused_layer_norm_with_residual(x, w, b, residual=r, is_rms=False, eps=1e-6, prenorm=True,
                                                       residual_in_fp32=True)
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(res_out.cpu(), rec["outputs"]["residual_out"], rtol=1e-5, atol=1e-6)
    y.sum().backward()
    for name, t in (("x", x), ("w", w), ("b", b), ("residual", r)):
        torch.testing.assert_close(t.grad.cpu(), rec["gradients"][name], rtol=1e-3, atol=2e-5)


def test_upstream_rms_norm():
    rec = fx.upstream("layer_norms", "rms_norm")
    i = rec["inputs"]
    x, w = cuda(i["x"], True), cuda(i["w"], True)
    y = _ops().fused_layer_norm(x, w, None, is_rms=True, eps=1e-6, prenorm=False, residual_in_fp32=False)
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    y.sum().backward()
    torch.testing.assert_close(x.grad.cpu(), rec["gradients"]["x"], rtol=1e-3, atol=2e-5)
    torch.testing.assert_close(w.grad.cpu(), rec["gradients"]["w"], rtol=1e-3, atol=2e-5)


@pytest.mark.parametrize("hidden", [1, 6, 64, 768, 770, 1024, 1536, 2048, 2500, 4096, 5120, 8192, 8200, 20000])
@pytest.mark.parametrize("is_rms", [False, True])
@pytest.mark.parametrize("prenorm", [True, False])
def test_fp32_matches_oracle(hidden, is_rms, prenorm):
    g = torch.Generator().manual_seed(hidden)
    x = torch.randn(2, 5, hidden, generator=g); r = torch.randn(2, 5, hidden, generator=g)
    w = torch.randn(hidden, generator=g); b = torch.randn(hidden, generator=g)
    check(run_pair(x, w, b, r, is_rms=is_rms, prenorm=prenorm, eps=1e-5), dict(rtol=1e-4, atol=1e-5),
          dict(rtol=1e-4, atol=1e-4))


def test_without_residual_and_bias():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 7, 96, generator=g); w = torch.randn(96, generator=g)
    check(run_pair(x, w, None, None, is_rms=True, eps=1e-5), dict(rtol=1e-4, atol=1e-5), dict(rtol=1e-4, atol=1e-4))
    check(run_pair(x, w, None, None, is_rms=False, eps=1e-5), dict(rtol=1e-4, atol=1e-5), dict(rtol=1e-4, atol=1e-4))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("is_rms", [False, True])
def test_half_input_fp32_residual(dtype, is_rms):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(4, 64, 768, generator=g).to(dtype); r = torch.randn(4, 64, 768, generator=g)
    w = torch.randn(768, generator=g); b = torch.randn(768, generator=g)
    pair = run_pair(x, w, b, r, is_rms=is_rms, prenorm=True, eps=1e-5, residual_in_fp32=True)
    assert pair[0]["y"].dtype == dtype and pair[0]["dr"].dtype == torch.float32
    check(pair, HALF_TOL, dict(rtol=2e-2, atol=0.3))


def test_residual_out_matches_oracle_and_dtype_rules():
    g = torch.Generator().manual_seed(9)
    x = torch.randn(2, 9, 128, generator=g).to(torch.bfloat16); r = torch.randn(2, 9, 128, generator=g)
    w = torch.randn(128, generator=g)
    y, ro = _ops().fused_layer_norm_with_residual(x.cuda(), w.cuda(), None, residual=r.cuda(), is_rms=True)
    yr, ror = O.fused_layer_norm_with_residual(x, w, None, residual=r, is_rms=True)
    assert ro.dtype == torch.float32
    torch.testing.assert_close(ro.cpu(), ror, **FP32_TOL)
    torch.testing.assert_close(y.float().cpu(), yr.float(), **HALF_TOL)


def test_config4_layer_shape_bf16():
    """(16, 2048, 768) bf16 x with an fp32 residual stream, RMSNorm eps 1e-5: the shape of
    one fused add+norm in the 130M model.  Rows are independent, so a row slice is
    replayed on the oracle; dw/db are compared on that slice via linearity in rows."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(16, 2048, 768, generator=g).to(torch.bfloat16)
    r = torch.randn(16, 2048, 768, generator=g)
    w = torch.randn(768, generator=g)
    y, ro = _ops().fused_layer_norm_with_residual(x.cuda(), w.cuda(), None, residual=r.cuda(), is_rms=True)
    sl = slice(0, 2048, 97)
    yr, ror = O.fused_layer_norm_with_residual(x[:, sl], w, None, residual=r[:, sl], is_rms=True)
    torch.testing.assert_close(y[:, sl].float().cpu(), yr.float(), **HALF_TOL)
    torch.testing.assert_close(ro[:, sl].cpu(), ror, **FP32_TOL)


@pytest.mark.parametrize("is_rms", [True, False])
def test_postnorm_backward_with_a_residual_that_needs_no_gradient(is_rms):
    """bf16 x, float32 residual added after the norm, gradient asked for x and the weight only: the typed
    backward reads its stand-in for the unused residual from the residual itself (same type and extent)."""
    g = torch.Generator().manual_seed(8)
    x = torch.randn(3, 37, 768, generator=g).to(torch.bfloat16)
    r = torch.randn(3, 37, 768, generator=g)
    w = torch.randn(768, generator=g)
    gy = torch.randn(3, 37, 768, generator=g).to(torch.bfloat16)
    xg, wg = x.clone().cuda().requires_grad_(True), w.clone().cuda().requires_grad_(True)
    y = _ops().fused_layer_norm(xg, wg, None, residual=r.cuda(), is_rms=is_rms, prenorm=False)
    y.backward(gy.cuda())
    xr, wr = x.clone().float().requires_grad_(True), w.clone().requires_grad_(True)
    yr = O.fused_layer_norm(xr, wr, None, residual=r, is_rms=is_rms, prenorm=False)
    yr.backward(gy.float())
    torch.testing.assert_close(xg.grad.float().cpu(), xr.grad, rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(wg.grad.cpu(), wr.grad, rtol=2e-2, atol=2e-2 * float(wr.grad.abs().max()))

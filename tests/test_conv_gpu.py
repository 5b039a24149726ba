"""GPU parity of ``dw_causal_conv`` forward and backward against the CPU
oracle (autograd through it) and the upstream causal-conv1d vectors."""

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


def run_pair(x, w, b, act, dtype=torch.float32, grads=True):
    """-> (y, dx, dw, db) from the GPU and from the oracle for upstream grad `go`."""
    g = torch.Generator().manual_seed(99)
    go = torch.randn(x.shape, generator=g).to(dtype)
    res = []
    for where in ("gpu", "cpu"):
        xx = x.to(dtype).clone()
        ww, bb, gg = w.clone(), (b.clone() if b is not None else None), go.clone()
        if where == "gpu":
            xx, ww, gg = xx.cuda(), ww.cuda(), gg.cuda()
            bb = bb.cuda() if bb is not None else None
        xx.requires_grad_(grads); ww.requires_grad_(grads)
        if bb is not None:
            bb.requires_grad_(grads)
        fn = _ops().dw_causal_conv if where == "gpu" else O.dw_causal_conv
        y = fn(xx, ww, bb, activation=act)
        if grads:
            y.backward(gg)
            res.append((y.detach().cpu(), xx.grad.cpu(), ww.grad.cpu(), bb.grad.cpu() if bb is not None else None))
        else:
            res.append((y.detach().cpu(), None, None, None))
    return res


def check(res, tol, wtol=None):
    (y, dx, dw, db), (yr, dxr, dwr, dbr) = res
    torch.testing.assert_close(y.float(), yr.float(), **tol)
    if dx is not None:
        torch.testing.assert_close(dx.float(), dxr.float(), **tol)
        wt = wtol or tol
        torch.testing.assert_close(dw, dwr, **wt)
        if db is not None:
            torch.testing.assert_close(db, dbr, **wt)


def test_upstream_channels_first_silu():
    rec = fx.upstream("dw_causal_conv", "channels_first_silu")
    i = rec["inputs"]
    x = i["x"].cuda().requires_grad_(True); w = i["weight"].cuda().requires_grad_(True)
    b = i["bias"].cuda().requires_grad_(True)
    y = _ops().dw_causal_conv(x, w, b, activation="silu")
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    y.sum().backward()
    torch.testing.assert_close(x.grad.cpu(), rec["gradients"]["x"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w.grad.cpu(), rec["gradients"]["weight"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(b.grad.cpu(), rec["gradients"]["bias"], rtol=1e-4, atol=1e-5)


def test_upstream_channels_last_identity():
    rec = fx.upstream("dw_causal_conv", "channels_last_identity")
    i = rec["inputs"]
    x = i["x"].cuda().requires_grad_(True); w = i["weight"].cuda().requires_grad_(True)
    y = _ops().dw_causal_conv(x, w, None, activation="identity")
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    y.sum().backward()
    torch.testing.assert_close(x.grad.cpu(), rec["gradients"]["x"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w.grad.cpu(), rec["gradients"]["weight"], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("K", [1, 2, 3, 4, 5, 7])
@pytest.mark.parametrize("act", ["silu", "identity"])
@pytest.mark.parametrize("shape", [(2, 3, 11), (2, 8, 64), (1, 16, 2048), (3, 5, 1000), (2, 4, 4)],
                         ids=lambda s: "x".join(map(str, s)))
def test_channels_first_fp32(K, act, shape):
    b, c, l = shape
    g = torch.Generator().manual_seed(K * 7 + l)
    x = torch.randn(b, c, l, generator=g); w = torch.rand(c, K, generator=g) - 0.5
    bias = torch.randn(c, generator=g) * 0.02
    check(run_pair(x, w, bias, act), FP32_TOL, dict(rtol=1e-4, atol=1e-4))


@pytest.mark.parametrize("K", [1, 3, 4, 6])
@pytest.mark.parametrize("act", ["swish", "none"])
@pytest.mark.parametrize("shape", [(2, 11, 3), (2, 64, 8), (1, 300, 64), (2, 37, 24)],
                         ids=lambda s: "x".join(map(str, s)))
def test_channels_last_fp32(K, act, shape):
    b, l, c = shape
    g = torch.Generator().manual_seed(K * 5 + l)
    x = torch.randn(b, l, c, generator=g); w = torch.rand(c, 1, K, generator=g) - 0.5
    bias = torch.randn(c, generator=g) * 0.02
    check(run_pair(x, w, bias, act), FP32_TOL, dict(rtol=1e-4, atol=1e-4))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["cf", "cl"])
def test_half(dtype, layout):
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, 32, 256, generator=g) if layout == "cf" else torch.randn(2, 256, 32, generator=g)
    w = torch.rand(32, 4, generator=g) - 0.5
    bias = torch.randn(32, generator=g) * 0.02
    res = run_pair(x, w, bias, "silu", dtype=dtype)
    check(res, HALF_TOL, dict(rtol=2e-2, atol=0.5))


def test_no_bias_and_layout_detection_prefers_channels_first():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(2, 8, 8, generator=g); w = torch.rand(8, 3, generator=g) - 0.5
    check(run_pair(x, w, None, "silu"), FP32_TOL, dict(rtol=1e-4, atol=1e-4))


def test_config1_shape_bf16():
    """B=8, C=1536, L=2048, K=4, bf16, SiLU: forward + backward at full size against
    the oracle on a channel slice (channels are independent)."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(8, 1536, 2048, generator=g).to(torch.bfloat16)
    w = torch.rand(1536, 4, generator=g) - 0.5
    b = torch.randn(1536, generator=g) * 0.02
    go = torch.randn(8, 1536, 2048, generator=g).to(torch.bfloat16)
    xg = x.cuda().requires_grad_(True); wg = w.cuda().requires_grad_(True); bg = b.cuda().requires_grad_(True)
    y = _ops().dw_causal_conv(xg, wg, bg, activation="silu")
    y.backward(go.cuda())
    idx = torch.arange(0, 1536, 128)
    xr = x[:, idx].clone().requires_grad_(True); wr = w[idx].clone().requires_grad_(True)
    br = b[idx].clone().requires_grad_(True)
    yr = O.dw_causal_conv(xr, wr, br, activation="silu")
    yr.backward(go[:, idx])
    torch.testing.assert_close(y[:, idx.cuda()].float().cpu(), yr.float(), **HALF_TOL)
    torch.testing.assert_close(xg.grad[:, idx.cuda()].float().cpu(), xr.grad.float(), **HALF_TOL)
    # weight/bias gradients sum 16384 bf16 products: compare against an fp32 evaluation of the slice
    torch.testing.assert_close(wg.grad[idx.cuda()].cpu(), wr.grad, rtol=2e-2, atol=1.0)
    torch.testing.assert_close(bg.grad[idx.cuda()].cpu(), br.grad, rtol=2e-2, atol=1.0)


def test_channels_last_entry_when_length_equals_channels():
    """A sequence as long as there are channels: the reference's rule reads it channels-first; the entry that names
    the layout convolves along dim 1, forward and backward, like the oracle on the transposed tensor."""
    from ssm_amd import ops
    from oracle import ops_oracle as O
    g = torch.Generator().manual_seed(5)
    n = 24
    x = torch.randn(2, n, n, generator=g)
    w = torch.randn(n, 4, generator=g) * 0.5
    b = torch.randn(n, generator=g) * 0.1
    want = O.dw_causal_conv(x.transpose(1, 2).contiguous(), w, b, activation="silu").transpose(1, 2)
    xg = x.cuda().requires_grad_(True)
    wg, bg = w.cuda().requires_grad_(True), b.cuda().requires_grad_(True)
    y = ops.dw_causal_conv_channels_last(xg, wg, bg, activation="silu")
    torch.testing.assert_close(y.detach().cpu(), want, rtol=1e-5, atol=1e-5)
    assert not torch.allclose(ops.dw_causal_conv(x.cuda(), w.cuda(), b.cuda()).cpu(), want, atol=1e-3)   # channels-first there
    go = torch.randn(2, n, n, generator=g)
    y.backward(go.cuda())
    xr = x.clone().requires_grad_(True)
    wr, br = w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    O.dw_causal_conv(xr.transpose(1, 2), wr, br, activation="silu").transpose(1, 2).backward(go)
    torch.testing.assert_close(xg.grad.cpu(), xr.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(wg.grad.cpu(), wr.grad, rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(bg.grad.cpu(), br.grad, rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ a (B,C,L) view of (B,L,C') rows, as it lies
# The reference's blocks convolve `projected.permute(0, 2, 1)` (src/ssm/modules/mamba1.py:209-215, where `projected`
# is one half of a wider projection; mamba2.py:159-165): a view whose memory runs channels innermost.

def _rows_case(batch, length, chans, wide, K, seed, dtype=torch.float32, offset=0):
    g = torch.Generator().manual_seed(seed)
    proj = torch.randn(batch, length, wide, generator=g).to(dtype)
    w = torch.rand(chans, K, generator=g) - 0.5
    b = torch.randn(chans, generator=g) * 0.1
    go = torch.randn(batch, chans, length, generator=g).to(dtype)
    return proj, w, b, go, (lambda p: p[:, :, offset:offset + chans].permute(0, 2, 1))


@pytest.mark.parametrize("K", [1, 2, 4, 5, 7])
@pytest.mark.parametrize("act,with_bias", [("silu", True), ("identity", False)])
@pytest.mark.parametrize("shape", [(2, 11, 8, 8, 0), (1, 300, 64, 128, 64), (3, 1000, 12, 40, 4), (2, 130, 68, 68, 0),
                                   (1, 5000, 4, 8, 4), (2, 257, 132, 264, 132), (2, 64, 6, 6, 0)],
                         ids=lambda s: "B{}L{}C{}of{}at{}".format(*s))
def test_view_of_rows_fp32(K, act, with_bias, shape):
    """Forward and backward on the view against the oracle on the same view (channel counts that are and are not
    multiples of the tile's 64, lengths that cross tiles and segments, a width the vector kernels do not take, and
    6 channels, which go through a copy)."""
    from ssm_amd import ops
    batch, length, chans, wide, offset = shape
    proj, w, b, go, view = _rows_case(batch, length, chans, wide, K, seed=length + K, offset=offset)
    if not with_bias:
        b = None
    res = []
    for where in ("gpu", "cpu"):
        to = (lambda t: None if t is None else t.cuda()) if where == "gpu" else (lambda t: None if t is None else t.clone())
        p_, w_, b_ = to(proj).requires_grad_(), to(w).requires_grad_(), (to(b).requires_grad_() if b is not None else None)
        fn = ops.dw_causal_conv if where == "gpu" else O.dw_causal_conv
        y = fn(view(p_), w_, b_, activation=act)
        assert y.shape == (batch, chans, length)
        y.backward(to(go))
        res.append((y.detach().cpu(), p_.grad.cpu(), w_.grad.cpu(), b_.grad.cpu() if b is not None else None))
    check(res, FP32_TOL, dict(rtol=1e-4, atol=1e-4))
    taken = ops._conv_rows_view(view(proj.cuda()), True, K)
    assert (taken is not None) == (chans % 4 == 0 and K <= 5 and not view(proj).is_contiguous())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(2, 256, 64, 128, 0), (2, 1001, 72, 144, 72), (8, 2048, 1536, 3072, 0)],
                         ids=lambda s: "B{}L{}C{}of{}at{}".format(*s))
def test_view_of_rows_equals_the_dense_copy(dtype, shape):
    """The kernels that read the view do the arithmetic of the (B,C,L) kernels in the same order: y and dx equal
    those of a dense copy of the view bit for bit; the sums for dweight and dbias are taken in another order."""
    from ssm_amd import ops
    batch, length, chans, wide, offset = shape
    proj, w, b, go, view = _rows_case(batch, length, chans, wide, 4, seed=7, dtype=dtype, offset=offset)
    proj, w, b, go = proj.cuda(), w.cuda(), b.cuda(), go.cuda()
    x = view(proj)
    assert ops._conv_rows_view(x, True, 4) is not None
    y = ops._conv_forward(x, w, b, "silu")
    dx, dw, db = ops._conv_backward(go, x, w, b, "silu")
    xd = x.contiguous()
    yd = ops._conv_forward(xd, w, b, "silu")
    dxd, dwd, dbd = ops._conv_backward(go, xd, w, b, "silu")
    assert y.is_contiguous() and dx.shape == x.shape and dx.stride() == (length * chans, 1, chans)
    assert torch.equal(y, yd)
    assert torch.equal(dx, dxd)
    scale = float(length * batch) ** 0.5
    tol = 1e-5 if dtype == torch.float32 else 1e-4      # two orders of summing the same fp32 terms
    torch.testing.assert_close(dw, dwd, rtol=1e-4, atol=tol * scale)
    torch.testing.assert_close(db, dbd, rtol=1e-4, atol=tol * scale)


def test_view_of_rows_that_starts_off_a_boundary_of_four_channels():
    """Channels 2..65 of a projection: the strides are what the kernels take, the start is not; the call copies the
    view into rows of its own and still returns dx in rows."""
    from ssm_amd import ops
    proj, w, b, go, view = _rows_case(2, 200, 64, 128, 4, seed=3, dtype=torch.bfloat16, offset=2)
    proj, w, b, go = proj.cuda(), w.cuda(), b.cuda(), go.cuda()
    x = view(proj)
    assert ops._conv_rows_view(x, True, 4) is not None and x.data_ptr() % 8 != 0
    y = ops._conv_forward(x, w, b, "silu")
    dx, dw, db = ops._conv_backward(go, x, w, b, "silu")
    xd = x.contiguous()
    assert torch.equal(y, ops._conv_forward(xd, w, b, "silu"))
    dxd, dwd, dbd = ops._conv_backward(go, xd, w, b, "silu")
    assert torch.equal(dx, dxd) and dx.stride() == (200 * 64, 1, 64)
    torch.testing.assert_close(dw, dwd, rtol=1e-4, atol=1e-2)
    torch.testing.assert_close(db, dbd, rtol=1e-4, atol=1e-2)

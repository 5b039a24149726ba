"""``ssm_norm_bwd_static``: the norm backward that allocates nothing on the device (its partial sums live in a
buffer that is part of the library) against ``ssm_norm_bwd`` with a caller's workspace, through the C ABI.
Two calls in a row, the second on a smaller input, so that what the first left in the shared buffer would show;
results must be bit-identical (same kernels, same grid, same order of sums)."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(lib_mod, name, x, res, dy, w, mean, rstd, is_rms, prenorm, with_bias):
    rows, hidden = x.shape
    dx = torch.empty_like(x)
    dres = torch.empty_like(res) if res is not None else None
    dw = torch.empty(hidden, dtype=torch.float32, device=x.device)
    db = torch.empty(hidden, dtype=torch.float32, device=x.device) if with_bias else None
    ws, nbytes = None, 0
    if name == "ssm_norm_bwd":
        nbytes = lib_mod.load().ssm_norm_bwd_workspace_bytes(rows, hidden)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    args = lib_mod.NormBwdArgs(
        x=lib_mod.ptr(x), residual=lib_mod.ptr(res), dy=lib_mod.ptr(dy), weight=lib_mod.ptr(w),
        mean=lib_mod.ptr(mean), rstd=lib_mod.ptr(rstd), dx=lib_mod.ptr(dx), dresidual=lib_mod.ptr(dres),
        dweight=lib_mod.ptr(dw), dbias=lib_mod.ptr(db), workspace=lib_mod.ptr(ws), workspace_bytes=nbytes,
        rows=rows, hidden=hidden, x_dtype=lib_mod.dtype_enum(x.dtype),
        residual_dtype=lib_mod.dtype_enum(res.dtype) if res is not None else 0,
        is_rms=int(is_rms), prenorm=int(prenorm))
    lib_mod.call(name, args, x.device)
    torch.cuda.synchronize()
    return dx, dres, dw, db


def _case(lib_mod, ops, seed, rows, hidden, dtype, is_rms, with_res, with_bias):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
    res = torch.randn(rows, hidden, generator=g).cuda() if with_res else None
    dy = torch.randn(rows, hidden, generator=g).to(dtype).cuda()
    w = (1.0 + 0.1 * torch.randn(hidden, generator=g)).cuda()
    b = (0.1 * torch.randn(hidden, generator=g)).cuda() if with_bias else None
    _, _, mean, rstd = ops._norm_forward(x[None], w, b, None if res is None else res[None], is_rms, 1e-5, True, True,
                                         want_stats=True)
    ref = _run(lib_mod, "ssm_norm_bwd", x, res, dy, w, mean, rstd, is_rms, True, with_bias)
    got = _run(lib_mod, "ssm_norm_bwd_static", x, res, dy, w, mean, rstd, is_rms, True, with_bias)
    for name, a, r in zip(("dx", "dres", "dw", "db"), got, ref):
        assert (a is None) == (r is None), name
        if a is not None:
            assert torch.equal(a, r), f"{name} differs at rows={rows} hidden={hidden}"
    return got


def test_static_norm_backward_matches_workspace_version_on_two_calls_in_a_row():
    from ssm_amd import _lib, ops
    # first a call that fills most of the built-in buffer, then a smaller one that reuses its front
    _case(_lib, ops, 1, 4096, 1024, torch.bfloat16, True, True, False)
    _case(_lib, ops, 2, 300, 768, torch.bfloat16, True, True, False)
    # LayerNorm with bias gradient, fp32, a hidden size that is not a multiple of the vector width
    _case(_lib, ops, 3, 1000, 1536, torch.float32, False, True, True)
    _case(_lib, ops, 4, 37, 101, torch.float32, False, False, True)


def test_static_norm_backward_matches_float64_autograd():
    """Independent of the workspace version: RMSNorm with residual against float64 autograd."""
    from ssm_amd import _lib, ops
    dx, dres, dw, _ = _case(_lib, ops, 5, 513, 768, torch.float32, True, True, False)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(513, 768, generator=g).double().requires_grad_()
    res = torch.randn(513, 768, generator=g).double().requires_grad_()
    dy = torch.randn(513, 768, generator=g).double()
    w = (1.0 + 0.1 * torch.randn(768, generator=g)).double().requires_grad_()
    s = x + res
    y = s * torch.rsqrt((s * s).mean(-1, keepdim=True) + 1e-5) * w
    y.backward(dy)
    torch.testing.assert_close(dx.cpu().double(), x.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dres.cpu().double(), res.grad, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(dw.cpu().double(), w.grad, rtol=1e-4, atol=1e-4)


def test_static_norm_backward_rejects_what_does_not_fit():
    from ssm_amd import _lib
    lib = _lib.load()
    hidden, rows = 4096, 8192                 # 1024 workgroups x 2 x 4096 floats = 32 MiB of partial sums
    x = torch.zeros(rows, hidden, device="cuda")
    w = torch.ones(hidden, device="cuda")
    r = torch.ones(rows, device="cuda")
    dw = torch.empty(hidden, device="cuda")
    args = _lib.NormBwdArgs(x=_lib.ptr(x), dy=_lib.ptr(x), weight=_lib.ptr(w), rstd=_lib.ptr(r), dx=_lib.ptr(x),
                            dweight=_lib.ptr(dw), rows=rows, hidden=hidden, is_rms=1, prenorm=1)
    rc = lib.ssm_norm_bwd_static(ctypes.byref(args), None)
    assert rc == -6
    assert b"built-in buffer" in lib.ssm_amd_last_error()

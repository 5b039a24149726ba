"""The five operators when the compute type is float64.

The reference computes in the promoted type of its inputs (src/ssm/ops/python/reference.py:9-19, :135-137) and
its tests run ``torch.autograd.gradcheck`` in float64 against a compiled backend
(tests/ops/test_backend_gradients.py:1172-1201 and the four tests after it).  The tuned kernels accumulate in
float32; a call whose compute type is float64 comes here and runs the ``ssm_f64_*`` kernels of the same library
(csrc/f64_ops.hip).  What this module does around them is bookkeeping on the device: casts to float64, views of
the projections the reference broadcasts (passed with their strides, 0 on a broadcast axis), and sums of the
dense gradients over those broadcast axes.

Each function mirrors the signature and the result contract of its float32 counterpart in ``ssm_amd.ops`` (the
callers are the same autograd wrappers and backend-module functions); gradients come back in float64 and are cast
to their tensors' types by those callers.
"""

from __future__ import annotations

import torch

from .. import _lib
from . import _contract as K

F64 = torch.float64


def _c(t):
    """Detached float64 contiguous copy-or-view of ``t`` (``None`` stays ``None``)."""
    if t is None:
        return None
    t = t.detach()
    if t.dtype != F64:
        t = t.to(F64)
    return t if t.is_contiguous() else t.contiguous()


def _strides(view, n):
    s = tuple(int(v) for v in view.stride())
    assert len(s) == n
    return (_lib._i64 * n)(*s)


def _new(shape, dev):
    return torch.empty(shape, dtype=F64, device=dev)


# ------------------------------------------------------------------------------------------- selective scan

def _scan_view(p, batch, dim, nstate, length):
    """A projection as a view over ``(B, D, N, L)`` (reference.py:22-56)."""
    p = _c(p)
    if p.ndim == 2:
        return p.view(1, dim, nstate, 1).expand(batch, dim, nstate, length)
    if p.ndim == 3:
        return p.unsqueeze(-1).expand(batch, dim, nstate, length)
    groups = int(p.shape[1])
    if groups != dim:
        p = p.repeat_interleave(dim // groups, dim=1)
    return p


def _scan_reduce(full, like, dim):
    """The dense ``(B, D, N, L)`` gradient of a projection summed back to the projection's shape."""
    if like.ndim == 2:
        return full.sum(dim=(0, 3))
    if like.ndim == 3:
        return full.sum(dim=3)
    groups = int(like.shape[1])
    if groups == dim:
        return full
    b, _, n, l = full.shape
    return full.view(b, groups, dim // groups, n, l).sum(dim=2)


def _scan_args(u, delta, A, B, C, D, z, dt_bias, softplus):
    batch, dim, length, nstate, _, _ = K.check_selective_scan(u, delta, A, B, C, D, z, dt_bias)
    dev = K.require_gpu(u, delta, A, B, C, D, z, dt_bias)
    keep = dict(u=_c(u), delta=_c(delta), z=_c(z), A=_c(A), D=_c(D), bias=_c(dt_bias),
                B=_scan_view(B, batch, dim, nstate, length), C=_scan_view(C, batch, dim, nstate, length))
    keep["last"] = _new((batch, dim, nstate), dev)
    args = _lib.F64ScanArgs(
        u=_lib.ptr(keep["u"]), delta=_lib.ptr(keep["delta"]), z=_lib.ptr(keep["z"]), A=_lib.ptr(keep["A"]),
        Bproj=_lib.ptr(keep["B"]), Cproj=_lib.ptr(keep["C"]), Dskip=_lib.ptr(keep["D"]),
        dt_bias=_lib.ptr(keep["bias"]), last_state=_lib.ptr(keep["last"]),
        b_stride=_strides(keep["B"], 4), c_stride=_strides(keep["C"], 4),
        batch=batch, dim=dim, seqlen=length, nstate=nstate, delta_softplus=int(bool(softplus)))
    return args, keep, dev, (batch, dim, length, nstate)


def scan_forward(u, delta, A, B, C, D, z, dt_bias, softplus, want_state):
    """-> ``(out, last_state | None)`` in ``u.dtype`` (reference.py:194-197)."""
    args, keep, dev, (batch, dim, length, _) = _scan_args(u, delta, A, B, C, D, z, dt_bias, softplus)
    out = _new((batch, dim, length), dev)
    args.out = _lib.ptr(out)
    _lib.call("ssm_f64_scan_fwd", args, dev)
    last = keep["last"] if want_state else None
    if u.dtype != F64:
        out = out.to(u.dtype)
        last = None if last is None else last.to(u.dtype)
    return out, last


def scan_backward(grad_out, grad_last, u, delta, A, B, C, D, z, dt_bias, softplus):
    """-> ``(du, ddelta, dA, dB, dC, dD, dz, ddt_bias)`` in float64, each with its tensor's shape."""
    args, keep, dev, (batch, dim, length, nstate) = _scan_args(u, delta, A, B, C, D, z, dt_bias, softplus)
    go, gl = _c(grad_out), _c(grad_last)
    states, ypre = _new((batch, dim, length, nstate), dev), _new((batch, dim, length), dev)
    du, ddl = _new((batch, dim, length), dev), _new((batch, dim, length), dev)
    dz = _new((batch, dim, length), dev) if z is not None else None
    dA_rows = _new((batch, dim, nstate), dev)
    dB, dC = _new((batch, dim, nstate, length), dev), _new((batch, dim, nstate, length), dev)
    dD_rows = _new((batch, dim), dev) if D is not None else None
    db_rows = _new((batch, dim), dev) if dt_bias is not None else None
    args.dout, args.dlast_state = _lib.ptr(go), _lib.ptr(gl)
    args.states, args.ypre = _lib.ptr(states), _lib.ptr(ypre)
    args.du, args.ddelta, args.dz = _lib.ptr(du), _lib.ptr(ddl), _lib.ptr(dz)
    args.dA_rows, args.dB, args.dC = _lib.ptr(dA_rows), _lib.ptr(dB), _lib.ptr(dC)
    args.dD_rows, args.dbias_rows = _lib.ptr(dD_rows), _lib.ptr(db_rows)
    _lib.call("ssm_f64_scan_bwd", args, dev)
    return (du, ddl, dA_rows.sum(0), _scan_reduce(dB, B, dim), _scan_reduce(dC, C, dim),
            None if dD_rows is None else dD_rows.sum(0), dz, None if db_rows is None else db_rows.sum(0))


# ------------------------------------------------------------------------------------- selective state step

def _step_view(p, batch, dim, nstate):
    """A projection as a view over ``(B, D, N)``; a 3-D tensor whose second axis is not ``D`` is grouped
    (reference.py:252-272)."""
    p = _c(p)
    if p.ndim == 2:
        return p.view(1, dim, nstate).expand(batch, dim, nstate)
    if int(p.shape[1]) != dim:
        p = p.repeat_interleave(dim // int(p.shape[1]), dim=1)
    return p


def _step_reduce(full, like, dim):
    if like.ndim == 2:
        return full.sum(dim=0)
    groups = int(like.shape[1])
    if groups == dim:
        return full
    b, _, n = full.shape
    return full.view(b, groups, dim // groups, n).sum(dim=2)


def _step_args(state64, x, dt, A, B, C, D, z, dt_bias, softplus, dims, dev):
    batch, dim, nstate = dims
    keep = dict(x=_c(x), dt=_c(dt), z=_c(z), A=_c(A), D=_c(D), bias=_c(dt_bias),
                B=_step_view(B, batch, dim, nstate), C=_step_view(C, batch, dim, nstate))
    args = _lib.F64StepArgs(
        state=_lib.ptr(state64), x=_lib.ptr(keep["x"]), dt=_lib.ptr(keep["dt"]), z=_lib.ptr(keep["z"]),
        A=_lib.ptr(keep["A"]), Bproj=_lib.ptr(keep["B"]), Cproj=_lib.ptr(keep["C"]), Dskip=_lib.ptr(keep["D"]),
        dt_bias=_lib.ptr(keep["bias"]), b_stride=_strides(keep["B"], 3), c_stride=_strides(keep["C"], 3),
        batch=batch, dim=dim, nstate=nstate, dt_softplus=int(bool(softplus)))
    return args, keep


def state_step(state, x, dt, A, B, C, D, z, dt_bias, softplus):
    """Updates ``state`` in place (in its own type); -> ``y (B, D)`` in float64."""
    batch, dim, nstate, _, _ = K.check_state_step(state, x, dt, A, B, C, D, z, dt_bias)
    dev = K.require_gpu(state, x, dt, A, B, C, D, z, dt_bias)
    in_place = state.dtype == F64 and state.is_contiguous()
    work = state.detach() if in_place else _c(state).clone()
    args, keep = _step_args(work, x, dt, A, B, C, D, z, dt_bias, softplus, (batch, dim, nstate), dev)
    out = _new((batch, dim), dev)
    args.out = _lib.ptr(out)
    _lib.call("ssm_f64_state_step", args, dev)
    if not in_place:
        state.detach().copy_(work)
    return out


def state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D, z, dt_bias, softplus):
    """-> gradients of ``(state, x, dt, A, B, C, D, z, dt_bias)`` in float64; ``state`` is the state before the step."""
    batch, dim, nstate, _, _ = K.check_state_step(state, x, dt, A, B, C, D, z, dt_bias)
    dev = K.require_gpu(state, x, dt, A, B, C, D, z, dt_bias, grad_out, grad_state)
    sc = _c(state)
    args, keep = _step_args(sc, x, dt, A, B, C, D, z, dt_bias, softplus, (batch, dim, nstate), dev)
    go, gs = _c(grad_out), _c(grad_state)
    dstate = _new((batch, dim, nstate), dev)
    dx, ddt = _new((batch, dim), dev), _new((batch, dim), dev)
    dz = _new((batch, dim), dev) if z is not None else None
    dA_rows, dB, dC = (_new((batch, dim, nstate), dev) for _ in range(3))
    dD_rows = _new((batch, dim), dev) if D is not None else None
    args.dout, args.dstate_new = _lib.ptr(go), _lib.ptr(gs)
    args.dstate, args.dx, args.ddt, args.dz = _lib.ptr(dstate), _lib.ptr(dx), _lib.ptr(ddt), _lib.ptr(dz)
    args.dA_rows, args.dB, args.dC, args.dD_rows = _lib.ptr(dA_rows), _lib.ptr(dB), _lib.ptr(dC), _lib.ptr(dD_rows)
    _lib.call("ssm_f64_state_step_bwd", args, dev)
    return (dstate, dx, ddt, dA_rows.sum(0), _step_reduce(dB, B, dim), _step_reduce(dC, C, dim),
            None if dD_rows is None else dD_rows.sum(0), dz, ddt.sum(0) if dt_bias is not None else None)


# ---------------------------------------------------------------------------------- diagonal chunk scan

def _chunk_view(p, batch, seqlen, heads, proj):
    """A projection ``(H, P)``, ``(B, H, P)`` or ``(B, L, H, P)`` as a view over ``(B, L, H, P)`` (reference.py:59-85)."""
    p = _c(p)
    if p.ndim == 2:
        return p.view(1, 1, heads, proj).expand(batch, seqlen, heads, proj)
    if p.ndim == 3:
        return p.unsqueeze(1).expand(batch, seqlen, heads, proj)
    return p


def _per_channel(p, heads, proj):
    """``(H,)`` or ``(H, P)`` -> dense ``(H, P)``."""
    p = _c(p)
    return p[:, None].expand(heads, proj).contiguous() if p.ndim == 1 else p


def _dscan_args(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states):
    batch, seqlen, heads, proj, *_ = K.check_chunk_scan(X, dt, A, B, C, chunk_size, D, z, initial_states)
    dev = K.require_gpu(X, dt, A, B, C, D, z, initial_states)
    zv = None                               # a gate per head (B, L, H) or per channel (B, L, H, P)
    if z is not None:
        zc = _c(z)
        zv = zc.unsqueeze(-1).expand(batch, seqlen, heads, proj) if zc.ndim == 3 else zc
    keep = dict(X=_c(X), dt=_c(dt), A=_per_channel(A, heads, proj),
                D=None if D is None else _per_channel(D, heads, proj), z=zv, init=_c(initial_states),
                B=_chunk_view(B, batch, seqlen, heads, proj), C=_chunk_view(C, batch, seqlen, heads, proj))
    args = _lib.F64DscanArgs(
        X=_lib.ptr(keep["X"]), dt=_lib.ptr(keep["dt"]), A=_lib.ptr(keep["A"]), Bproj=_lib.ptr(keep["B"]),
        Cproj=_lib.ptr(keep["C"]), Dskip=_lib.ptr(keep["D"]), z=_lib.ptr(zv), init=_lib.ptr(keep["init"]),
        lengths=_lib.ptr(lengths), b_stride=_strides(keep["B"], 4), c_stride=_strides(keep["C"], 4),
        z_stride=_strides(zv, 4) if zv is not None else (_lib._i64 * 4)(0, 0, 0, 0),
        batch=batch, seqlen=seqlen, heads=heads, hdim=proj)
    return args, keep, dev, (batch, seqlen, heads, proj)


def dscan_forward(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states):
    """-> ``Y (B, L, H, P)`` in ``X.dtype`` (reference.py:477-480)."""
    args, keep, dev, dims = _dscan_args(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)
    Y = _new(dims, dev)
    args.Y = _lib.ptr(Y)
    _lib.call("ssm_f64_dscan_fwd", args, dev)
    return Y if X.dtype == F64 else Y.to(X.dtype)


def _chunk_reduce(full, like, batch, heads, proj):
    if like.ndim == 2:
        return full.sum(dim=(0, 1))
    if like.ndim == 3:
        return full.sum(dim=1)
    return full


def dscan_backward(grad_y, X, dt, A, B, C, chunk_size, D, z, lengths, initial_states):
    """-> ``(dX, ddt, dA, dB, dC, dD, dz, dinitial_states)`` in float64, each with its tensor's shape."""
    args, keep, dev, dims = _dscan_args(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)
    batch, seqlen, heads, proj = dims
    gy = _c(grad_y)
    states = _new(dims, dev)
    dX, ddt_rows, dB, dC = (_new(dims, dev) for _ in range(4))
    dz = _new(dims, dev) if z is not None else None
    dA_rows = _new((batch, heads, proj), dev)
    dD_rows = _new((batch, heads, proj), dev) if D is not None else None
    dinit = _new((batch, heads, proj), dev) if initial_states is not None else None
    args.dY, args.states = _lib.ptr(gy), _lib.ptr(states)
    args.dX, args.ddt_rows, args.dB, args.dC, args.dz = (_lib.ptr(dX), _lib.ptr(ddt_rows), _lib.ptr(dB), _lib.ptr(dC),
                                                         _lib.ptr(dz))
    args.dA_rows, args.dD_rows, args.dinit = _lib.ptr(dA_rows), _lib.ptr(dD_rows), _lib.ptr(dinit)
    _lib.call("ssm_f64_dscan_bwd", args, dev)
    dA = dA_rows.sum(0)
    if A.ndim == 1:
        dA = dA.sum(-1)
    dD = None
    if D is not None:
        dD = dD_rows.sum(0)
        if D.ndim == 1:
            dD = dD.sum(-1)
    if dz is not None and z.ndim == 3:
        dz = dz.sum(-1)
    return (dX, ddt_rows.sum(-1), dA, _chunk_reduce(dB, B, batch, heads, proj), _chunk_reduce(dC, C, batch, heads, proj),
            dD, dz, dinit)


# ------------------------------------------------------------------------------ depthwise causal convolution

def _conv_args(x, weight, bias, activation, channels_last):
    batch, chans, length, width, channels_first, silu = K.check_conv(x, weight, bias, activation, channels_last)
    dev = K.require_gpu(x, weight, bias)
    xc = _c(x)
    w = weight.detach()
    wc = _c(w[:, 0, :] if w.ndim == 3 else w)
    bcl = (lambda t: t) if channels_first else (lambda t: t.permute(0, 2, 1))
    keep = dict(x=xc, w=wc, bias=_c(bias))
    args = _lib.F64ConvArgs(
        x=_lib.ptr(xc), weight=_lib.ptr(wc), bias=_lib.ptr(keep["bias"]), x_stride=_strides(bcl(xc), 3),
        batch=batch, channels=chans, seqlen=length, width=width,
        activation=_lib.ACT_SILU if silu else _lib.ACT_IDENTITY)
    return args, keep, dev, bcl, (batch, chans, length, width)


def conv_forward(x, weight, bias, activation, channels_last=None):
    """-> ``y`` with the layout and type of ``x`` (reference.py:483-533)."""
    args, keep, dev, bcl, _ = _conv_args(x, weight, bias, activation, channels_last)
    y = torch.empty_like(keep["x"])
    args.y, args.y_stride = _lib.ptr(y), _strides(bcl(y), 3)
    _lib.call("ssm_f64_conv_fwd", args, dev)
    return y if x.dtype == F64 else y.to(x.dtype)


def conv_backward(grad_out, x, weight, bias, activation, channels_last=None):
    """-> ``(dx, dweight (C, K), dbias (C,) | None)`` in float64."""
    args, keep, dev, bcl, (batch, chans, length, width) = _conv_args(x, weight, bias, activation, channels_last)
    gy = _c(grad_out)
    dx = torch.empty_like(keep["x"])
    dpre = _new((batch, chans, length), dev)
    dw = _new((chans, width), dev)
    db = _new((chans,), dev) if bias is not None else None
    args.dy, args.dy_stride = _lib.ptr(gy), _strides(bcl(gy), 3)
    args.dx, args.dx_stride = _lib.ptr(dx), _strides(bcl(dx), 3)
    args.dpre, args.dw, args.db = _lib.ptr(dpre), _lib.ptr(dw), _lib.ptr(db)
    _lib.call("ssm_f64_conv_bwd", args, dev)
    return dx, dw, db


# ---------------------------------------------------------------------- residual add + LayerNorm / RMSNorm

def norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, want_residual_out=False):
    """-> ``(y, residual_out | None, mean, rstd)``: ``y`` in ``x.dtype``, the rest in float64.  The sum with the
    residual is formed in float64 whatever ``residual_in_fp32`` says (the reference would narrow a float64 sum
    to float32 there, reference.py:575-578; keeping the wider type is the more accurate reading of the flag)."""
    rows, hidden = K.check_norm(x, weight, bias, residual)
    dev = K.require_gpu(x, weight, bias, residual)
    xc, rc, wc, bc = _c(x), _c(residual), _c(weight), _c(bias)
    y = torch.empty_like(xc)
    res_out = torch.empty_like(xc) if want_residual_out else None
    mean, rstd = _new((rows,), dev), _new((rows,), dev)
    args = _lib.F64NormArgs(
        x=_lib.ptr(xc), residual=_lib.ptr(rc), weight=_lib.ptr(wc), bias=_lib.ptr(bc), y=_lib.ptr(y),
        residual_out=_lib.ptr(res_out), mean=_lib.ptr(mean), rstd=_lib.ptr(rstd), rows=rows, hidden=hidden,
        is_rms=int(bool(is_rms)), prenorm=int(bool(prenorm)), eps=float(eps))
    _lib.call("ssm_f64_norm_fwd", args, dev)
    return (y if x.dtype == F64 else y.to(x.dtype)), res_out, mean, rstd


def norm_backward(grad_out, x, weight, residual, mean, rstd, is_rms, prenorm, want_dbias, want_dres):
    """-> ``(dx, dresidual | None, dweight, dbias | None)`` in float64."""
    rows, hidden = K.check_norm(x, weight, None, residual)
    dev = K.require_gpu(x, weight, residual, grad_out)
    xc, rc, wc, gy, mc, sc = _c(x), _c(residual), _c(weight), _c(grad_out), _c(mean), _c(rstd)
    dx = torch.empty_like(xc)
    dres = torch.empty_like(xc) if (want_dres and rc is not None) else None
    dw = _new((hidden,), dev)
    db = _new((hidden,), dev) if want_dbias else None
    args = _lib.F64NormArgs(
        x=_lib.ptr(xc), residual=_lib.ptr(rc), weight=_lib.ptr(wc), mean=_lib.ptr(mc), rstd=_lib.ptr(sc),
        dy=_lib.ptr(gy), dx=_lib.ptr(dx), dresidual=_lib.ptr(dres), dw=_lib.ptr(dw), db=_lib.ptr(db),
        rows=rows, hidden=hidden, is_rms=int(bool(is_rms)), prenorm=int(bool(prenorm)), eps=0.0)
    _lib.call("ssm_f64_norm_bwd", args, dev)
    return dx, dres, dw, db

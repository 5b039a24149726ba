"""Operator façade of the MI355X backend.

Mirrors the public surface of the reference's ``ssm.ops``
(src/ssm/ops/__init__.py:1255-1701): the same five functions with the same
signatures, broadcasting rules, in-place behaviour and ``ValueError`` contract,
plus the two backend-status probes.  Every call runs hand-written gfx950
kernels through the C ABI in ``include/ssm_amd.h``; there is no Python or CPU
compute path behind these functions.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from .. import _lib
from . import _contract as K
from ._contract import DeviceError


@dataclass(frozen=True)
class _BackendCandidate:
    """Same shape as the reference's status record (src/ssm/ops/__init__.py:32-35)."""
    name: str
    available: bool


def _hip_backend_status() -> _BackendCandidate:
    ok = _lib.available() and torch.cuda.is_available()
    return _BackendCandidate(name="hip", available=ok)


def _cuda_backend_status() -> _BackendCandidate:
    """ROCm devices report as ``cuda``; this is the slot the HIP backend fills."""
    return _BackendCandidate(name="cuda", available=_hip_backend_status().available)


def _cpu_backend_status() -> _BackendCandidate:
    """There is no CPU backend in this package."""
    return _BackendCandidate(name="cpu", available=False)


# ---------------------------------------------------------------------------
# selective scan
# ---------------------------------------------------------------------------

class ScanPlan:
    """A fully prepared ``ssm_scan_fwd`` call: argument struct, the tensors it
    points into (kept alive here) and the output buffers.  ``run()`` may be
    called repeatedly; it enqueues one launch on the current stream."""

    def __init__(self, u, delta, A, B, C, D, z, dt_bias, softplus, want_state, tune_items=0,
                 out=None, last=None, want_chunk_states=False):
        batch, dim, length, nstate, (bkind, bgroups), (ckind, cgroups) = \
            K.check_selective_scan(u, delta, A, B, C, D, z, dt_bias)
        self.device = K.require_gpu(u, delta, A, B, C, D, z, dt_bias)
        self.result_dtype = u.dtype
        self.chunk_states = None
        self.f64 = None
        if K.f64_compute(u, A):           # computed in double precision by kernels of their own
            self.f64 = (u, delta, A, B, C, D, z, dt_bias, softplus, want_state)
            return
        u, delta, A, B, C, D, z, dt_bias = K.narrow(u, delta, A, B, C, D, z, dt_bias)
        io = K.common_io_dtype([u, delta, z])
        bc = K.common_io_dtype([B, C])
        self.result_dtype = u.dtype
        self.keep = dict(u=K.cast_c(u, io), delta=K.cast_c(delta, io), z=K.cast_c(z, io),
                         B=K.cast_c(B, bc), C=K.cast_c(C, bc), A=K.as_f32_vec(A),
                         D=K.as_f32_vec(D), bias=K.as_f32_vec(dt_bias))
        k = self.keep
        self.out = out if out is not None else torch.empty_like(k["u"])
        self.last = last
        if want_state and last is None:
            self.last = torch.empty(batch, dim, nstate, dtype=io, device=self.device)
        self.chunk_states = None
        if want_chunk_states:
            chunk = _lib.load().ssm_scan_chunk_len()
            nchunks = (length + chunk - 1) // chunk
            self.chunk_states = torch.empty(batch, dim, nchunks, nstate, dtype=torch.float32,
                                            device=self.device)
        self.args = _lib.ScanFwdArgs(
            u=_lib.ptr(k["u"]), delta=_lib.ptr(k["delta"]), z=_lib.ptr(k["z"]), A=_lib.ptr(k["A"]),
            Bproj=_lib.ptr(k["B"]), Cproj=_lib.ptr(k["C"]), Dskip=_lib.ptr(k["D"]),
            dt_bias=_lib.ptr(k["bias"]), out=_lib.ptr(self.out), last_state=_lib.ptr(self.last),
            chunk_states=_lib.ptr(self.chunk_states),
            batch=batch, dim=dim, seqlen=length, nstate=nstate,
            io_dtype=_lib.dtype_enum(io), bc_dtype=_lib.dtype_enum(bc),
            b_kind=bkind, c_kind=ckind, b_groups=bgroups, c_groups=cgroups,
            delta_softplus=int(bool(softplus)), reserved=int(tune_items))

    def run(self):
        if self.f64 is not None:
            from . import _f64
            return _f64.scan_forward(*self.f64)
        _lib.call("ssm_scan_fwd", self.args, self.device)
        return self.out, self.last


# Argument structs of calls that were validated before, by everything the validation looks at: a repeated call of
# the same form (a block calls with one form for its whole life) fills in its pointers and goes.
_SCAN_FORMS = {}
_F32 = torch.float32


def _scan_forward_again(u, delta, A, B, C, D, z, dt_bias, softplus, want_state):
    """The call through a struct remembered from an earlier call of the same form, or ``None`` if this form is new
    or any tensor needs a cast or a copy first (those go the long way, which also produces the error messages)."""
    dt = u.dtype
    if not (K.on_gpu(u) and delta.dtype == dt and A.dtype == _F32 and B.dtype == C.dtype and u.is_contiguous()
            and delta.is_contiguous() and A.is_contiguous() and B.is_contiguous() and C.is_contiguous()):
        return None
    for t, want in ((D, _F32), (z, dt), (dt_bias, _F32)):
        if t is not None and not (t.dtype == want and t.is_contiguous()):
            return None
    if (u.data_ptr() | delta.data_ptr() | B.data_ptr() | C.data_ptr() | (0 if z is None else z.data_ptr())) & 15:
        return None                      # a view off the 16-byte grid: the long way copies it
    dev = u.device
    key = (u.shape, dt, delta.shape, A.shape, B.shape, B.dtype, C.shape, None if D is None else D.shape,
           None if z is None else z.shape, None if dt_bias is None else dt_bias.shape, bool(softplus),
           bool(want_state), dev.index)
    form = _SCAN_FORMS.get(key)
    if form is None:
        return None
    for t in (delta, A, B, C, D, z, dt_bias):
        if t is not None and t.device != dev:
            return None
    args = _lib.ScanFwdArgs.from_buffer_copy(form)
    out = torch.empty_like(u)
    last = torch.empty((u.shape[0], u.shape[1], A.shape[1]), dtype=dt, device=dev) if want_state else None
    args.u, args.delta, args.A, args.Bproj, args.Cproj, args.out = (u.data_ptr(), delta.data_ptr(), A.data_ptr(),
                                                                    B.data_ptr(), C.data_ptr(), out.data_ptr())
    args.Dskip = None if D is None else D.data_ptr()
    args.z = None if z is None else z.data_ptr()
    args.dt_bias = None if dt_bias is None else dt_bias.data_ptr()
    args.last_state = None if last is None else last.data_ptr()
    _lib.call("ssm_scan_fwd", args, dev)
    return out, last, key


def _scan_forward(u, delta, A, B, C, D, z, dt_bias, softplus, want_state, tune_items=0):
    """Validate, normalise dtypes/layout, and run ``ssm_scan_fwd``."""
    if not tune_items:
        again = _scan_forward_again(u, delta, A, B, C, D, z, dt_bias, softplus, want_state)
        if again is not None:
            return again[0], again[1]
    plan = ScanPlan(u, delta, A, B, C, D, z, dt_bias, softplus, want_state, tune_items)
    out, last = plan.run()
    if plan.f64 is not None:
        return out, last
    if not tune_items and plan.chunk_states is None and len(_SCAN_FORMS) < 256:
        # remembered under the key that _scan_forward_again forms from the caller's tensors: only a call whose
        # tensors went in as they were (no cast, no copy) can be repeated through it
        k = plan.keep
        same = all(a is None or b is None or a.data_ptr() == b.data_ptr()
                   for a, b in ((u, k["u"]), (delta, k["delta"]), (z, k["z"]), (B, k["B"]), (C, k["C"]), (A, k["A"]),
                                (D, k["D"]), (dt_bias, k["bias"])))
        if same and K.on_gpu(u):
            key = (u.shape, u.dtype, delta.shape, A.shape, B.shape, B.dtype, C.shape, None if D is None else D.shape,
                   None if z is None else z.shape, None if dt_bias is None else dt_bias.shape, bool(softplus),
                   bool(want_state), u.device.index)
            _SCAN_FORMS[key] = bytes(plan.args)
    if out.dtype != plan.result_dtype:
        out = out.to(plan.result_dtype)
        last = last.to(plan.result_dtype) if last is not None else None
    return out, last


_BWD_MAX_STATES = 16     # states handled by one ssm_scan_bwd call


def _slice_states(p, kind, lo, hi):
    if kind == _lib.PROJ_DN:
        return p[:, lo:hi]
    if kind == _lib.PROJ_BDN:
        return p[:, :, lo:hi]
    return p[:, :, lo:hi, :]


def _scan_backward(grad_out, grad_last, u, delta, A, B, C, D, z, dt_bias, softplus, chunk_states=None,
                   tune_items=0, grads_in_input_dtype=False):
    """Run ``ssm_scan_bwd``; returns fp32/io-dtype gradients in input order
    ``(du, ddelta, dA, dB, dC, dD, dz, ddt_bias)``.  State sizes above 16 are
    processed in blocks of 16 states (the recurrence is independent per state and
    every gradient is additive over states).  With ``grads_in_input_dtype``, ``dB`` and ``dC`` of projections that
    every channel has for itself, ``(B, D, N, L)``, come back in the projections' own type where the kernel for
    that form writes them (no float32 tensors of that size, and no cast of them afterwards)."""
    if K.f64_compute(u, A):
        from . import _f64
        return _f64.scan_backward(grad_out, grad_last, u, delta, A, B, C, D, z, dt_bias, softplus)
    u, delta, A, B, C, D, z, dt_bias = K.narrow(u, delta, A, B, C, D, z, dt_bias)
    batch, dim, length, nstate, (bkind, bgroups), (ckind, cgroups) = \
        K.check_selective_scan(u, delta, A, B, C, D, z, dt_bias)
    dev = K.require_gpu(u, delta, A, B, C, D, z, dt_bias, grad_out)
    io = K.common_io_dtype([u, delta, z])
    bc = K.common_io_dtype([B, C])
    u_c, dl_c, z_c = K.cast_c(u, io), K.cast_c(delta, io), K.cast_c(z, io)
    go_c = K.cast_c(grad_out, io)
    A_f, D_f, bias_f = K.as_f32_vec(A), K.as_f32_vec(D), K.as_f32_vec(dt_bias)
    B_c, C_c = K.cast_c(B, bc), K.cast_c(C, bc)
    glast = K.as_f32_vec(grad_last) if grad_last is not None else None
    lib = _lib.load()

    dA = torch.empty(dim, nstate, dtype=torch.float32, device=dev)
    dB = dC = None                    # allocated once the element type is known (first block of states)
    dD = torch.empty(dim, dtype=torch.float32, device=dev) if D is not None else None
    dbias = torch.empty(dim, dtype=torch.float32, device=dev) if dt_bias is not None else None
    blocks = [(lo, min(nstate, lo + _BWD_MAX_STATES)) for lo in range(0, nstate, _BWD_MAX_STATES)]
    single = len(blocks) == 1
    du = ddl = dz = None
    for bi, (lo, hi) in enumerate(blocks):
        n_blk = hi - lo
        if single:
            A_b, B_b, C_b, gl_b = A_f, B_c, C_c, glast
            cs = chunk_states
        else:
            A_b = A_f[:, lo:hi].contiguous()
            B_b = _slice_states(B_c, bkind, lo, hi).contiguous()
            C_b = _slice_states(C_c, ckind, lo, hi).contiguous()
            gl_b = glast[:, :, lo:hi].contiguous() if glast is not None else None
            cs = None
        D_b = D_f if bi == 0 else None
        if cs is None:      # regenerate the chunk checkpoints for this block of states
            fwd = ScanPlan(u_c, dl_c, A_b, B_b, C_b, D_b, z_c, bias_f, softplus, False,
                           want_chunk_states=True)
            fwd.run()
            cs = fwd.chunk_states
        du_b, ddl_b = torch.empty_like(u_c), torch.empty_like(u_c)
        dz_b = torch.empty_like(u_c) if z_c is not None else None
        dA_b = dA if single else torch.empty(dim, n_blk, dtype=torch.float32, device=dev)
        dB_b = dC_b = None
        dD_b = dD if bi == 0 else None
        dbias_b = torch.empty(dim, dtype=torch.float32, device=dev) if dt_bias is not None else None
        args = _lib.ScanBwdArgs(
            u=_lib.ptr(u_c), delta=_lib.ptr(dl_c), z=_lib.ptr(z_c), dout=_lib.ptr(go_c), A=_lib.ptr(A_b),
            Bproj=_lib.ptr(B_b), Cproj=_lib.ptr(C_b), Dskip=_lib.ptr(D_b), dt_bias=_lib.ptr(bias_f),
            dlast_state=_lib.ptr(gl_b), chunk_states=_lib.ptr(cs), du=_lib.ptr(du_b), ddelta=_lib.ptr(ddl_b),
            dz=_lib.ptr(dz_b), dA=_lib.ptr(dA_b), dB=256, dC=256, dD=_lib.ptr(dD_b),       # (dB, dC: set below)
            ddt_bias=_lib.ptr(dbias_b), workspace=None, workspace_bytes=0,
            batch=batch, dim=dim, seqlen=length, nstate=n_blk, io_dtype=_lib.dtype_enum(io),
            bc_dtype=_lib.dtype_enum(bc), b_kind=bkind, c_kind=ckind, b_groups=bgroups, c_groups=cgroups,
            delta_softplus=int(bool(softplus)), reserved=int(tune_items))
        # projections of their own per channel: no partial sums of dB and dC, and their own type on request
        nbytes = int((_lib.load_test_hooks() if tune_items else lib).ssm_scan_bwd_per_row_workspace_bytes(args))
        g_dtype = bc if (nbytes and grads_in_input_dtype and single) else torch.float32
        dB_b, dC_b = (torch.empty(B_b.shape, dtype=g_dtype, device=dev), torch.empty(C_b.shape, dtype=g_dtype, device=dev))
        args.dB, args.dC, args.dbc_dtype = _lib.ptr(dB_b), _lib.ptr(dC_b), _lib.dtype_enum(g_dtype)
        if single:
            dB, dC = dB_b, dC_b
        elif dB is None:
            dB = torch.empty(B_c.shape, dtype=torch.float32, device=dev)
            dC = torch.empty(C_c.shape, dtype=torch.float32, device=dev)
        if not nbytes:
            nbytes = lib.ssm_scan_bwd_workspace_bytes(batch, dim, length, n_blk, bkind, ckind, bgroups, cgroups)
        ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=dev)
        args.workspace, args.workspace_bytes = (ws.data_ptr() + 255) // 256 * 256, nbytes
        _lib.call("ssm_scan_bwd", args, dev)
        if single:
            du, ddl, dz, dbias = du_b, ddl_b, dz_b, dbias_b
        else:
            dA[:, lo:hi] = dA_b
            _slice_states(dB, bkind, lo, hi).copy_(dB_b)
            _slice_states(dC, ckind, lo, hi).copy_(dC_b)
            if bi == 0:
                du, ddl = du_b.float(), ddl_b.float()
                dz = dz_b.float() if dz_b is not None else None
                if dbias is not None:
                    dbias.copy_(dbias_b)
            else:
                du += du_b
                ddl += ddl_b
                if dz is not None:
                    dz += dz_b
                if dbias is not None:
                    dbias += dbias_b
    return du, ddl, dA, dB, dC, dD, dz, dbias


def selective_scan(u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False,
                   return_last_state=False):
    """Selective scan (Mamba-1) on the GPU.

    ``h_t = exp(delta_t A) h_{t-1} + delta_t u_t B_t``, ``y_t = <h_t, C_t> + D u_t``,
    optionally gated by ``silu(z_t)``; the state starts at zero and accumulates
    in float32.

    Args:
        u: Input drive ``(B, D, L)``; float32, bfloat16 or float16.
        delta: Step sizes ``(B, D, L)``.
        A: State matrix ``(D, N)``.
        B: Input projection ``(D, N)``, ``(B, D, N)`` or grouped/time-varying
            ``(B, G, N, L)`` with ``G`` dividing ``D``.
        C: Output projection, same accepted shapes as ``B``.
        D: Optional skip ``(D,)``.
        z: Optional gate ``(B, D, L)``; ``silu`` is applied.
        dt_bias: Optional bias ``(D,)`` added to ``delta`` before ``softplus``.
        softplus: Apply ``softplus`` to the (biased) ``delta``.
        return_last_state: Also return the final state ``(B, D, N)`` in ``u.dtype``.

    Returns:
        ``(B, D, L)`` tensor in ``u.dtype``, or ``(output, last_state)``.
    """
    tensors = (u, delta, A, B, C, D, z, dt_bias)
    if any(t is not None and t.requires_grad for t in tensors) and torch.is_grad_enabled():
        from ._autograd import SelectiveScanFn
        out, last = SelectiveScanFn.apply(u, delta, A, B, C, D, z, dt_bias, bool(softplus),
                                          bool(return_last_state))
    else:
        out, last = _scan_forward(u, delta, A, B, C, D, z, dt_bias, softplus, return_last_state)
    if return_last_state:
        return out, last
    return out


# ---------------------------------------------------------------------------
# selective state step (decode)
# ---------------------------------------------------------------------------

class StepPlan:
    """A prepared ``ssm_state_step`` call that updates ``state`` in place."""

    def __init__(self, state, x, dt, A, B, C, D, z, dt_bias, softplus, out=None):
        batch, dim, nstate, (bkind, bgroups), (ckind, cgroups) = \
            K.check_state_step(state, x, dt, A, B, C, D, z, dt_bias)
        self.device = K.require_gpu(state, x, dt, A, B, C, D, z, dt_bias)
        self.result_dtype = x.dtype
        self.f64 = None
        if K.f64_compute(state, A):       # computed in double precision by kernels of their own
            self.f64 = (state, x, dt, A, B, C, D, z, dt_bias, softplus)
            return
        x, dt, A, B, C, D, z, dt_bias = K.narrow(x, dt, A, B, C, D, z, dt_bias)
        if not state.is_contiguous():
            raise ValueError("state must be contiguous to be updated in place")
        io = K.common_io_dtype([x, dt, z])
        bc = K.common_io_dtype([B, C])
        self.result_dtype = x.dtype
        # z and grouped B / C may be slices of wider rows (a block's projected row): taken as they are, with the
        # distance between batch rows, instead of being copied
        zk, z_bs = _rows_as_given(z, io)
        Bk, b_bs = _rows_as_given(B, bc) if bkind == _lib.PROJ_BGNL else (K.cast_c(B, bc), 0)
        Ck, c_bs = _rows_as_given(C, bc) if ckind == _lib.PROJ_BGNL else (K.cast_c(C, bc), 0)
        self.keep = dict(x=K.cast_c(x, io), dt=K.cast_c(dt, io), z=zk, B=Bk, C=Ck, A=K.as_f32_vec(A),
                         D=K.as_f32_vec(D), bias=K.as_f32_vec(dt_bias))
        k = self.keep
        self.state = state.detach()
        self.out = out if out is not None else torch.empty(batch, dim, dtype=io, device=self.device)
        self.args = _lib.StateStepArgs(
            state=_lib.ptr(self.state), x=_lib.ptr(k["x"]), dt=_lib.ptr(k["dt"]), z=_lib.ptr(k["z"]),
            A=_lib.ptr(k["A"]), Bproj=_lib.ptr(k["B"]), Cproj=_lib.ptr(k["C"]), Dskip=_lib.ptr(k["D"]),
            dt_bias=_lib.ptr(k["bias"]), out=_lib.ptr(self.out),
            batch=batch, dim=dim, nstate=nstate,
            state_dtype=_lib.dtype_enum(state.dtype), io_dtype=_lib.dtype_enum(io),
            bc_dtype=_lib.dtype_enum(bc), b_kind=bkind, c_kind=ckind, b_groups=bgroups, c_groups=cgroups,
            dt_softplus=int(bool(softplus)), z_batch_stride=z_bs, b_batch_stride=b_bs, c_batch_stride=c_bs)

    def run(self):
        if self.f64 is not None:
            from . import _f64
            return _f64.state_step(*self.f64)
        _lib.call("ssm_state_step", self.args, self.device)
        return self.out


def _rows_as_given(t, dtype):
    """``(tensor, batch stride)`` for ``ssm_state_step``: a tensor of the right dtype whose batch rows are
    contiguous but apart from each other (a slice of wider rows) is passed as it is with its batch stride;
    anything else as a dense copy with stride 0 (= dense)."""
    if t is None:
        return None, 0
    if t.dtype == dtype and t.ndim >= 2 and t.shape[0] > 1 and not t.is_contiguous():
        row = t[0]
        if row.is_contiguous() and t.stride(0) >= row.numel() and (t.stride(0) * t.element_size()) % 8 == 0 \
                and t.data_ptr() % 8 == 0:
            return t, int(t.stride(0))
    return K.cast_c(t, dtype), 0


def _state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D, z, dt_bias, softplus):
    """Run ``ssm_state_step_bwd``: the nine gradients of one state update, in the order
    ``(state, x, dt, A, B, C, D, z, dt_bias)``.  ``state`` is the state before the step;
    ``grad_out`` / ``grad_state`` (gradient of the updated state) may be ``None``.
    Parameter gradients come back in float32, the others in the dtype of their tensor."""
    if K.f64_compute(state, A):
        from . import _f64
        return _f64.state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D, z, dt_bias, softplus)
    x, dt, A, B, C, D, z, dt_bias = K.narrow(x, dt, A, B, C, D, z, dt_bias)
    batch, dim, nstate, (bkind, bgroups), (ckind, cgroups) = \
        K.check_state_step(state, x, dt, A, B, C, D, z, dt_bias)
    dev = K.require_gpu(state, x, dt, A, B, C, D, z, dt_bias, grad_out, grad_state)
    io = K.common_io_dtype([x, dt, z])
    bc = K.common_io_dtype([B, C])
    sc = K.cast_c(state, state.dtype)
    xc, dtc, zc = K.cast_c(x, io), K.cast_c(dt, io), K.cast_c(z, io)
    Bc, Cc = K.cast_c(B, bc), K.cast_c(C, bc)
    Af, Df, bf = K.as_f32_vec(A), K.as_f32_vec(D), K.as_f32_vec(dt_bias)
    go = K.cast_c(grad_out, io) if grad_out is not None else None
    gs = K.cast_c(grad_state, state.dtype) if grad_state is not None else None
    dstate = torch.empty_like(sc)
    dx, ddt = torch.empty_like(xc), torch.empty_like(dtc)
    dz = torch.empty_like(zc) if zc is not None else None
    dA = torch.empty(dim, nstate, dtype=torch.float32, device=dev)
    dB = torch.empty(Bc.shape, dtype=torch.float32, device=dev)
    dC = torch.empty(Cc.shape, dtype=torch.float32, device=dev)
    dD = torch.empty(dim, dtype=torch.float32, device=dev) if D is not None else None
    dbias = torch.empty(dim, dtype=torch.float32, device=dev) if dt_bias is not None else None
    nbytes = int(_lib.load().ssm_state_step_bwd_workspace_bytes(batch, dim, nstate))
    work = torch.empty(nbytes // 4, dtype=torch.float32, device=dev)
    args = _lib.StateStepBwdArgs(
        grad_out=_lib.ptr(go), grad_state=_lib.ptr(gs), state=_lib.ptr(sc), x=_lib.ptr(xc), dt=_lib.ptr(dtc),
        z=_lib.ptr(zc), A=_lib.ptr(Af), Bproj=_lib.ptr(Bc), Cproj=_lib.ptr(Cc), Dskip=_lib.ptr(Df),
        dt_bias=_lib.ptr(bf), dstate=_lib.ptr(dstate), dx=_lib.ptr(dx), ddt=_lib.ptr(ddt), dz=_lib.ptr(dz),
        dA=_lib.ptr(dA), dB=_lib.ptr(dB), dC=_lib.ptr(dC), dD=_lib.ptr(dD), ddt_bias=_lib.ptr(dbias),
        workspace=_lib.ptr(work), workspace_bytes=nbytes, batch=batch, dim=dim, nstate=nstate,
        state_dtype=_lib.dtype_enum(sc.dtype), io_dtype=_lib.dtype_enum(io), bc_dtype=_lib.dtype_enum(bc),
        b_kind=bkind, c_kind=ckind, b_groups=bgroups, c_groups=cgroups, dt_softplus=int(bool(softplus)))
    _lib.call("ssm_state_step_bwd", args, dev)
    return dstate, dx, ddt, dA, dB, dC, dD, dz, dbias


# Argument structs of state steps that were validated before, keyed by everything the validation looks at (as
# _SCAN_FORMS for the scan): a decoding loop calls with one form for its whole life, a new token's tensors each time.
_STEP_FORMS = {}


def _state_step_again(state, x, dt, A, B, C, D, z, dt_bias, softplus):
    """The step through a struct remembered from an earlier call of the same form, or ``None`` if the form is new or
    a tensor would need a cast, a copy or a batch stride first (those go the long way)."""
    io = x.dtype
    if not (K.on_gpu(state) and dt.dtype == io and A.dtype == _F32 and B.dtype == C.dtype and state.is_contiguous()
            and x.is_contiguous() and dt.is_contiguous() and A.is_contiguous() and B.is_contiguous() and C.is_contiguous()):
        return None
    for t, want in ((D, _F32), (z, io), (dt_bias, _F32)):
        if t is not None and not (t.dtype == want and t.is_contiguous()):
            return None
    if (state.data_ptr() | x.data_ptr() | dt.data_ptr() | A.data_ptr() | B.data_ptr() | C.data_ptr()
            | (0 if z is None else z.data_ptr()) | (0 if D is None else D.data_ptr())
            | (0 if dt_bias is None else dt_bias.data_ptr())) & 15:
        return None
    dev = state.device
    key = (state.shape, state.dtype, x.shape, io, A.shape, B.shape, B.dtype, C.shape, D is None or D.shape,
           z is None or z.shape, dt_bias is None or dt_bias.shape, bool(softplus), dev.index)
    form = _STEP_FORMS.get(key)
    if form is None:
        return None
    for t in (x, dt, A, B, C, D, z, dt_bias):
        if t is not None and t.device != dev:
            return None
    args = _lib.StateStepArgs.from_buffer_copy(form)
    out = torch.empty_like(x)
    args.state, args.x, args.dt, args.A, args.Bproj, args.Cproj, args.out = (
        state.data_ptr(), x.data_ptr(), dt.data_ptr(), A.data_ptr(), B.data_ptr(), C.data_ptr(), out.data_ptr())
    args.z = None if z is None else z.data_ptr()
    args.Dskip = None if D is None else D.data_ptr()
    args.dt_bias = None if dt_bias is None else dt_bias.data_ptr()
    _lib.call("ssm_state_step", args, dev)
    return out


def selective_state_step(state, x, dt, A, B, C, D=None, z=None, dt_bias=None, softplus=True):
    """Advance the selective state by one token on the GPU; ``state`` is updated in place.

    Args:
        state: Recurrent state ``(B, D, N)`` (float32, bfloat16 or float16), overwritten.
        x: Input drive ``(B, D)``.
        dt: Time-step ``(B, D)``.
        A: State matrix ``(D, N)``.
        B: Input projection ``(D, N)``, ``(B, D, N)`` or grouped ``(B, G, N)`` with ``G | D``.
        C: Output projection, same accepted shapes as ``B``.
        D: Optional skip ``(D,)``.
        z: Optional gate ``(B, D)``; ``silu`` is applied.
        dt_bias: Optional bias ``(D,)`` added before ``softplus``.
        softplus: Apply ``softplus`` to the biased ``dt`` (default ``True``).

    Returns:
        Output ``(B, D)`` in ``x.dtype``.
    """
    tensors = (state, x, dt, A, B, C, D, z, dt_bias)
    if any(t is not None and t.requires_grad for t in tensors) and torch.is_grad_enabled():
        from ._autograd import state_step_with_grad
        return state_step_with_grad(state, x, dt, A, B, C, D, z, dt_bias, bool(softplus))
    again = _state_step_again(state, x, dt, A, B, C, D, z, dt_bias, softplus)
    if again is not None:
        return again
    if state.is_contiguous():
        plan = StepPlan(state, x, dt, A, B, C, D, z, dt_bias, softplus)
        out = plan.run()
        if plan.f64 is None and len(_STEP_FORMS) < 256 and out.dtype == x.dtype:
            # remembered only when every tensor went in as it was (no cast, no copy, no batch stride): that is what
            # _state_step_again can repeat
            k, a = plan.keep, plan.args
            same = all(p is None or q is None or p.data_ptr() == q.data_ptr()
                       for p, q in ((x, k["x"]), (dt, k["dt"]), (z, k["z"]), (B, k["B"]), (C, k["C"]), (A, k["A"]),
                                    (D, k["D"]), (dt_bias, k["bias"])))
            if same and not (a.z_batch_stride or a.b_batch_stride or a.c_batch_stride) and K.on_gpu(state):
                key = (state.shape, state.dtype, x.shape, x.dtype, A.shape, B.shape, B.dtype, C.shape,
                       D is None or D.shape, z is None or z.shape, dt_bias is None or dt_bias.shape, bool(softplus),
                       state.device.index)
                _STEP_FORMS[key] = bytes(a)
    else:
        work = state.contiguous()
        plan = StepPlan(work, x, dt, A, B, C, D, z, dt_bias, softplus)
        out = plan.run()
        state.copy_(work)
    return out if out.dtype == x.dtype else out.to(x.dtype)


class DecodePlan:
    """A prepared fused decode step (``ssm_decode_step``): rolls ``conv_state`` and
    updates ``ssm_state`` in place on every :meth:`run`."""

    def __init__(self, conv_state, ssm_state, x, dt, A, B, C, conv_weight, conv_bias=None, D=None, z=None,
                 dt_bias=None, softplus=True, activation="silu", want_conv_out=False):
        step = StepPlan(ssm_state, x, dt, A, B, C, D, z, dt_bias, softplus)
        batch, dim = int(x.shape[0]), int(x.shape[1])
        if conv_state.ndim != 3 or tuple(conv_state.shape[:2]) != (batch, dim):
            raise ValueError("conv_state must have shape (B, D, K).")
        width = int(conv_state.shape[2])
        w = conv_weight[:, 0, :] if conv_weight.ndim == 3 else conv_weight
        if tuple(w.shape) != (dim, width):
            raise ValueError("conv_weight must have shape (D, K) matching conv_state.")
        if conv_bias is not None and tuple(conv_bias.shape) != (dim,):
            raise ValueError("conv_bias must have shape (D,).")
        act = str(activation).lower()
        if act not in ("silu", "swish", "identity", "none"):
            raise ValueError(f"Unsupported activation '{activation}'.")
        K.require_gpu(conv_state, conv_weight, conv_bias, x)
        io = step.keep["x"].dtype
        if conv_state.dtype != io or not conv_state.is_contiguous():
            raise ValueError("conv_state must be contiguous and share the dtype of x, dt and z")
        self.step = step
        self.device = step.device
        self.out = step.out
        self.keep = dict(w=K.as_f32_vec(w), b=K.as_f32_vec(conv_bias), conv_state=conv_state.detach())
        self.conv_out = torch.empty(batch, dim, dtype=io, device=self.device) if want_conv_out else None
        self.args = _lib.DecodeStepArgs(
            step=step.args, conv_state=_lib.ptr(self.keep["conv_state"]), conv_weight=_lib.ptr(self.keep["w"]),
            conv_bias=_lib.ptr(self.keep["b"]), conv_out=_lib.ptr(self.conv_out), conv_width=width,
            conv_activation=_lib.ACT_SILU if act in ("silu", "swish") else _lib.ACT_IDENTITY)

    def run(self):
        _lib.call("ssm_decode_step", self.args, self.device)
        return self.out


def decode_step(conv_state, ssm_state, x, dt, A, B, C, conv_weight, conv_bias=None, D=None, z=None,
                dt_bias=None, softplus=True, activation="silu", return_conv_out=False):
    """One fused decode step: causal-conv window update + activation + selective state update.

    Equivalent to rolling ``conv_state`` left by one, writing ``x`` into its last slot,
    ``xc = act(bias + sum_k conv_state[..., k] * conv_weight[:, k])`` (rounded to the dtype of
    ``x``) and ``selective_state_step(ssm_state, xc, dt, A, B, C, D, z, dt_bias, softplus)``;
    both states are updated in place.

    Args:
        conv_state: ``(B, D, K)`` window of the last ``K`` inputs, same dtype as ``x``.
        ssm_state: ``(B, D, N)`` recurrent state.
        x: New (pre-convolution) input ``(B, D)``.
        dt, A, B, C, D, z, dt_bias, softplus: as in :func:`selective_state_step`.
        conv_weight: ``(D, K)`` or ``(D, 1, K)``.
        conv_bias: Optional ``(D,)``.
        activation: ``"silu"``/``"swish"`` or ``"identity"``/``"none"``.
        return_conv_out: Also return the activated convolution output ``(B, D)``.

    Returns:
        ``y (B, D)`` in ``x.dtype``, or ``(y, conv_out)``.
    """
    plan = DecodePlan(conv_state, ssm_state, x, dt, A, B, C, conv_weight, conv_bias, D, z, dt_bias, softplus,
                      activation, want_conv_out=return_conv_out)
    y = plan.run()
    if return_conv_out:
        return y, plan.conv_out
    return y


def mamba2_decode_step(zxbcdt, conv_state, ssm_state, conv_weight, conv_bias, A, D=None, dt_bias=None,
                       ngroups=1, softplus=True, gate=True, return_conv_out=False):
    """One decoding step of a Mamba-2 (SSD) block on cached states, consuming the row of the input
    projection as it is (two launches: convolution on the cached windows, state update per head).

    Args:
        zxbcdt: ``(B, 2*d_inner + 2*G*N + H)`` row of the input projection, ``z | x B C | dt``.
        conv_state: ``(B, d_inner + 2*G*N, K)`` last ``K`` inputs of every convolution channel (oldest
            first), dtype of ``zxbcdt``; rolled in place.
        ssm_state: ``(B, H, P, N)`` float32, updated in place.
        conv_weight: ``(d_inner + 2*G*N, K)``; conv_bias: ``(d_inner + 2*G*N,)`` or ``None``.
        A: ``(H,)``; D: ``(H,)`` or ``(H, P)`` or ``None``; dt_bias: ``(H,)`` or ``None``.
        ngroups: ``G``, the number of B/C groups.
        softplus: Apply softplus to ``dt + dt_bias``.
        gate: Multiply ``y`` by ``silu(z)``.
        return_conv_out: Also return the activated convolution output ``(B, d_inner + 2*G*N)`` (float32).

    Returns:
        ``y (B, d_inner)`` in ``zxbcdt.dtype``, or ``(y, conv_out)``.
    """
    if ssm_state.ndim != 4 or zxbcdt.ndim != 2 or conv_state.ndim != 3:
        raise ValueError("zxbcdt must be (B, proj), conv_state (B, C, K) and ssm_state (B, H, P, N).")
    batch, heads, hdim, nstate = (int(v) for v in ssm_state.shape)
    G = int(ngroups)
    di, conv_dim = heads * hdim, heads * hdim + 2 * G * nstate
    K_ = int(conv_state.shape[2])
    if tuple(zxbcdt.shape) != (batch, 2 * di + 2 * G * nstate + heads):
        raise ValueError("zxbcdt must have 2*d_inner + 2*G*N + H columns.")
    if tuple(conv_state.shape) != (batch, conv_dim, K_) or conv_state.dtype != zxbcdt.dtype:
        raise ValueError("conv_state must be (B, d_inner + 2*G*N, K) in the dtype of zxbcdt.")
    if ssm_state.dtype != torch.float32 or not ssm_state.is_contiguous() or not conv_state.is_contiguous():
        raise ValueError("ssm_state must be contiguous float32 and conv_state contiguous (both are updated in place).")
    if tuple(A.shape) != (heads,) or (D is not None and tuple(D.shape) not in ((heads,), (heads, hdim))):
        raise ValueError("A must be (H,) and D (H,) or (H, P).")
    dev = K.require_gpu(zxbcdt, conv_state, ssm_state, conv_weight, conv_bias, A, D, dt_bias)
    K.check_float("zxbcdt", zxbcdt)
    row = K.cast_c(zxbcdt, zxbcdt.dtype)
    wf = K.as_f32_vec(conv_weight.reshape(conv_dim, K_))
    bf, Af, Df, biasf = K.as_f32_vec(conv_bias), K.as_f32_vec(A), K.as_f32_vec(D), K.as_f32_vec(dt_bias)
    xbc = torch.empty(batch, conv_dim, dtype=torch.float32, device=dev)
    y = torch.empty(batch, di, dtype=zxbcdt.dtype, device=dev)
    args = _lib.Mamba2DecodeArgs(
        zxbcdt=_lib.ptr(row), conv_state=_lib.ptr(conv_state), conv_weight=_lib.ptr(wf), conv_bias=_lib.ptr(bf),
        xbc=_lib.ptr(xbc), ssm_state=_lib.ptr(ssm_state), A=_lib.ptr(Af), Dskip=_lib.ptr(Df), dt_bias=_lib.ptr(biasf),
        y=_lib.ptr(y), batch=batch, heads=heads, headdim=hdim, groups=G, nstate=nstate, conv_width=K_,
        io_dtype=_lib.dtype_enum(row.dtype), d_per_p=int(D is not None and D.ndim == 2),
        dt_softplus=int(bool(softplus)), gate=int(bool(gate)))
    _lib.call("ssm_mamba2_decode_step", args, dev)
    return (y, xbc) if return_conv_out else y


def conv_window_step(conv_state, x, weight, bias=None, activation="silu"):
    """The depthwise causal convolution for one new token on a cached window.

    ``conv_state`` moves on by one (its oldest column drops out, ``x`` becomes the newest) and the
    result is ``act(bias + sum_k weight[:, k] * conv_state[:, :, k])``: what ``dw_causal_conv`` returns
    at the last position of the sequence the window ends.

    Args:
        conv_state: ``(B, C, K)`` last ``K`` inputs of every channel, oldest first; updated in place.
        x: ``(B, C)`` new input in the dtype of ``conv_state``; a column slice of a wider matrix is read
            in place (unit stride along ``C``).
        weight: ``(C, K)`` or ``(C, 1, K)``; bias: ``(C,)`` or ``None``.
        activation: ``"silu"``/``"swish"`` or ``"identity"``/``"none"``.

    Returns:
        ``(B, C)`` tensor in ``x.dtype``.
    """
    if conv_state.ndim != 3 or x.ndim != 2 or tuple(conv_state.shape[:2]) != tuple(x.shape):
        raise ValueError("conv_state must have shape (B, C, K) and x (B, C).")
    batch, chans, width = (int(v) for v in conv_state.shape)
    w = weight[:, 0, :] if weight.ndim == 3 else weight
    if tuple(w.shape) != (chans, width):
        raise ValueError("weight must have shape (C, K) matching conv_state.")
    if bias is not None and tuple(bias.shape) != (chans,):
        raise ValueError("bias must have shape (C,).")
    act = str(activation).lower()
    if act not in ("silu", "swish", "identity", "none"):
        raise ValueError(f"Unsupported activation '{activation}'.")
    dev = K.require_gpu(conv_state, x, weight, bias)
    K.check_float("x", x)
    if conv_state.dtype != x.dtype or not conv_state.is_contiguous():
        raise ValueError("conv_state must be contiguous and share the dtype of x (it is updated in place).")
    xs = x.detach()
    if xs.stride(1) != 1 or xs.stride(0) < chans:
        xs = xs.contiguous()
    wf, bf = K.as_f32_vec(w), K.as_f32_vec(bias)
    out = torch.empty(batch, chans, dtype=x.dtype, device=dev)
    args = _lib.Conv1dUpdateArgs(
        x=_lib.ptr(xs), conv_state=_lib.ptr(conv_state), weight=_lib.ptr(wf), bias=_lib.ptr(bf), out=_lib.ptr(out),
        x_row_stride=int(xs.stride(0)), batch=batch, channels=chans, width=width,
        io_dtype=_lib.dtype_enum(x.dtype), activation=_lib.ACT_SILU if act in ("silu", "swish") else _lib.ACT_IDENTITY)
    _lib.call("ssm_conv1d_update", args, dev)
    return out


# ---------------------------------------------------------------------------
# diagonal chunk scan (the reference's ``ssd_chunk_scan``)
# ---------------------------------------------------------------------------

def _dscan_forward(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states, want_round_states=False):
    """Validate, normalise dtypes/layout, and run ``ssm_dscan_fwd``; ``lengths`` is the
    int32 device tensor of valid steps per batch row (or ``None``).  With ``want_round_states``
    returns ``(Y, round_states)``: the state entering every 64 steps, ``(B, ceil(L/64), H*P)`` float32, which
    :func:`_dscan_backward` takes instead of sweeping forward itself -- or ``None`` when the call does not run the
    kernel that can write it."""
    if K.f64_compute(X, A):
        from . import _f64
        Y = _f64.dscan_forward(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)
        return (Y, None) if want_round_states else Y
    dt, A, B, C, D, z, initial_states = K.narrow(dt, A, B, C, D, z, initial_states)
    batch, seqlen, heads, proj, a_per_p, bk, ck, d_per_p, z_per_p = \
        K.check_chunk_scan(X, dt, A, B, C, chunk_size, D, z, initial_states)
    dev = K.require_gpu(X, dt, A, B, C, D, z, initial_states)
    bc = K.common_io_dtype([B, C])
    Xc, dtc = K.cast_c(X, X.dtype), K.cast_c(dt, dt.dtype)
    Bc, Cc = K.cast_c(B, bc), K.cast_c(C, bc)
    zc = K.cast_c(z, z.dtype) if z is not None else None
    ic = K.cast_c(initial_states, initial_states.dtype) if initial_states is not None else None
    Af, Df = K.as_f32_vec(A), K.as_f32_vec(D)
    Y = torch.empty_like(Xc)
    nbytes = _lib.load().ssm_dscan_fwd_workspace_bytes(batch, seqlen, heads, proj)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device=dev)
    args = _lib.DscanFwdArgs(
        X=_lib.ptr(Xc), dt=_lib.ptr(dtc), A=_lib.ptr(Af), Bproj=_lib.ptr(Bc), Cproj=_lib.ptr(Cc),
        Dskip=_lib.ptr(Df), z=_lib.ptr(zc), initial_states=_lib.ptr(ic), seq_lens=_lib.ptr(lengths),
        Y=_lib.ptr(Y), workspace=_lib.ptr(ws), workspace_bytes=nbytes,
        batch=batch, seqlen=seqlen, heads=heads, proj=proj,
        x_dtype=_lib.dtype_enum(Xc.dtype), dt_dtype=_lib.dtype_enum(dtc.dtype), bc_dtype=_lib.dtype_enum(bc),
        z_dtype=_lib.dtype_enum(zc.dtype) if zc is not None else 0,
        init_dtype=_lib.dtype_enum(ic.dtype) if ic is not None else 0,
        b_kind=bk, c_kind=ck, a_per_p=int(a_per_p), d_per_p=int(d_per_p), z_per_p=int(z_per_p))
    table = None
    if want_round_states and _lib.load().ssm_dscan_fwd_one_pass(args):
        table = torch.empty(batch, (seqlen + 63) // 64, heads * proj, dtype=torch.float32, device=dev)
        args.round_states = _lib.ptr(table)
    _lib.call("ssm_dscan_fwd", args, dev)
    return (Y, table) if want_round_states else Y


def _dscan_backward(grad_y, X, dt, A, B, C, chunk_size, D, z, lengths, initial_states, grads_in_input_dtype=False,
                    two_kernels=False, round_states=None):
    """Run ``ssm_dscan_bwd``: gradients ``(dX, ddt, dA, dB, dC, dD, dz, dinitial_states)``.
    ``dX`` comes back in ``X.dtype``, the rest in float32 with the shape of its tensor; with
    ``grads_in_input_dtype`` the kernel writes a per-token ``dB`` / ``dC`` and a per-channel ``dz`` in their
    tensors' own types (no float32 copy of a tensor of ``X``'s size is made and converted afterwards).
    ``two_kernels`` keeps the general path for a call the one-pass kernels cover; ``round_states`` is what
    :func:`_dscan_forward` returned for the same inputs (or ``None``)."""
    if K.f64_compute(X, A):
        from . import _f64
        return _f64.dscan_backward(grad_y, X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)
    dt, A, B, C, D, z, initial_states = K.narrow(dt, A, B, C, D, z, initial_states)
    batch, seqlen, heads, proj, a_per_p, bk, ck, d_per_p, z_per_p = \
        K.check_chunk_scan(X, dt, A, B, C, chunk_size, D, z, initial_states)
    dev = K.require_gpu(X, dt, A, B, C, D, z, initial_states, grad_y)
    bc = K.common_io_dtype([B, C])
    Xc, dtc = K.cast_c(X, X.dtype), K.cast_c(dt, dt.dtype)
    gy = K.cast_c(grad_y, X.dtype)
    Bc, Cc = K.cast_c(B, bc), K.cast_c(C, bc)
    zc = K.cast_c(z, z.dtype) if z is not None else None
    ic = K.cast_c(initial_states, initial_states.dtype) if initial_states is not None else None
    Af, Df = K.as_f32_vec(A), K.as_f32_vec(D)
    f32 = dict(dtype=torch.float32, device=dev)
    dX = torch.empty_like(Xc)
    ddt = torch.empty(batch, seqlen, heads, **f32)
    dA = torch.empty(A.shape, **f32)
    io = bool(grads_in_input_dtype)
    dB = torch.empty(Bc.shape, dtype=bc if (io and bk == _lib.CHUNK_BLHP) else torch.float32, device=dev)
    dC = torch.empty(Cc.shape, dtype=bc if (io and ck == _lib.CHUNK_BLHP) else torch.float32, device=dev)
    dD = torch.empty(D.shape, **f32) if D is not None else None
    dz = None
    if zc is not None:
        dz = torch.empty(zc.shape, dtype=zc.dtype if (io and z_per_p) else torch.float32, device=dev)
    dinit = torch.empty(batch, heads, proj, **f32) if ic is not None else None
    nbytes = int(_lib.load().ssm_dscan_bwd_workspace_bytes(batch, seqlen, heads, proj))
    ws = torch.empty(nbytes // 4, **f32)
    args = _lib.DscanBwdArgs(
        grad_y=_lib.ptr(gy), X=_lib.ptr(Xc), dt=_lib.ptr(dtc), A=_lib.ptr(Af), Bproj=_lib.ptr(Bc),
        Cproj=_lib.ptr(Cc), Dskip=_lib.ptr(Df), z=_lib.ptr(zc), initial_states=_lib.ptr(ic),
        seq_lens=_lib.ptr(lengths), dX=_lib.ptr(dX), ddt=_lib.ptr(ddt), dA=_lib.ptr(dA), dB=_lib.ptr(dB),
        dC=_lib.ptr(dC), dD=_lib.ptr(dD), dz=_lib.ptr(dz), dinitial_states=_lib.ptr(dinit),
        workspace=_lib.ptr(ws), workspace_bytes=nbytes, batch=batch, seqlen=seqlen, heads=heads, proj=proj,
        x_dtype=_lib.dtype_enum(Xc.dtype), dt_dtype=_lib.dtype_enum(dtc.dtype), bc_dtype=_lib.dtype_enum(bc),
        z_dtype=_lib.dtype_enum(zc.dtype) if zc is not None else 0,
        init_dtype=_lib.dtype_enum(ic.dtype) if ic is not None else 0,
        b_kind=bk, c_kind=ck, a_per_p=int(a_per_p), d_per_p=int(d_per_p), z_per_p=int(z_per_p),
        grads_in_io_dtype=int(io), reserved=int(bool(two_kernels)))
    if round_states is not None:
        want = (batch, (seqlen + 63) // 64, heads * proj)
        if tuple(round_states.shape) != want or round_states.dtype != torch.float32 or not round_states.is_contiguous():
            raise ValueError(f"round_states must be a contiguous float32 tensor of shape {want}.")
        args.round_states = _lib.ptr(round_states)
    _lib.call("ssm_dscan_bwd", args, dev)
    return dX, ddt, dA, dB, dC, dD, dz, dinit


def ssd_chunk_scan(X, dt, A, B, C, chunk_size, D=None, z=None, seq_meta=None, initial_states=None):
    """Chunked diagonal state-space scan on the GPU (the reference's "SSD chunk scan").

    ``s_t = exp(dt_t A) s_{t-1} + dt_t B_t X_t``, ``y_t = s_t C_t + D X_t`` per
    ``(batch, head, p)`` channel, optionally gated by ``silu(z_t)``; ``dt`` is used
    as given.  ``chunk_size`` is validated but does not affect the result.
    Differentiable in every tensor argument.

    Args:
        X: Activations ``(B, L, H, P)``.
        dt: Per-head time-steps ``(B, L, H)``.
        A: ``(H, P)`` or ``(H,)``.
        B: ``(H, P)``, ``(B, H, P)`` or time-varying ``(B, L, H, P)``.
        C: Same accepted shapes as ``B``.
        chunk_size: Positive integer.
        D: Optional skip ``(H,)`` or ``(H, P)``.
        z: Optional gate ``(B, L, H)`` or ``(B, L, H, P)``.
        seq_meta: Optional dict with ``cu_seqlens`` (length ``B + 1``) or ``seq_lens``
            (length ``B``); steps at or beyond a row's length produce zeros.
        initial_states: Optional initial state ``(B, H, P)``.

    Returns:
        Tensor ``(B, L, H, P)`` in ``X.dtype``.
    """
    tensors = (X, dt, A, B, C, D, z, initial_states)
    K.check_chunk_scan(X, dt, A, B, C, chunk_size, D, z, initial_states)
    dev = K.require_gpu(X, dt, A, B, C, D, z, initial_states)
    lengths = K.sequence_lengths(seq_meta, int(X.shape[0]), dev)
    if any(t is not None and t.requires_grad for t in tensors) and torch.is_grad_enabled():
        from ._autograd import DiagScanFn
        return DiagScanFn.apply(X, dt, A, B, C, int(chunk_size), D, z, lengths, initial_states)
    return _dscan_forward(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)


# ---------------------------------------------------------------------------
# depthwise causal convolution
# ---------------------------------------------------------------------------

def _conv_weight_f32(weight):
    w = weight.detach()
    if w.ndim == 3:
        w = w[:, 0, :]
    return w.to(torch.float32).contiguous()


def _conv_rows_view(x, channels_first, width):
    """Whether ``x (B, C, L)`` is a view whose memory runs channels innermost -- what the reference's blocks pass
    (src/ssm/modules/mamba1.py:209-215, mamba2.py:159-165: ``projected.permute(0, 2, 1)``, in the first one half of
    a wider projection) -- in a form the kernels read as it lies: -> (batch stride, row stride) in elements, or
    None (the caller then takes a dense copy).  A rule on shapes and strides only, so that the layout of the
    results can be told without the data (fake tensors)."""
    if not channels_first or x.dtype == torch.float64 or x.ndim != 3:
        return None
    batch, chans, length = x.shape
    sb, sc, sl = x.stride()
    if (x.is_contiguous() or sc != 1 or chans % 4 or width > 5 or sl < chans or sl % 4 or sb % 4
            or (batch > 1 and sb < (length - 1) * sl + chans)):
        return None
    return int(sb), int(sl)


def _conv_rows_input(x, rows):
    """``x`` as the rows-in kernels take it: detached, and starting on a boundary of 4 elements (a view that starts
    elsewhere is copied into rows of its own)."""
    x = x.detach()
    if x.data_ptr() % (4 * x.element_size()):
        x = x.permute(0, 2, 1).contiguous().permute(0, 2, 1)
        rows = (int(x.stride(0)), int(x.stride(2)))
    return x, rows


def _conv_forward(x, weight, bias, activation, channels_last=None):
    if K.f64_compute(x):
        from . import _f64
        return _f64.conv_forward(x, weight, bias, activation, channels_last)
    weight, bias = K.narrow(weight, bias)
    batch, chans, length, width, channels_first, silu = K.check_conv(x, weight, bias, activation, channels_last)
    dev = K.require_gpu(x, weight, bias)
    wf, bf = _conv_weight_f32(weight), K.as_f32_vec(bias)
    rows = _conv_rows_view(x, channels_first, width)
    if rows is not None:
        xc, rows = _conv_rows_input(x, rows)
        y = torch.empty(x.shape, dtype=x.dtype, device=dev)
        layout, strides = _lib.LAYOUT_ROWS_TO_BCL, rows
    else:
        xc = K.cast_c(x, x.dtype)
        y = torch.empty_like(xc)
        layout, strides = (_lib.LAYOUT_BCL if channels_first else _lib.LAYOUT_BLC), (0, 0)
    args = _lib.Conv1dFwdArgs(
        x=_lib.ptr(xc), weight=_lib.ptr(wf), bias=_lib.ptr(bf), y=_lib.ptr(y),
        batch=batch, channels=chans, seqlen=length, width=width, io_dtype=_lib.dtype_enum(xc.dtype),
        layout=layout, activation=_lib.ACT_SILU if silu else _lib.ACT_IDENTITY,
        x_batch_stride=strides[0], x_row_stride=strides[1])
    _lib.call("ssm_conv1d_fwd", args, dev)
    return y


def _conv_backward(grad_out, x, weight, bias, activation, channels_last=None):
    """-> (dx, dweight (C,K) fp32, dbias (C,) fp32 or None).  ``dx`` has the shape of ``x``; for an ``x`` whose
    memory runs channels innermost (see :func:`_conv_rows_view`) so does the memory of ``dx``."""
    if K.f64_compute(x):
        from . import _f64
        return _f64.conv_backward(grad_out, x, weight, bias, activation, channels_last)
    weight, bias = K.narrow(weight, bias)
    batch, chans, length, width, channels_first, silu = K.check_conv(x, weight, bias, activation, channels_last)
    dev = K.require_gpu(x, weight, bias, grad_out)
    wf, bf = _conv_weight_f32(weight), K.as_f32_vec(bias)
    gc = K.cast_c(grad_out, x.dtype)
    rows = _conv_rows_view(x, channels_first, width)
    if rows is not None:
        xc, rows = _conv_rows_input(x, rows)
        dx_rows = torch.empty(batch, length, chans, dtype=x.dtype, device=dev)
        dx, dx_mem = dx_rows.permute(0, 2, 1), dx_rows
        layout, strides = _lib.LAYOUT_ROWS_TO_BCL, rows
    else:
        xc = K.cast_c(x, x.dtype)
        dx = dx_mem = torch.empty_like(xc)
        layout, strides = (_lib.LAYOUT_BCL if channels_first else _lib.LAYOUT_BLC), (0, 0)
    dw = torch.empty(chans, width, dtype=torch.float32, device=dev)
    db = torch.empty(chans, dtype=torch.float32, device=dev) if bias is not None else None
    nbytes = _lib.load().ssm_conv1d_bwd_workspace_bytes(batch, chans, width)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    args = _lib.Conv1dBwdArgs(
        x=_lib.ptr(xc), dout=_lib.ptr(gc), weight=_lib.ptr(wf), bias=_lib.ptr(bf), dx=_lib.ptr(dx_mem),
        dweight=_lib.ptr(dw), dbias=_lib.ptr(db), workspace=_lib.ptr(ws), workspace_bytes=nbytes,
        batch=batch, channels=chans, seqlen=length, width=width, io_dtype=_lib.dtype_enum(xc.dtype),
        layout=layout, activation=_lib.ACT_SILU if silu else _lib.ACT_IDENTITY,
        x_batch_stride=strides[0], x_row_stride=strides[1])
    _lib.call("ssm_conv1d_bwd", args, dev)
    return dx, dw, db


def dw_causal_conv(x, weight, bias=None, activation="silu"):
    """Depthwise causal 1-D convolution with optional SiLU on the GPU.

    Args:
        x: Input ``(B, C, L)`` or ``(B, L, C)``; the layout is channels-first when
            ``x.shape[1] == C`` (tested first), else channels-last.
        weight: Depthwise kernel ``(C, K)`` or ``(C, 1, K)``.
        bias: Optional bias ``(C,)``.
        activation: ``"silu"``/``"swish"`` or ``"identity"``/``"none"``.

    Returns:
        Tensor with the layout and dtype of ``x``.
    """
    return _dw_causal_conv(x, weight, bias, activation, None)


def dw_causal_conv_channels_last(x, weight, bias=None, activation="silu"):
    """:func:`dw_causal_conv` on ``x (B, L, C)`` whatever ``L`` is.  Not in the reference, whose layout rule
    (src/ssm/ops/python/reference.py:483-533) reads a sequence as long as there are channels as ``(B, C, L)``."""
    return _dw_causal_conv(x, weight, bias, activation, True)


def _dw_causal_conv(x, weight, bias, activation, channels_last):
    tensors = (x, weight, bias)
    if any(t is not None and t.requires_grad for t in tensors) and torch.is_grad_enabled():
        from ._autograd import CausalConvFn
        return CausalConvFn.apply(x, weight, bias, activation, channels_last)
    return _conv_forward(x, weight, bias, activation, channels_last)


# ---------------------------------------------------------------------------
# residual-add + LayerNorm / RMSNorm
# ---------------------------------------------------------------------------

def _norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32,
                  want_residual_out=False, want_stats=False):
    if K.f64_compute(x):
        from . import _f64
        return _f64.norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, want_residual_out)
    weight, bias, residual = K.narrow(weight, bias, residual)
    rows, hidden = K.check_norm(x, weight, bias, residual)
    dev = K.require_gpu(x, weight, bias, residual)
    xc = K.cast_c(x, x.dtype)
    rc = K.cast_c(residual, residual.dtype) if residual is not None else None
    wf, bf = K.as_f32_vec(weight), K.as_f32_vec(bias)
    y = torch.empty_like(xc)
    res_out = None
    if want_residual_out:
        # what the next block should carry: fp32 when a fp32 residual stream is requested,
        # otherwise the residual's (or x's) own dtype
        if residual is not None:
            ro_dtype = torch.float32 if residual_in_fp32 else residual.dtype
        else:
            ro_dtype = torch.float32 if residual_in_fp32 else x.dtype
        res_out = torch.empty(x.shape, dtype=ro_dtype, device=dev)
    mean = torch.empty(rows, dtype=torch.float32, device=dev) if want_stats else None
    rstd = torch.empty(rows, dtype=torch.float32, device=dev) if want_stats else None
    args = _lib.NormFwdArgs(
        x=_lib.ptr(xc), residual=_lib.ptr(rc), weight=_lib.ptr(wf), bias=_lib.ptr(bf), y=_lib.ptr(y),
        residual_out=_lib.ptr(res_out), mean=_lib.ptr(mean), rstd=_lib.ptr(rstd),
        rows=rows, hidden=hidden, x_dtype=_lib.dtype_enum(xc.dtype),
        residual_dtype=_lib.dtype_enum(rc.dtype) if rc is not None else 0,
        residual_out_dtype=_lib.dtype_enum(res_out.dtype) if res_out is not None else 0,
        is_rms=int(bool(is_rms)), prenorm=int(bool(prenorm)), eps=float(eps))
    _lib.call("ssm_norm_fwd", args, dev)
    return y, res_out, mean, rstd


def _norm_backward(grad_out, x, weight, residual, mean, rstd, is_rms, prenorm, want_dbias, want_dres,
                   out=None):
    """``ssm_norm_bwd``.  With ``out = (dx, dres, dw, db)`` (preallocated, contiguous; ``None`` where a
    gradient is not wanted) the call goes to ``ssm_norm_bwd_static`` instead and allocates nothing on
    the device: inputs must then already be contiguous and ``weight`` float32."""
    if K.f64_compute(x):
        if out is not None:
            raise ValueError("the allocation-free norm backward takes float32, bfloat16 or float16 tensors")
        from . import _f64
        return _f64.norm_backward(grad_out, x, weight, residual, mean, rstd, is_rms, prenorm, want_dbias, want_dres)
    weight, residual = K.narrow(weight, residual)
    rows, hidden = K.check_norm(x, weight, None, residual)
    if out is not None:
        dev = K.require_gpu(x, weight, residual, grad_out)
        dx, dres, dw, db = out
        for t in (x, grad_out, residual, weight):
            if t is not None and not t.is_contiguous():
                raise ValueError("the allocation-free norm backward takes contiguous tensors")
        if weight.dtype != torch.float32 or grad_out.dtype != x.dtype:
            raise ValueError("the allocation-free norm backward takes a float32 weight and grad_out of x's dtype")
        args = _lib.NormBwdArgs(
            x=_lib.ptr(x), residual=_lib.ptr(residual), dy=_lib.ptr(grad_out), weight=_lib.ptr(weight),
            mean=_lib.ptr(mean), rstd=_lib.ptr(rstd), dx=_lib.ptr(dx), dresidual=_lib.ptr(dres),
            dweight=_lib.ptr(dw), dbias=_lib.ptr(db), workspace=None, workspace_bytes=0, rows=rows,
            hidden=hidden, x_dtype=_lib.dtype_enum(x.dtype),
            residual_dtype=_lib.dtype_enum(residual.dtype) if residual is not None else 0,
            is_rms=int(bool(is_rms)), prenorm=int(bool(prenorm)))
        _lib.call("ssm_norm_bwd_static", args, dev)
        return dx, dres, dw, db
    dev = K.require_gpu(x, weight, residual, grad_out)
    xc, gc = K.cast_c(x, x.dtype), K.cast_c(grad_out, x.dtype)
    rc = K.cast_c(residual, residual.dtype) if residual is not None else None
    wf = K.as_f32_vec(weight)
    dx = torch.empty_like(xc)
    dres = torch.empty_like(rc) if (want_dres and rc is not None) else None
    dw = torch.empty(hidden, dtype=torch.float32, device=dev)
    db = torch.empty(hidden, dtype=torch.float32, device=dev) if want_dbias else None
    nbytes = _lib.load().ssm_norm_bwd_workspace_bytes(rows, hidden)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    args = _lib.NormBwdArgs(
        x=_lib.ptr(xc), residual=_lib.ptr(rc), dy=_lib.ptr(gc), weight=_lib.ptr(wf), mean=_lib.ptr(mean),
        rstd=_lib.ptr(rstd), dx=_lib.ptr(dx), dresidual=_lib.ptr(dres), dweight=_lib.ptr(dw),
        dbias=_lib.ptr(db), workspace=_lib.ptr(ws), workspace_bytes=nbytes, rows=rows, hidden=hidden,
        x_dtype=_lib.dtype_enum(xc.dtype),
        residual_dtype=_lib.dtype_enum(rc.dtype) if rc is not None else 0,
        is_rms=int(bool(is_rms)), prenorm=int(bool(prenorm)))
    _lib.call("ssm_norm_bwd", args, dev)
    return dx, dres, dw, db


def fused_layer_norm(x, weight, bias, residual=None, is_rms=False, eps=1e-5, prenorm=True,
                     residual_in_fp32=True):
    """Residual addition fused with LayerNorm or RMSNorm on the GPU.

    Args:
        x: Input ``(B, L, D)``.
        weight: Scale ``(D,)``.
        bias: Optional shift ``(D,)``.
        residual: Optional residual, same shape as ``x`` (any supported dtype).
        is_rms: RMSNorm when ``True``, LayerNorm otherwise.
        eps: Numerical stabiliser.
        prenorm: Add the residual before normalising (``True``) or after (``False``).
        residual_in_fp32: Kept for signature parity; sums are always formed in float32.

    Returns:
        Normalised tensor with the shape and dtype of ``x``.
    """
    tensors = (x, weight, bias, residual)
    if any(t is not None and t.requires_grad for t in tensors) and torch.is_grad_enabled():
        from ._autograd import FusedNormFn
        return FusedNormFn.apply(x, weight, bias, residual, bool(is_rms), float(eps), bool(prenorm),
                                 bool(residual_in_fp32), False)[0]
    return _norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32)[0]


def fused_layer_norm_with_residual(x, weight, bias, residual=None, is_rms=False, eps=1e-5,
                                   prenorm=True, residual_in_fp32=True):
    """Like :func:`fused_layer_norm` but also returns the pre-normalisation sum.

    The reference's operator returns only the normalised tensor
    (src/ssm/ops/python/reference.py:609), so a block has to redo ``x + residual``
    to carry the residual stream; this entry returns both from one pass.

    Args:
        x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32: as in
            :func:`fused_layer_norm`.

    Returns:
        ``(y, residual_out)`` where ``residual_out = x (+ residual if prenorm)`` in
        float32 when ``residual_in_fp32`` else in the residual's (or ``x``'s) dtype.
    """
    tensors = (x, weight, bias, residual)
    if any(t is not None and t.requires_grad for t in tensors) and torch.is_grad_enabled():
        from ._autograd import FusedNormFn
        return FusedNormFn.apply(x, weight, bias, residual, bool(is_rms), float(eps), bool(prenorm),
                                 bool(residual_in_fp32), True)
    y, res_out, _, _ = _norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32,
                                     want_residual_out=True)
    return y, res_out


__all__ = [
    "selective_scan",
    "selective_state_step",
    "decode_step",
    "mamba2_decode_step",
    "conv_window_step",
    "ssd_chunk_scan",
    "dw_causal_conv",
    "dw_causal_conv_channels_last",
    "fused_layer_norm",
    "fused_layer_norm_with_residual",
    "_cpu_backend_status",
    "_cuda_backend_status",
    "_hip_backend_status",
    "DeviceError",
]

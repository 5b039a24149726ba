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
                 out=None, last=None):
        batch, dim, length, nstate, (bkind, bgroups), (ckind, cgroups) = \
            K.check_selective_scan(u, delta, A, B, C, D, z, dt_bias)
        self.device = K.require_gpu(u, delta, A, B, C, D, z, dt_bias)
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
        self.args = _lib.ScanFwdArgs(
            u=_lib.ptr(k["u"]), delta=_lib.ptr(k["delta"]), z=_lib.ptr(k["z"]), A=_lib.ptr(k["A"]),
            Bproj=_lib.ptr(k["B"]), Cproj=_lib.ptr(k["C"]), Dskip=_lib.ptr(k["D"]),
            dt_bias=_lib.ptr(k["bias"]), out=_lib.ptr(self.out), last_state=_lib.ptr(self.last),
            batch=batch, dim=dim, seqlen=length, nstate=nstate,
            io_dtype=_lib.dtype_enum(io), bc_dtype=_lib.dtype_enum(bc),
            b_kind=bkind, c_kind=ckind, b_groups=bgroups, c_groups=cgroups,
            delta_softplus=int(bool(softplus)), tune_items=int(tune_items))

    def run(self):
        _lib.call("ssm_scan_fwd", self.args, self.device)
        return self.out, self.last


def _scan_forward(u, delta, A, B, C, D, z, dt_bias, softplus, want_state, tune_items=0):
    """Validate, normalise dtypes/layout, and run ``ssm_scan_fwd``."""
    plan = ScanPlan(u, delta, A, B, C, D, z, dt_bias, softplus, want_state, tune_items)
    out, last = plan.run()
    if out.dtype != plan.result_dtype:
        out = out.to(plan.result_dtype)
        last = last.to(plan.result_dtype) if last is not None else None
    return out, last


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


__all__ = [
    "selective_scan",
    "_cpu_backend_status",
    "_cuda_backend_status",
    "_hip_backend_status",
    "DeviceError",
]

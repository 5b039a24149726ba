"""The compiled-backend module the reference's ``ssm.ops`` façade expects, on top of this package.

The façade loads one module per device kind and calls ten functions on it by attribute
(/root/reference/src/ssm/ops/__init__.py: the autograd wrappers' ``_invoke_cuda`` calls at :317, :447, :595,
:653, :809, :868, :978, :1017, :1148, :1204 and the direct calls at :1289-1304, :1395-1411, :1516-1531,
:1594-1600, :1640-1655; argument names and defaults as the pybind signatures of
src/ssm/ops/cuda/bindings.cpp:96-152).  A ROCm build of PyTorch reports its devices as ``"cuda"``, so a
maintainer makes ``_load_cuda_ops()`` return :func:`load` and every call site above lands here unchanged.

Every function takes exactly the positional list of its call site and returns what the site unpacks:

====================================  ==========================================================================
``selective_scan``                    ``(y, last_state | None, cache)``; ``cache`` holds the row states entering
                                      each 512-step chunk, which ``selective_scan_backward`` restarts from.  (The
                                      direct call at :1289 unpacks two values where the autograd wrapper at :317
                                      unpacks three; the three-value form of the CUDA binding is kept, so that one
                                      site reads ``result[:2]``.)
``selective_scan_backward``           8 gradients ``(u, delta, A, B, C, D, z, dt_bias)``
``selective_state_step``              ``y``; ``state`` is updated in place
``selective_state_step_backward``     9 gradients ``(state, x, dt, A, B, C, D, z, dt_bias)``
``ssd_chunk_scan``                    ``Y``
``ssd_chunk_scan_backward``           8 gradients ``(X, dt, A, B, C, D, z, initial_states)``
``dw_causal_conv``                    ``y``
``dw_causal_conv_backward``           ``(dx, dweight, dbias | None)``
``fused_layer_norm``                  ``y``
``fused_layer_norm_backward``         ``(dx, dweight, dbias | None, dresidual | None)``
====================================  ==========================================================================

Gradients come back in the dtype of their tensor, ``None`` for an absent optional input.  Contract violations
surface as ``ValueError`` from the checks in ``ops._contract`` (the façade turns a backend's ``RuntimeError`` into
``ValueError`` anyway, :1237-1252).
"""

from __future__ import annotations

from typing import Optional

import torch

from . import ops as _ops
from .ops import _contract as _K


def _as(grad: Optional[torch.Tensor], ref: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if grad is None or ref is None:
        return None
    return grad.to(ref.dtype).reshape(ref.shape)


class HipBackend:
    """Namespace object with the ten entry points; ``name`` and ``available`` as the façade's status objects."""

    name = "hip"

    @property
    def available(self) -> bool:
        return bool(_ops._hip_backend_status().available)

    # ------------------------------------------------------------------ selective scan
    @staticmethod
    def selective_scan(u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False, return_last_state=False):
        plan = _ops.ScanPlan(u, delta, A, B, C, D, z, dt_bias, softplus, bool(return_last_state),
                             want_chunk_states=True)
        out, last = plan.run()
        if out.dtype != plan.result_dtype:
            out = out.to(plan.result_dtype)
            last = last.to(plan.result_dtype) if last is not None else None
        return out, last, plan.chunk_states

    @staticmethod
    def selective_scan_backward(grad_out, grad_last_state, u, delta, A, B, C, D=None, z=None, dt_bias=None,
                                softplus=False, forward_output=None, cache=None):
        nstate = A.shape[1]
        cs = cache if (cache is not None and cache.numel() > 0 and nstate <= 16) else None
        du, ddl, dA, dB, dC, dD, dz, dbias = _ops._scan_backward(grad_out, grad_last_state, u, delta, A, B, C, D, z,
                                                                 dt_bias, softplus, chunk_states=cs)
        return (_as(du, u), _as(ddl, delta), _as(dA, A), _as(dB, B), _as(dC, C), _as(dD, D), _as(dz, z),
                _as(dbias, dt_bias))

    # ------------------------------------------------------------------ single step
    @staticmethod
    def selective_state_step(state, x, dt, A, B, C, D=None, z=None, dt_bias=None, softplus=True):
        return _ops.selective_state_step(state, x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, softplus=softplus)

    @staticmethod
    def selective_state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D=None, z=None, dt_bias=None,
                                      softplus=True):
        grads = _ops._state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D, z, dt_bias, softplus)
        refs = (state, x, dt, A, B, C, D, z, dt_bias)
        return tuple(_as(g, r) for g, r in zip(grads, refs))

    # ------------------------------------------------------------------ diagonal chunk scan
    @staticmethod
    def _lengths(X, seq_lens, cu_seqlens):
        if cu_seqlens is not None:
            meta = {"cu_seqlens": cu_seqlens}
        elif seq_lens is not None:
            meta = {"seq_lens": seq_lens}
        else:
            meta = None
        return _K.sequence_lengths(meta, X.shape[0], X.device)

    @staticmethod
    def ssd_chunk_scan(X, dt, A, B, C, chunk_size, D=None, z=None, seq_lens=None, cu_seqlens=None,
                       initial_states=None):
        lengths = HipBackend._lengths(X, seq_lens, cu_seqlens)
        return _ops._dscan_forward(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)

    @staticmethod
    def ssd_chunk_scan_backward(grad_out, X, dt, A, B, C, chunk_size, D=None, z=None, seq_lens=None,
                                cu_seqlens=None, initial_states=None):
        lengths = HipBackend._lengths(X, seq_lens, cu_seqlens)
        grads = _ops._dscan_backward(grad_out, X, dt, A, B, C, chunk_size, D, z, lengths, initial_states)
        refs = (X, dt, A, B, C, D, z, initial_states)
        return tuple(_as(g, r) for g, r in zip(grads, refs))

    # ------------------------------------------------------------------ causal depthwise convolution
    @staticmethod
    def dw_causal_conv(x, weight, bias=None, activation="silu"):
        return _ops._conv_forward(x, weight, bias, activation)

    @staticmethod
    def dw_causal_conv_backward(grad_out, x, weight, bias=None, activation="silu"):
        dx, dw, db = _ops._conv_backward(grad_out, x, weight, bias, activation)
        return _as(dx, x), _as(dw, weight), _as(db, bias)

    # ------------------------------------------------------------------ residual add + norm
    @staticmethod
    def fused_layer_norm(x, weight, bias=None, residual=None, is_rms=False, eps=1e-5, prenorm=True,
                         residual_in_fp32=True):
        return _ops._norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32)[0]

    @staticmethod
    def fused_layer_norm_backward(grad_out, x, weight, bias=None, residual=None, is_rms=False, eps=1e-5,
                                  prenorm=True, residual_in_fp32=True):
        # the façade saves no row statistics (:1159-1170), so they are formed again here
        _, _, mean, rstd = _ops._norm_forward(x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32,
                                              want_stats=True)
        dx, dres, dw, db = _ops._norm_backward(grad_out, x, weight, residual, mean, rstd, is_rms, prenorm,
                                               bias is not None, residual is not None)
        return _as(dx, x), _as(dw, weight), _as(db, bias), _as(dres, residual)


def load() -> HipBackend:
    """The object to return from the façade's ``_load_cuda_ops()``; raises ``BackendUnavailable`` when the
    library cannot be loaded (the façade records that as its load error and falls back to its Python path)."""
    from . import _lib

    _lib.load()
    return HipBackend()

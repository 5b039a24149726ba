"""Dispatcher-level registration: the ten backend functions as ``torch.ops.ssm_amd.*``.

The reference's compiled backends declare their operators to PyTorch's dispatcher
(``TORCH_LIBRARY(ssm, ...)`` at /root/reference/src/ssm/ops/cpu/bindings.cpp:151-189, implementations for the
CPU at :191-203 and for CUDA at src/ssm/ops/cuda/bindings.cpp:155-165), which makes them visible to tracing:
an exported or compiled graph holds one opaque node per operator call.  This module does the same for this
backend: schemas, implementations for ROCm devices (PyTorch's ``CUDA`` dispatch key) that run the HIP kernels
through :mod:`ssm_amd.backend_module`, shape-only implementations for fake / meta tensors, and autograd
formulas that call the registered backward operators.

The namespace is ``ssm_amd`` and not ``ssm``: the reference's own declaration is not self-consistent (it
declares ``selective_state_step`` as returning two tensors and binds a function that returns one; it binds
``ssd_chunk_scan`` without declaring it), so its schemas cannot be taken over verbatim, and a second
``TORCH_LIBRARY(ssm)`` definition in one process is an error.  Argument names, order and defaults are the
reference's.  Differences, all of them in what a schema must say to be truthful:

* ``selective_state_step`` updates ``state`` in place and says so (``Tensor(a!) state``); it returns ``y``.
* ``selective_scan`` returns ``(y, last_state)``; ``last_state`` has no elements when it was not asked for.
* gradients of absent optional inputs come back as ``None`` (``Tensor?``), as in the reference.

Importing this module registers everything once; nothing else in the package depends on it.
"""

from __future__ import annotations

from typing import Optional

import torch

from .backend_module import HipBackend as _B

_NS = "ssm_amd"
_lib = torch.library.Library(_NS, "DEF")

_T = "Tensor"
_SCHEMAS = {
    "selective_scan":
        "(Tensor u, Tensor delta, Tensor A, Tensor B, Tensor C, Tensor? D=None, Tensor? z=None, "
        "Tensor? dt_bias=None, bool softplus=False, bool return_last_state=False) -> (Tensor, Tensor)",
    "selective_scan_backward":
        "(Tensor grad_output, Tensor? grad_last_state, Tensor u, Tensor delta, Tensor A, Tensor B, Tensor C, "
        "Tensor? D=None, Tensor? z=None, Tensor? dt_bias=None, bool softplus=False) "
        "-> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor?, Tensor?, Tensor?)",
    "selective_state_step":
        "(Tensor(a!) state, Tensor x, Tensor dt, Tensor A, Tensor B, Tensor C, Tensor? D=None, Tensor? z=None, "
        "Tensor? dt_bias=None, bool softplus=True) -> Tensor",
    "selective_state_step_backward":
        "(Tensor grad_output, Tensor? grad_state, Tensor state, Tensor x, Tensor dt, Tensor A, Tensor B, Tensor C, "
        "Tensor? D=None, Tensor? z=None, Tensor? dt_bias=None, bool softplus=True) "
        "-> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor, Tensor?, Tensor?, Tensor?)",
    "ssd_chunk_scan":
        "(Tensor X, Tensor dt, Tensor A, Tensor B, Tensor C, int chunk_size, Tensor? D=None, Tensor? z=None, "
        "Tensor? seq_lens=None, Tensor? cu_seqlens=None, Tensor? initial_states=None) -> Tensor",
    "ssd_chunk_scan_backward":
        "(Tensor grad_output, Tensor X, Tensor dt, Tensor A, Tensor B, Tensor C, int chunk_size, Tensor? D=None, "
        "Tensor? z=None, Tensor? seq_lens=None, Tensor? cu_seqlens=None, Tensor? initial_states=None) "
        "-> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor?, Tensor?, Tensor?)",
    "dw_causal_conv":
        "(Tensor x, Tensor weight, Tensor? bias=None, str activation='silu') -> Tensor",
    "dw_causal_conv_backward":
        "(Tensor grad_output, Tensor x, Tensor weight, Tensor? bias=None, str activation='silu') "
        "-> (Tensor, Tensor, Tensor?)",
    "fused_layer_norm":
        "(Tensor x, Tensor weight, Tensor? bias=None, Tensor? residual=None, bool is_rms=False, float eps=1e-5, "
        "bool prenorm=True, bool residual_in_fp32=True) -> Tensor",
    "fused_layer_norm_backward":
        "(Tensor grad_output, Tensor x, Tensor weight, Tensor? bias=None, Tensor? residual=None, bool is_rms=False, "
        "float eps=1e-5, bool prenorm=True, bool residual_in_fp32=True) -> (Tensor, Tensor, Tensor?, Tensor?)",
}
for _name, _schema in _SCHEMAS.items():
    _lib.define(_name + _schema)


def _like(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    """A dense tensor of the shape and type of ``t``: what the operators return whatever the strides of ``t`` are
    (a compiler plans the consumers of an output on the strides its fake promises)."""
    return None if t is None else torch.empty_like(t, memory_format=torch.contiguous_format)


# ------------------------------------------------------------------ implementations on the device

def _scan(u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False, return_last_state=False):
    out, last, _ = _B.selective_scan(u, delta, A, B, C, D, z, dt_bias, softplus, return_last_state)
    return out, (last if last is not None else u.new_empty(0))


def _scan_bwd(grad_output, grad_last_state, u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False):
    return _B.selective_scan_backward(grad_output, grad_last_state, u, delta, A, B, C, D, z, dt_bias, softplus)


_IMPLS = {
    "selective_scan": _scan,
    "selective_scan_backward": _scan_bwd,
    "selective_state_step": _B.selective_state_step,
    "selective_state_step_backward": _B.selective_state_step_backward,
    "ssd_chunk_scan": _B.ssd_chunk_scan,
    "ssd_chunk_scan_backward": _B.ssd_chunk_scan_backward,
    "dw_causal_conv": _B.dw_causal_conv,
    "dw_causal_conv_backward": _B.dw_causal_conv_backward,
    "fused_layer_norm": _B.fused_layer_norm,
    "fused_layer_norm_backward": _B.fused_layer_norm_backward,
}


# ------------------------------------------------------------------ shapes only (fake and meta tensors)

def _scan_meta(u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False, return_last_state=False):
    last = u.new_empty((u.shape[0], u.shape[1], A.shape[1])) if return_last_state else u.new_empty(0)
    return _like(u), last


def _scan_bwd_meta(grad_output, grad_last_state, u, delta, A, B, C, D=None, z=None, dt_bias=None, softplus=False):
    return tuple(_like(t) for t in (u, delta, A, B, C, D, z, dt_bias))


def _step_meta(state, x, dt, A, B, C, D=None, z=None, dt_bias=None, softplus=True):
    return _like(x)


def _step_bwd_meta(grad_output, grad_state, state, x, dt, A, B, C, D=None, z=None, dt_bias=None, softplus=True):
    return tuple(_like(t) for t in (state, x, dt, A, B, C, D, z, dt_bias))


def _chunk_meta(X, dt, A, B, C, chunk_size, D=None, z=None, seq_lens=None, cu_seqlens=None, initial_states=None):
    return _like(X)


def _chunk_bwd_meta(grad_output, X, dt, A, B, C, chunk_size, D=None, z=None, seq_lens=None, cu_seqlens=None,
                    initial_states=None):
    return tuple(_like(t) for t in (X, dt, A, B, C, D, z, initial_states))


def _conv_meta(x, weight, bias=None, activation="silu"):
    return _like(x)


def _conv_bwd_meta(grad_output, x, weight, bias=None, activation="silu"):
    # the gradient of a (B, C, L) view of rows of channels lies in rows of channels itself (ops._conv_backward)
    w = weight[:, 0, :] if weight.ndim == 3 else weight
    channels_first = x.ndim == 3 and x.shape[1] == w.shape[0]
    from .ops import _conv_rows_view
    if _conv_rows_view(x, channels_first, int(w.shape[-1])) is not None:
        dx = x.new_empty((x.shape[0], x.shape[2], x.shape[1])).permute(0, 2, 1)
    else:
        dx = _like(x)
    return dx, _like(weight), _like(bias)


def _norm_meta(x, weight, bias=None, residual=None, is_rms=False, eps=1e-5, prenorm=True, residual_in_fp32=True):
    return _like(x)


def _norm_bwd_meta(grad_output, x, weight, bias=None, residual=None, is_rms=False, eps=1e-5, prenorm=True,
                   residual_in_fp32=True):
    return _like(x), _like(weight), _like(bias), _like(residual)


_METAS = {
    "selective_scan": _scan_meta, "selective_scan_backward": _scan_bwd_meta,
    "selective_state_step": _step_meta, "selective_state_step_backward": _step_bwd_meta,
    "ssd_chunk_scan": _chunk_meta, "ssd_chunk_scan_backward": _chunk_bwd_meta,
    "dw_causal_conv": _conv_meta, "dw_causal_conv_backward": _conv_bwd_meta,
    "fused_layer_norm": _norm_meta, "fused_layer_norm_backward": _norm_bwd_meta,
}

for _name in _SCHEMAS:
    _lib.impl(_name, _IMPLS[_name], "CUDA")
    _lib.impl(_name, _METAS[_name], "Meta")


# ------------------------------------------------------------------ autograd of the functional operators
# (the in-place state step is a decoding operator; its gradients are reached through
#  ssm_amd::selective_state_step_backward or through ssm_amd.ops.selective_state_step)

_ops = getattr(torch.ops, _NS)


def _scan_setup(ctx, inputs, output):
    u, delta, A, B, C, D, z, dt_bias, softplus, return_last_state = inputs
    ctx.save_for_backward(u, delta, A, B, C, D, z, dt_bias)
    ctx.softplus, ctx.with_last = softplus, return_last_state


def _scan_autograd(ctx, grad_out, grad_last):
    u, delta, A, B, C, D, z, dt_bias = ctx.saved_tensors
    grads = _ops.selective_scan_backward(grad_out.contiguous(), grad_last if ctx.with_last else None, u, delta, A, B, C,
                                         D, z, dt_bias, ctx.softplus)
    return (*grads, None, None)


def _chunk_setup(ctx, inputs, output):
    X, dt, A, B, C, chunk_size, D, z, seq_lens, cu_seqlens, initial_states = inputs
    ctx.save_for_backward(X, dt, A, B, C, D, z, seq_lens, cu_seqlens, initial_states)
    ctx.chunk_size = chunk_size


def _chunk_autograd(ctx, grad_out):
    X, dt, A, B, C, D, z, seq_lens, cu_seqlens, initial_states = ctx.saved_tensors
    dX, ddt, dA, dB, dC, dD, dz, dinit = _ops.ssd_chunk_scan_backward(grad_out.contiguous(), X, dt, A, B, C,
                                                                       ctx.chunk_size, D, z, seq_lens, cu_seqlens,
                                                                       initial_states)
    return dX, ddt, dA, dB, dC, None, dD, dz, None, None, dinit


def _conv_setup(ctx, inputs, output):
    x, weight, bias, activation = inputs
    ctx.save_for_backward(x, weight, bias)
    ctx.activation = activation


def _conv_autograd(ctx, grad_out):
    x, weight, bias = ctx.saved_tensors
    dx, dw, db = _ops.dw_causal_conv_backward(grad_out.contiguous(), x, weight, bias, ctx.activation)
    return dx, dw, db, None


def _norm_setup(ctx, inputs, output):
    x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32 = inputs
    ctx.save_for_backward(x, weight, bias, residual)
    ctx.flags = (is_rms, eps, prenorm, residual_in_fp32)


def _norm_autograd(ctx, grad_out):
    x, weight, bias, residual = ctx.saved_tensors
    dx, dw, db, dres = _ops.fused_layer_norm_backward(grad_out.contiguous(), x, weight, bias, residual, *ctx.flags)
    return dx, dw, db, dres, None, None, None, None


torch.library.register_autograd(f"{_NS}::selective_scan", _scan_autograd, setup_context=_scan_setup, lib=_lib)
torch.library.register_autograd(f"{_NS}::ssd_chunk_scan", _chunk_autograd, setup_context=_chunk_setup, lib=_lib)
torch.library.register_autograd(f"{_NS}::dw_causal_conv", _conv_autograd, setup_context=_conv_setup, lib=_lib)
torch.library.register_autograd(f"{_NS}::fused_layer_norm", _norm_autograd, setup_context=_norm_setup, lib=_lib)

OPERATORS = tuple(_SCHEMAS)

"""``torch.autograd.Function`` wrappers that route backward passes to the HIP
kernels.

They play the role of the reference's ``_SelectiveScanCudaFunction`` ...
``_FusedLayerNormCudaFunction`` (src/ssm/ops/__init__.py:198-1224): what is
saved for backward, which inputs get gradients, and the rule that an input
which did not require a gradient receives ``None`` (``:284-291``).  Gradients
are returned in the dtype of the corresponding input.
"""

from __future__ import annotations

import torch

from . import _contract as K


def _like(grad, ref):
    """Cast/reshape a kernel gradient to what autograd expects for ``ref``."""
    if grad is None or ref is None:
        return None
    if grad.shape != ref.shape:
        grad = grad.reshape(ref.shape)
    return grad if grad.dtype == ref.dtype else grad.to(ref.dtype)


class CausalConvFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, activation, channels_last=None):
        from . import _conv_forward

        y = _conv_forward(x, weight, bias, activation, channels_last)
        ctx.save_for_backward(x, weight, bias)
        ctx.activation = activation
        ctx.channels_last = channels_last
        return y

    @staticmethod
    def backward(ctx, grad_out):
        from . import _conv_backward

        x, weight, bias = ctx.saved_tensors
        dx, dw, db = _conv_backward(grad_out, x, weight, bias, ctx.activation, ctx.channels_last)
        need = ctx.needs_input_grad
        return (_like(dx, x) if need[0] else None,
                _like(dw, weight) if need[1] else None,
                _like(db, bias) if (bias is not None and need[2]) else None,
                None, None)


class FusedNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, residual, is_rms, eps, prenorm, residual_in_fp32, want_res_out):
        from . import _norm_forward

        y, res_out, mean, rstd = _norm_forward(x, weight, bias, residual, is_rms, eps, prenorm,
                                               residual_in_fp32, want_residual_out=want_res_out,
                                               want_stats=True)
        ctx.save_for_backward(x, weight, bias, residual, mean, rstd)
        ctx.cfg = (is_rms, prenorm)
        if res_out is None:
            res_out = x.new_empty(0)
            ctx.mark_non_differentiable(res_out)
        ctx.has_res_out = want_res_out
        return y, res_out

    @staticmethod
    def backward(ctx, grad_y, grad_res_out):
        from . import _norm_backward

        x, weight, bias, residual, mean, rstd = ctx.saved_tensors
        is_rms, prenorm = ctx.cfg
        need = ctx.needs_input_grad
        want_dres = residual is not None and need[3]
        dx, dres, dw, db = _norm_backward(grad_y.contiguous(), x, weight, residual, mean, rstd, is_rms,
                                          prenorm, bias is not None, want_dres)
        if ctx.has_res_out and grad_res_out is not None and grad_res_out.numel() == x.numel():
            # residual_out = x (+ residual when prenorm): its gradient flows straight through
            dx = dx + grad_res_out.to(dx.dtype)
            if dres is not None and prenorm:
                dres = dres + grad_res_out.to(dres.dtype)
        return (_like(dx, x) if need[0] else None,
                _like(dw, weight) if need[1] else None,
                _like(db, bias) if (bias is not None and need[2]) else None,
                _like(dres, residual) if want_dres else None,
                None, None, None, None, None)


class SelectiveScanFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, u, delta, A, B, C, D, z, dt_bias, softplus, want_state):
        from . import ScanPlan, _BWD_MAX_STATES

        keep_cs = A.shape[-1] <= _BWD_MAX_STATES
        plan = ScanPlan(u, delta, A, B, C, D, z, dt_bias, softplus, want_state, want_chunk_states=keep_cs)
        out, last = plan.run()
        if out.dtype != u.dtype:
            out = out.to(u.dtype)
            last = last.to(u.dtype) if last is not None else None
        ctx.save_for_backward(u, delta, A, B, C, D, z, dt_bias, plan.chunk_states)
        ctx.softplus = softplus
        if last is None:
            last = u.new_empty(0)
            ctx.mark_non_differentiable(last)
        return out, last

    @staticmethod
    def backward(ctx, grad_out, grad_last):
        from . import _scan_backward

        u, delta, A, B, C, D, z, dt_bias, chunk_states = ctx.saved_tensors
        if grad_last is not None and grad_last.numel() == 0:
            grad_last = None
        grads = _scan_backward(grad_out, grad_last, u, delta, A, B, C, D, z, dt_bias, ctx.softplus,
                               chunk_states=chunk_states, grads_in_input_dtype=True)
        need = ctx.needs_input_grad
        refs = (u, delta, A, B, C, D, z, dt_bias)
        out = tuple(_like(g, r) if (r is not None and need[i]) else None
                    for i, (g, r) in enumerate(zip(grads, refs)))
        return out + (None, None)


class DiagScanFn(torch.autograd.Function):
    """The diagonal chunk scan; the role of the reference's ``_SsdChunkScanCudaFunction``
    (src/ssm/ops/__init__.py:780-905)."""

    @staticmethod
    def forward(ctx, X, dt, A, B, C, chunk_size, D, z, lengths, initial_states):
        from . import _dscan_forward

        # the forward leaves the state entering every 64 steps for the backward when its kernel can
        Y, table = _dscan_forward(X, dt, A, B, C, chunk_size, D, z, lengths, initial_states, want_round_states=True)
        ctx.save_for_backward(X, dt, A, B, C, D, z, lengths, initial_states, table)
        ctx.chunk_size = chunk_size
        return Y

    @staticmethod
    def backward(ctx, grad_y):
        from . import _dscan_backward

        X, dt, A, B, C, D, z, lengths, init, table = ctx.saved_tensors
        dX, ddt, dA, dB, dC, dD, dz, dinit = _dscan_backward(grad_y, X, dt, A, B, C, ctx.chunk_size, D, z, lengths,
                                                             init, grads_in_input_dtype=True, round_states=table)
        need = ctx.needs_input_grad
        pick = lambda i, g, r: _like(g, r) if (r is not None and need[i]) else None
        return (pick(0, dX, X), pick(1, ddt, dt), pick(2, dA, A), pick(3, dB, B), pick(4, dC, C), None,
                pick(6, dD, D), pick(7, dz, z), None, pick(9, dinit, init))


class StateStepFn(torch.autograd.Function):
    """One state update as a function ``(state, ...) -> (y, new_state)``; the role of the
    reference's ``_SelectiveStateStepCudaFunction`` (src/ssm/ops/__init__.py:570-668)."""

    @staticmethod
    def forward(ctx, state, x, dt, A, B, C, D, z, dt_bias, softplus):
        from . import StepPlan

        work = state.detach().clone().contiguous()
        plan = StepPlan(work, x.detach(), dt.detach(), A.detach(), B.detach(), C.detach(),
                        None if D is None else D.detach(), None if z is None else z.detach(),
                        None if dt_bias is None else dt_bias.detach(), softplus)
        out = plan.run()
        if out.dtype != plan.result_dtype:
            out = out.to(plan.result_dtype)
        # the caller overwrites `state` afterwards: keep the values the step started from
        ctx.save_for_backward(state.detach().clone(), x, dt, A, B, C, D, z, dt_bias)
        ctx.softplus = softplus
        return out, work

    @staticmethod
    def backward(ctx, grad_out, grad_state):
        from . import _state_step_backward

        state, x, dt, A, B, C, D, z, dt_bias = ctx.saved_tensors
        grads = _state_step_backward(grad_out, grad_state, state, x, dt, A, B, C, D, z, dt_bias, ctx.softplus)
        refs = (state, x, dt, A, B, C, D, z, dt_bias)
        need = ctx.needs_input_grad
        return tuple(_like(g, r) if (r is not None and need[i]) else None
                     for i, (g, r) in enumerate(zip(grads, refs))) + (None,)


def state_step_with_grad(state, x, dt, A, B, C, D, z, dt_bias, softplus):
    """Differentiable state update: runs the kernels through ``StateStepFn`` and then
    overwrites ``state`` with the new state, as the reference does
    (src/ssm/ops/__init__.py:1376-1393)."""
    out, new_state = StateStepFn.apply(state, x, dt, A, B, C, D, z, dt_bias, softplus)
    state.copy_(new_state)
    return out


class SsdCombinedFn(torch.autograd.Function):
    """Mamba-2 SSD ``(x, dt, A, B, C, ...) -> (y, final_states)``.  The reference has no code for
    this operator; the gradients it ships (``ssd_combined.combined_full`` in
    tests/mamba_reference_cases.json, made by the call at scripts/refresh_mamba_goldens.py:588-606)
    pin the backward."""

    @staticmethod
    def forward(ctx, x, dt, A, B, C, chunk_size, D, z, dt_bias, initial_states, dt_softplus, dt_limit,
                states_dtype, force_generic, fused, seq_idx=None):
        from .ssd import _ssd_combined_forward

        y, final = _ssd_combined_forward(x.detach(), dt.detach(), A.detach(), B.detach(), C.detach(), chunk_size,
                                         D=None if D is None else D.detach(), z=None if z is None else z.detach(),
                                         dt_bias=None if dt_bias is None else dt_bias.detach(),
                                         initial_states=None if initial_states is None else initial_states.detach(),
                                         dt_softplus=dt_softplus, dt_limit=dt_limit, return_final_states=True,
                                         states_dtype=states_dtype, force_generic=force_generic, fused=fused,
                                         seq_idx=seq_idx)
        ctx.save_for_backward(x, dt, A, B, C, D, z, dt_bias, initial_states)
        ctx.conf = (chunk_size, dt_softplus, dt_limit)
        ctx.seq_idx = seq_idx
        return y, final

    @staticmethod
    def backward(ctx, grad_y, grad_final):
        from .ssd import ssd_combined_backward

        x, dt, A, B, C, D, z, dt_bias, init = ctx.saved_tensors
        Q, softplus, limit = ctx.conf
        if grad_y is None:
            grad_y = torch.zeros_like(x)
        dx, ddt, dA, dB, dC, dD, dz, dbias, dinit = ssd_combined_backward(
            grad_y, grad_final, x, dt, A, B, C, Q, D=D, z=z, dt_bias=dt_bias, initial_states=init,
            dt_softplus=softplus, dt_limit=limit, seq_idx=ctx.seq_idx, grads_in_input_dtype=True)
        need = ctx.needs_input_grad
        pick = lambda i, g, r: _like(g, r) if (r is not None and g is not None and need[i]) else None
        return (pick(0, dx, x), pick(1, ddt, dt), pick(2, dA, A), pick(3, dB, B), pick(4, dC, C), None,
                pick(6, dD, D), pick(7, dz, z), pick(8, dbias, dt_bias), pick(9, dinit, init),
                None, None, None, None, None, None)


class SsdVarlenStatesFn(torch.autograd.Function):
    """The state at the last step of every sequence of a packed batch row, ``(nseq, H, P, N)``: the
    ``return_varlen_states`` output of the call at scripts/refresh_mamba_goldens.py:618-632 (the reference
    ships its values, ``ssd_combined.combined_varlen``; no gradients of it)."""

    @staticmethod
    def forward(ctx, x, dt, A, B, chunk_size, dt_bias, initial_states, dt_softplus, dt_limit, states_dtype,
                force_generic, seq_idx, cu_seqlens):
        from .ssd import _check_boundaries, _need, _ssd_shapes, _varlen_states_forward

        _need(_ssd_shapes(x, B)[0] == 1, "cu_seqlens describes one packed batch row: batch size must be 1.")
        _check_boundaries(seq_idx, [int(v) for v in cu_seqlens.tolist()], int(x.shape[1]))
        det = lambda t: None if t is None else t.detach()
        out = _varlen_states_forward(det(x), det(dt), det(A), det(B), chunk_size, det(dt_bias), det(initial_states),
                                     dt_softplus, dt_limit, states_dtype, force_generic, seq_idx, cu_seqlens)
        ctx.save_for_backward(x, dt, A, B, dt_bias, initial_states, cu_seqlens)
        ctx.conf = (dt_softplus, dt_limit)
        ctx.seq_idx = seq_idx
        return out

    @staticmethod
    def backward(ctx, grad_states):
        from .ssd import varlen_states_backward

        x, dt, A, B, dt_bias, init, cu = ctx.saved_tensors
        softplus, limit = ctx.conf
        dx, ddt, dA, dB, dbias, dinit = varlen_states_backward(
            grad_states, x, dt, A, B, cu, dt_bias=dt_bias, initial_states=init, dt_softplus=softplus,
            dt_limit=limit, seq_idx=ctx.seq_idx)
        need = ctx.needs_input_grad
        pick = lambda i, g, r: _like(g, r) if (r is not None and g is not None and need[i]) else None
        return (pick(0, dx, x), pick(1, ddt, dt), pick(2, dA, A), pick(3, dB, B), None, pick(5, dbias, dt_bias),
                pick(6, dinit, init), None, None, None, None, None, None)

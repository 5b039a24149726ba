"""CPU oracle for the five ``ssm.ops`` operators (test infrastructure only).

This module restates, on CPU tensors and with explicit time loops, what the
reference's pure-PyTorch path computes:

* ``selective_scan``        -> src/ssm/ops/python/reference.py:87-194
* ``selective_state_step``  -> src/ssm/ops/python/reference.py:197-309
* ``ssd_chunk_scan``        -> src/ssm/ops/python/reference.py:312-463
* ``dw_causal_conv``        -> src/ssm/ops/python/reference.py:466-537
* ``fused_layer_norm``      -> src/ssm/ops/python/reference.py:540-609
* accumulation dtype rule   -> src/ssm/ops/python/reference.py:9-19
* B/C broadcasting rules    -> src/ssm/ops/python/reference.py:22-84

Pinned by (see tests/test_oracle_golden.py): the reference's own JSON
goldens (``selective_scan_case1``, ``selective_scan_grouped``,
``selective_scan_reference`` x3, ``ssd_chunk_scan_case1``,
``ssd_chunk_scan_varlen``), the upstream-CUDA vectors in
``mamba_reference_cases.json`` (selective_scan fwd + gradients,
selective_state_update, dw_causal_conv fwd + gradients, layer norms fwd +
gradients), library special cases (``F.conv1d``, ``F.layer_norm``,
``F.rms_norm``) and closed forms (geometric series).

Every function takes ``acc`` (default ``None``): ``None`` applies the
reference's dtype policy (half/bfloat16 accumulate in float32, others in
their own dtype); ``torch.float64`` forces a double-precision evaluation used
to arbitrate between two float32 implementations that differ only by
re-association.

Gradients are obtained by running ``torch.autograd`` through these loops,
exactly as the reference defines its backward pass.
"""

from __future__ import annotations

from typing import Any, Optional

import torch
import torch.nn.functional as F


# ----------------------------------------------------------------------------
# dtype policy
# ----------------------------------------------------------------------------

def accumulation_dtype(t: torch.Tensor, A: Optional[torch.Tensor] = None,
                       acc: Optional[torch.dtype] = None) -> torch.dtype:
    """Accumulation dtype: half/bf16 -> fp32, otherwise unchanged; a non-fp32
    ``A`` promotes (reference.py:9-19, :135-137)."""
    if acc is not None:
        return acc
    if t.dtype in (torch.float16, torch.bfloat16):
        dt = torch.float32
    elif t.dtype == torch.complex32:
        dt = torch.complex64
    else:
        dt = t.dtype
    if A is not None and A.dtype != torch.float32 and A.dtype != dt:
        dt = torch.promote_types(dt, A.dtype)
    return dt


def _scan_proj(name: str, p: torch.Tensor, batch: int, dim: int, nstate: int,
               length: int, dt: torch.dtype) -> torch.Tensor:
    """Return a broadcastable view of a B/C projection indexed ``[b, d, n, t]``.

    Accepted forms (reference.py:22-56): ``(D,N)``, ``(B,D,N)`` and grouped
    time-varying ``(B,G,N,L)`` where channel ``d`` reads group ``d // (D/G)``.
    """
    if p.dim() == 2:
        if tuple(p.shape) != (dim, nstate):
            raise ValueError(f"{name} must have shape (D, N).")
        return p.to(dt)[None, :, :, None].expand(batch, dim, nstate, length)
    if p.dim() == 3:
        if tuple(p.shape) != (batch, dim, nstate):
            raise ValueError(f"{name} must have shape (B, D, N) when 3-D.")
        return p.to(dt)[:, :, :, None].expand(batch, dim, nstate, length)
    if p.dim() == 4:
        if p.shape[0] != batch or p.shape[3] != length:
            raise ValueError(f"{name} must have shape (B, G, N, L) when 4-D.")
        groups = p.shape[1]
        if groups == 0 or dim % groups != 0:
            raise ValueError("Group dimension must divide D.")
        if p.shape[2] != nstate:
            raise ValueError(f"{name} has mismatched state dimension.")
        per = dim // groups
        v = p.to(dt)[:, :, None, :, :].expand(batch, groups, per, nstate, length)
        return v.reshape(batch, dim, nstate, length)
    raise ValueError(f"Unsupported rank for {name}.")


# ----------------------------------------------------------------------------
# selective scan
# ----------------------------------------------------------------------------

def selective_scan(u, delta, A, B, C, D=None, z=None, dt_bias=None,
                   softplus=False, return_last_state=False, *, acc=None):
    """``h_t = exp(dt_t A) h_{t-1} + dt_t u_t B_t ; y_t = <h_t, C_t> + D u_t``,
    optionally gated by ``silu(z_t)``; zero initial state."""
    if u.ndim != 3 or delta.ndim != 3:
        raise ValueError("u and delta must have shape (B, D, L).")
    batch, dim, length = u.shape
    if tuple(delta.shape) != (batch, dim, length):
        raise ValueError("delta must match the shape of u.")
    if A.ndim != 2 or A.shape[0] != dim:
        raise ValueError("A must have shape (D, N).")
    nstate = A.shape[1]
    ct = accumulation_dtype(u, A, acc)

    uu = u.to(ct)
    dd = delta.to(ct)
    AA = A.to(ct)
    Bf = _scan_proj("B", B, batch, dim, nstate, length, ct)
    Cf = _scan_proj("C", C, batch, dim, nstate, length, ct)
    if D is not None and tuple(D.shape) != (dim,):
        raise ValueError("D must have shape (D,).")
    if z is not None and tuple(z.shape) != (batch, dim, length):
        raise ValueError("z must have shape (B, D, L).")
    if dt_bias is not None:
        if tuple(dt_bias.shape) != (dim,):
            raise ValueError("dt_bias must have shape (D,).")
        dd = dd + dt_bias.to(ct)[None, :, None]
    if softplus:
        dd = F.softplus(dd)

    h = torch.zeros(batch, dim, nstate, dtype=ct, device=u.device)
    ys = []
    for t in range(length):
        step = dd[:, :, t]
        h = torch.exp(step[:, :, None] * AA[None]) * h \
            + step[:, :, None] * (Bf[:, :, :, t] * uu[:, :, t, None])
        y = (h * Cf[:, :, :, t]).sum(dim=-1)
        if D is not None:
            y = y + D.to(ct)[None, :] * uu[:, :, t]
        if z is not None:
            y = y * F.silu(z[:, :, t].to(ct))
        ys.append(y)
    if ys:
        out = torch.stack(ys, dim=-1).to(u.dtype)
    else:
        out = torch.zeros_like(u)
    if return_last_state:
        return out, h.to(u.dtype)
    return out


# ----------------------------------------------------------------------------
# single-token state step
# ----------------------------------------------------------------------------

def _step_proj(name, p, batch, dim, nstate, dt):
    """B/C for one token: ``(D,N)``, ``(B,D,N)`` or grouped ``(B,G,N)`` which is
    recognised as "3-D, dim0 == batch, dim1 != D" (reference.py:252-272)."""
    if p.dim() == 3 and p.shape[0] == batch and p.shape[1] != dim:
        groups = p.shape[1]
        if groups == 0 or dim % groups != 0:
            raise ValueError(f"{name} group dimension must divide D.")
        if p.shape[2] != nstate:
            raise ValueError(f"{name} must have matching state dimension.")
        per = dim // groups
        p = p[:, :, None, :].expand(batch, groups, per, nstate).reshape(batch, dim, nstate)
    return _scan_proj(name, p, batch, dim, nstate, 1, dt)[:, :, :, 0]


def selective_state_step_functional(state, x, dt, A, B, C, D=None, z=None,
                                    dt_bias=None, softplus=True, *, acc=None):
    """Pure version: returns ``(y, new_state)`` in accumulation dtype casts
    applied as the reference does (``y`` -> ``x.dtype``, state -> ``state.dtype``)."""
    if state.ndim != 3:
        raise ValueError("state must have shape (B, D, N).")
    if x.ndim != 2 or dt.ndim != 2:
        raise ValueError("x and dt must have shape (B, D).")
    batch, dim, nstate = state.shape
    if tuple(x.shape) != (batch, dim) or tuple(dt.shape) != (batch, dim):
        raise ValueError("x and dt must match the first two dimensions of state.")
    if tuple(A.shape) != (dim, nstate):
        raise ValueError("A must have shape (D, N).")
    ct = accumulation_dtype(state, A, acc)
    Bf = _step_proj("B", B, batch, dim, nstate, ct)
    Cf = _step_proj("C", C, batch, dim, nstate, ct)
    if D is not None and tuple(D.shape) != (dim,):
        raise ValueError("D must have shape (D,).")
    if z is not None and tuple(z.shape) != (batch, dim):
        raise ValueError("z must have shape (B, D).")
    step = dt.to(ct)
    if dt_bias is not None:
        if tuple(dt_bias.shape) != (dim,):
            raise ValueError("dt_bias must have shape (D,).")
        step = step + dt_bias.to(ct)[None, :]
    if softplus:
        step = F.softplus(step)
    xx = x.to(ct)
    new_state = torch.exp(step[:, :, None] * A.to(ct)[None]) * state.to(ct) \
        + step[:, :, None] * (Bf * xx[:, :, None])
    y = (new_state * Cf).sum(dim=-1)
    if D is not None:
        y = y + D.to(ct)[None, :] * xx
    if z is not None:
        y = y * F.silu(z.to(ct))
    return y.to(x.dtype), new_state.to(state.dtype)


def selective_state_step(state, x, dt, A, B, C, D=None, z=None, dt_bias=None,
                         softplus=True, *, acc=None):
    """In-place flavour: ``state`` is overwritten (reference.py:308)."""
    y, new_state = selective_state_step_functional(
        state, x, dt, A, B, C, D=D, z=z, dt_bias=dt_bias, softplus=softplus, acc=acc)
    with torch.no_grad():
        state.copy_(new_state)
    return y


# ----------------------------------------------------------------------------
# "ssd_chunk_scan" with the reference's semantics: a diagonal, element-wise
# recurrence over (b, h, p); chunking is a no-op on the result.
# ----------------------------------------------------------------------------

def _chunk_proj(name, p, batch, seqlen, heads, proj, dt):
    if p.dim() == 2:
        if tuple(p.shape) != (heads, proj):
            raise ValueError(f"{name} must have shape (H, P).")
        return p.to(dt)[None, None].expand(batch, seqlen, heads, proj)
    if p.dim() == 3:
        if tuple(p.shape) != (batch, heads, proj):
            raise ValueError(f"{name} must be (B, H, P) when 3-D.")
        return p.to(dt)[:, None].expand(batch, seqlen, heads, proj)
    if p.dim() == 4:
        if tuple(p.shape) != (batch, seqlen, heads, proj):
            raise ValueError(f"{name} must have shape (B, L, H, P) when 4-D.")
        return p.to(dt)
    raise ValueError(f"Unsupported rank for {name}.")


def sequence_lengths(seq_meta: Optional[dict[str, Any]], batch: int, seqlen: int):
    """Valid length per batch row: ``cu_seqlens`` (B+1) wins over ``seq_lens``
    (B); absent -> full length (reference.py:413-428)."""
    if seq_meta is None:
        return [seqlen] * batch
    if "cu_seqlens" in seq_meta and seq_meta["cu_seqlens"] is not None:
        cu = torch.as_tensor(seq_meta["cu_seqlens"]).to(torch.long).flatten()
        if cu.numel() != batch + 1:
            raise ValueError("cu_seqlens must have length B + 1.")
        return [int(v) for v in (cu[1:] - cu[:-1]).tolist()]
    if "seq_lens" in seq_meta and seq_meta["seq_lens"] is not None:
        sl = torch.as_tensor(seq_meta["seq_lens"]).to(torch.long).flatten()
        if sl.numel() != batch:
            raise ValueError("seq_lens must have length B.")
        return [int(v) for v in sl.tolist()]
    raise ValueError("seq_meta must provide cu_seqlens or seq_lens.")


def ssd_chunk_scan(X, dt, A, B, C, chunk_size, D=None, z=None, seq_meta=None,
                   initial_states=None, *, acc=None):
    """``s_t = exp(dt_t A) s_{t-1} + dt_t B_t X_t ; y_t = s_t C_t + D X_t`` per
    ``(b, h, p)``; rows at or beyond the valid length are zero."""
    if X.ndim != 4:
        raise ValueError("X must have shape (B, L, H, P).")
    if dt.ndim != 3:
        raise ValueError("dt must have shape (B, L, H).")
    batch, seqlen, heads, proj = X.shape
    if tuple(dt.shape) != (batch, seqlen, heads):
        raise ValueError("dt must align with (B, L, H).")
    ct = accumulation_dtype(X, A, acc)
    if A.ndim == 1:
        if A.shape[0] != heads:
            raise ValueError("A must have shape (H,) when 1-D.")
        AA = A.to(ct)[:, None].expand(heads, proj)
    elif A.ndim == 2:
        if tuple(A.shape) != (heads, proj):
            raise ValueError("A must have shape (H, P) when 2-D.")
        AA = A.to(ct)
    else:
        raise ValueError("A must be 1-D or 2-D.")
    Bf = _chunk_proj("B", B, batch, seqlen, heads, proj, ct)
    Cf = _chunk_proj("C", C, batch, seqlen, heads, proj, ct)
    if D is None:
        Dv = None
    elif D.ndim == 1:
        if D.shape[0] != heads:
            raise ValueError("D must have shape (H,).")
        Dv = D.to(ct)[:, None].expand(heads, proj)
    elif D.ndim == 2:
        if tuple(D.shape) != (heads, proj):
            raise ValueError("D must have shape (H, P) when 2-D.")
        Dv = D.to(ct)
    else:
        raise ValueError("Unsupported rank for D.")
    if z is None:
        zz = None
    elif z.ndim == 3:
        if tuple(z.shape) != (batch, seqlen, heads):
            raise ValueError("z must have shape (B, L, H) when 3-D.")
        zz = z.to(ct)[..., None].expand(batch, seqlen, heads, proj)
    elif z.ndim == 4:
        if tuple(z.shape) != (batch, seqlen, heads, proj):
            raise ValueError("z must have shape (B, L, H, P) when 4-D.")
        zz = z.to(ct)
    else:
        raise ValueError("Unsupported rank for z.")
    if initial_states is not None:
        if tuple(initial_states.shape) != (batch, heads, proj):
            raise ValueError("initial_states must have shape (B, H, P).")
        s = initial_states.to(ct)
    else:
        s = torch.zeros(batch, heads, proj, dtype=ct, device=X.device)
    if int(chunk_size) <= 0:
        raise ValueError("chunk_size must be positive.")
    lengths = sequence_lengths(seq_meta, batch, seqlen)
    valid = torch.tensor(lengths, dtype=torch.long)
    if bool((valid < 0).any()) or bool((valid > seqlen).any()):
        raise ValueError("sequence lengths must lie in [0, L].")

    XX = X.to(ct)
    dd = dt.to(ct)
    rows = []
    # one view per step, split off up front: autograd then assembles each input's gradient once
    # instead of writing a tensor of the input's size per step
    X_t, dt_t, B_t, C_t = XX.unbind(1), dd.unbind(1), Bf.unbind(1), Cf.unbind(1)
    z_t = zz.unbind(1) if zz is not None else None
    for t in range(seqlen):
        live = (valid > t).to(ct)[:, None, None]          # (B,1,1)
        step = dt_t[t][:, :, None]                         # (B,H,1)
        s_new = torch.exp(step * AA[None]) * s + step * (B_t[t] * X_t[t])
        y = s_new * C_t[t]
        if Dv is not None:
            y = y + Dv[None] * X_t[t]
        if zz is not None:
            y = y * F.silu(z_t[t])
        # finished sequences neither advance their state nor emit output
        s = torch.where(live.bool(), s_new, s)
        rows.append(torch.where(live.bool(), y, torch.zeros_like(y)))
    if rows:
        out = torch.stack(rows, dim=1)
    else:
        out = torch.zeros(batch, 0, heads, proj, dtype=ct)
    return out.to(X.dtype)


# ----------------------------------------------------------------------------
# depthwise causal conv
# ----------------------------------------------------------------------------

def dw_causal_conv(x, weight, bias=None, activation="silu", *, acc=None):
    """``y[b,c,t] = act(bias[c] + sum_k w[c,k] x[b,c,t-(K-1)+k])`` written as an
    explicit tap sum (the reference calls ``F.conv1d`` on a left-padded input;
    tests/test_oracle_golden.py checks the two agree)."""
    if x.ndim != 3:
        raise ValueError("x must have shape (B, C, L) or (B, L, C).")
    chans = weight.shape[0]
    if x.shape[1] == chans:
        first = True
    elif x.shape[2] == chans:
        first = False
    else:
        raise ValueError("weight channel dimension must match x.")
    if weight.ndim == 2:
        w2 = weight
    elif weight.ndim == 3:
        if weight.shape[1] != 1:
            raise ValueError("Expected depthwise weights with shape (C, 1, K).")
        w2 = weight[:, 0, :]
    else:
        raise ValueError("weight must have 2 or 3 dimensions.")
    if bias is not None and tuple(bias.shape) != (chans,):
        raise ValueError("bias must have shape (C,).")
    act = str(activation).lower()
    if act not in ("silu", "swish", "identity", "none"):
        raise ValueError(f"Unsupported activation '{activation}'.")
    ct = accumulation_dtype(x, None, acc)
    xc = (x if first else x.permute(0, 2, 1)).to(ct)        # (B,C,L)
    length = xc.shape[2]
    K = w2.shape[1]
    wc = w2.to(ct)
    out = torch.zeros_like(xc)
    if bias is not None:
        out = out + bias.to(ct)[None, :, None]
    xp = F.pad(xc, (K - 1, 0))
    for k in range(K):
        out = out + wc[None, :, k, None] * xp[:, :, k:k + length]
    if act in ("silu", "swish"):
        out = F.silu(out)
    out = out if first else out.permute(0, 2, 1)
    return out.to(x.dtype)


# ----------------------------------------------------------------------------
# residual-add + LayerNorm / RMSNorm
# ----------------------------------------------------------------------------

def fused_layer_norm_with_residual(x, weight, bias, residual=None, is_rms=False,
                                   eps=1e-5, prenorm=True, residual_in_fp32=True,
                                   *, acc=None):
    """Returns ``(y, norm_input)``; ``norm_input`` is the pre-normalisation sum
    ``x (+ residual)`` in the base dtype (the "residual_out" of a fused block)."""
    if x.ndim != 3:
        raise ValueError("x must have shape (B, L, D).")
    hidden = x.shape[-1]
    if tuple(weight.shape) != (hidden,):
        raise ValueError("weight must match the last dimension of x.")
    if bias is not None and tuple(bias.shape) != (hidden,):
        raise ValueError("bias must match the last dimension of x.")
    if residual is not None and tuple(residual.shape) != tuple(x.shape):
        raise ValueError("residual must match the shape of x.")
    ct = accumulation_dtype(x, None, None)
    base = torch.float32 if (residual_in_fp32 and residual is not None) else ct
    if acc is not None:
        base = acc
    v = x.to(base)
    r = residual.to(base) if residual is not None else None
    if r is not None and prenorm:
        v = v + r
    if is_rms:
        normed = v * torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    else:
        mu = v.mean(dim=-1, keepdim=True)
        cen = v - mu
        normed = cen * torch.rsqrt((cen * cen).mean(dim=-1, keepdim=True) + eps)
    y = normed * weight.to(normed.dtype)
    if bias is not None:
        y = y + bias.to(normed.dtype)
    if r is not None and not prenorm:
        y = y + r.to(y.dtype)
    return y.to(x.dtype), v


def fused_layer_norm(x, weight, bias, residual=None, is_rms=False, eps=1e-5,
                     prenorm=True, residual_in_fp32=True, *, acc=None):
    return fused_layer_norm_with_residual(
        x, weight, bias, residual=residual, is_rms=is_rms, eps=eps,
        prenorm=prenorm, residual_in_fp32=residual_in_fp32, acc=acc)[0]

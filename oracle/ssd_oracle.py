"""CPU oracle for the state-space-duality (Mamba-2) operator family.

TEST INFRASTRUCTURE ONLY.

The reference repository has no code for this family (its ``ssd_chunk_scan``
is an element-wise diagonal recurrence, see ``ops_oracle.ssd_chunk_scan``).
Its semantics are fixed by vectors the reference ships, captured from the
third-party ``mamba_ssm`` Triton kernels (state-spaces/mamba, commit
10b5d6358f27966f6a40e4bf0baa17a460688128; recorded in the ``meta`` block of
tests/mamba_reference_cases.json) through the call sites in
scripts/refresh_mamba_goldens.py:405-486 (components), :568-632 (combined)
and :677-705 (bmm).  That dependency's source is not part of the reference
tree, so its published algorithm is restated here:

    dt'  = clamp(softplus(dt + dt_bias), dt_min, dt_max)
    h_t  = exp(dt'_t A_h) h_{t-1} + dt'_t x_t (outer) B_t          (P x N per head)
    y_t  = h_t C_t + D x_t ;  y_t *= silu(z_t)

and decomposed over chunks of Q tokens as

    chunk_cumsum   dA_cs[c,l]   = sum_{j<=l} dt'_j A_h
    bmm_chunk      CB[c,l,s]    = <C_l, B_s>
    chunk_state    S_c[p,n]     = sum_l B_l[n] exp(dA_cs[last]-dA_cs[l]) dt'_l x_l[p]
    state_passing  H_{c+1}      = exp(dA_cs[c,last]) H_c + S_c
    chunk_scan     y_l          = exp(dA_cs[l]) C_l.H_c
                                  + sum_{s<=l} CB[l,s] exp(dA_cs[l]-dA_cs[s]) dt'_s x_s + D x_l

Pinned by tests/test_oracle_golden.py against the fixture sections
``ssd_components`` (chunk_cumsum, chunk_cumsum_clamped, chunk_state,
state_passing, chunk_scan_*), ``ssd_bmm`` and ``ssd_combined.combined_full``
and by the identity "chunked == sequential" in float64.  The upstream kernels
evaluate ``exp(min(x, 0))`` for the intra-chunk decay factors; with A < 0 (the
only regime used by models) the clamp is inactive, but the fixtures use
random-sign A, so ``clamp_decay=True`` reproduces them.
"""

from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F


def prepare_dt(dt, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf")), acc=torch.float64):
    """(B,L,H) raw step -> effective step."""
    v = dt.to(acc)
    if dt_bias is not None:
        v = v + dt_bias.to(acc)[None, None, :]
    if dt_softplus:
        v = F.softplus(v)
    lo, hi = dt_limit
    # always applied, also with the default limits: a negative raw step (no softplus) becomes 0,
    # as the vectors of `ssd_combined.combined_varlen` show (y = 0 at their first token)
    return v.clamp(min=lo, max=hi)


def ssd_sequential(x, dt, A, B, C, D=None, z=None, dt_bias=None, dt_softplus=False,
                   dt_limit=(0.0, float("inf")), initial_states=None, acc=torch.float64):
    """Token-by-token recurrence; returns ``(y (B,L,H,P), final_states (B,H,P,N))``.

    Shapes: x (B,L,H,P); dt (B,L,H); A (H,); B,C (B,L,G,N); D (H,)|(H,P);
    z (B,L,H,P); initial_states (B,H,P,N).  ``A`` may also be given per step,
    ``(B,L,H)`` (the same value repeated): autograd then returns the terms
    ``dt_t q_t`` whose sum over batch and time is the gradient of ``A``, which
    lets a test measure an error in that sum against the size of its terms."""
    batch, seqlen, heads, hdim = x.shape
    groups, nstate = B.shape[2], B.shape[3]
    per = heads // groups
    dtv = prepare_dt(dt, dt_bias, dt_softplus, dt_limit, acc)
    xx = x.to(acc)
    Bh = B.to(acc).repeat_interleave(per, dim=2)     # (B,L,H,N)
    Ch = C.to(acc).repeat_interleave(per, dim=2)
    AA = A.to(acc)
    h = (initial_states.to(acc) if initial_states is not None
         else torch.zeros(batch, heads, hdim, nstate, dtype=acc))
    ys = []
    for t in range(seqlen):
        step = dtv[:, t]                                           # (B,H)
        decay = torch.exp(step * (AA[None] if AA.ndim == 1 else AA[:, t]))   # (B,H)
        h = decay[:, :, None, None] * h \
            + (step[:, :, None] * xx[:, t])[:, :, :, None] * Bh[:, t][:, :, None, :]
        y = (h * Ch[:, t][:, :, None, :]).sum(-1)                  # (B,H,P)
        if D is not None:
            Dv = D.to(acc)
            y = y + (Dv[None, :, None] if Dv.ndim == 1 else Dv[None]) * xx[:, t]
        if z is not None:
            y = y * F.silu(z[:, t].to(acc))
        ys.append(y)
    return torch.stack(ys, dim=1), h


def _pad_to_chunks(t, Q, dim=1):
    L = t.shape[dim]
    pad = (-L) % Q
    if pad == 0:
        return t
    shape = list(t.shape)
    shape[dim] = pad
    return torch.cat([t, torch.zeros(shape, dtype=t.dtype)], dim=dim)


def chunk_cumsum(dt, A, chunk_size, dt_bias=None, dt_softplus=False,
                 dt_limit=(0.0, float("inf")), acc=torch.float64):
    """-> ``(dA_cumsum, dt_out)`` each (B,H,nc,Q); the tail of a ragged last
    chunk has dt'=0."""
    Q = int(chunk_size)
    dtv = prepare_dt(dt, dt_bias, dt_softplus, dt_limit, acc)
    dtv = _pad_to_chunks(dtv, Q, dim=1)
    batch, Lp, heads = dtv.shape
    nc = Lp // Q
    dtc = dtv.view(batch, nc, Q, heads).permute(0, 3, 1, 2)          # (B,H,nc,Q)
    dA = dtc * A.to(acc)[None, :, None, None]
    return dA.cumsum(dim=-1), dtc.contiguous()


def bmm_chunk(a, b, chunk_size, seq_idx=None, causal=False, acc=torch.float64):
    """``out[b,c,(g,)l,s] = <a[b,cQ+l,(g,)], b[b,cQ+s,(g,)]>``; entries whose
    ``l`` and ``s`` lie in different sequences (``seq_idx``) are 0; with
    ``causal`` the strict upper triangle is returned as 0 (unspecified by the
    fixtures)."""
    Q = int(chunk_size)
    grouped = a.dim() == 4
    aa = a.to(acc) if grouped else a.to(acc)[:, :, None, :]
    bb = b.to(acc) if grouped else b.to(acc)[:, :, None, :]
    aa = _pad_to_chunks(aa, Q)
    bb = _pad_to_chunks(bb, Q)
    batch, Lp, G, K = aa.shape
    nc = Lp // Q
    ac = aa.view(batch, nc, Q, G, K)
    bc = bb.view(batch, nc, Q, G, K)
    out = torch.einsum("bclgk,bcsgk->bcgls", ac, bc)
    if seq_idx is not None:
        si = _pad_to_chunks(seq_idx.to(torch.long) + 1, Q).view(batch, nc, Q) - 1
        same = si[:, :, :, None] == si[:, :, None, :]
        out = out * same[:, :, None].to(acc)
    if causal:
        out = out * torch.tril(torch.ones(Q, Q, dtype=acc))
    return out if grouped else out[:, :, 0]


def _seg_exp(delta, clamp_decay):
    return torch.exp(delta.clamp(max=0.0)) if clamp_decay else torch.exp(delta)


def _chunk_last_ids(seq_idx, Q):
    """Sequence id of the last real step of every chunk: (B, nc)."""
    L = seq_idx.shape[1]
    nc = (L + Q - 1) // Q
    last = torch.tensor([min((c + 1) * Q, L) - 1 for c in range(nc)])
    return seq_idx.to(torch.long)[:, last]


def chunk_state(B, x, dt_c, dA_cumsum, clamp_decay=True, acc=torch.float64, seq_idx=None):
    """-> states (B,nc,H,P,N): contribution of each chunk to the state at its end.
    With ``seq_idx`` (B,L) only the steps that share the sequence id of the chunk's
    last step contribute."""
    batch, H, nc, Q = dt_c.shape
    G, N = B.shape[2], B.shape[3]
    per = H // G
    xx = _pad_to_chunks(x.to(acc), Q).view(batch, nc, Q, H, -1)
    Bh = _pad_to_chunks(B.to(acc), Q).view(batch, nc, Q, G, N).repeat_interleave(per, dim=3)
    dA = dA_cumsum.to(acc)
    w = _seg_exp(dA[..., -1:] - dA, clamp_decay) * dt_c.to(acc)      # (B,H,nc,Q)
    if seq_idx is not None:
        ids = _pad_to_chunks(seq_idx.to(torch.long) + 1, Q).view(batch, nc, Q) - 1      # padding: id -1
        same = ids == _chunk_last_ids(seq_idx, Q)[:, :, None]                           # (B,nc,Q)
        w = w * same[:, None].to(acc)
    return torch.einsum("bclhn,bhcl,bclhp->bchpn", Bh, w, xx)


def state_passing(states, dA_chunk_last, initial_states=None, acc=torch.float64, seq_idx=None, chunk_size=None):
    """states (B,nc,H,...); dA_chunk_last (B,H,nc).  Returns ``(entering, final)``
    where ``entering[:,c]`` is the state at the START of chunk c.  With ``seq_idx`` the
    carried state is dropped where the id of a chunk's last step differs from that of
    the chunk before; the initial state belongs to id 0."""
    st = states.to(acc)
    batch, nc, H = st.shape[:3]
    cur = (initial_states.to(acc).reshape(st[:, 0].shape) if initial_states is not None
           else torch.zeros_like(st[:, 0]))
    outs = []
    extra = (1,) * (st.dim() - 3)
    last_ids = _chunk_last_ids(seq_idx, int(chunk_size)) if seq_idx is not None else None
    prev_id = torch.zeros(batch, dtype=torch.long)
    for c in range(nc):
        outs.append(cur)
        g = torch.exp(dA_chunk_last.to(acc)[:, :, c]).view(batch, H, *extra)
        if last_ids is not None:
            keep = (last_ids[:, c] == prev_id).to(acc).view(batch, 1, *extra)
            g = g * keep
            prev_id = last_ids[:, c]
        cur = g * cur + st[:, c]
    return torch.stack(outs, dim=1), cur


def chunk_scan(B, C, x, dt_c, dA_cumsum, prev_states, D=None, z=None,
               clamp_decay=True, acc=torch.float64, seq_idx=None):
    """-> y (B,L,H,P) from entering states ``prev_states`` (B,nc,H,P,N).  With
    ``seq_idx`` the entering state only reaches steps whose id equals that of the last
    step of the chunk before (0 for the first chunk) and products across sequences
    inside a chunk are dropped."""
    batch, H, nc, Q = dt_c.shape
    L = x.shape[1]
    G, N = B.shape[2], B.shape[3]
    per = H // G
    P = x.shape[3]
    xx = _pad_to_chunks(x.to(acc), Q).view(batch, nc, Q, H, P)
    Bh = _pad_to_chunks(B.to(acc), Q).view(batch, nc, Q, G, N).repeat_interleave(per, dim=3)
    Ch = _pad_to_chunks(C.to(acc), Q).view(batch, nc, Q, G, N).repeat_interleave(per, dim=3)
    dA = dA_cumsum.to(acc)                                            # (B,H,nc,Q)
    # inter-chunk: exp(dA_cs[l]) * C_l . H_c
    y_off = torch.einsum("bclhn,bchpn->bclhp", Ch, prev_states.to(acc)) \
        * torch.exp(dA).permute(0, 2, 3, 1)[..., None]
    ids = None
    if seq_idx is not None:
        ids = _pad_to_chunks(seq_idx.to(torch.long) + 1, Q).view(batch, nc, Q) - 1
        last_ids = _chunk_last_ids(seq_idx, Q)
        prev_ids = torch.cat([torch.zeros(batch, 1, dtype=torch.long), last_ids[:, :-1]], dim=1)   # (B,nc)
        y_off = y_off * (ids == prev_ids[:, :, None]).to(acc)[..., None, None]
    # intra-chunk: sum_{s<=l} CB[l,s] * exp(dA_cs[l]-dA_cs[s]) * dt_s * x_s
    CB = torch.einsum("bclhn,bcshn->bchls", Ch, Bh)
    seg = dA.permute(0, 2, 1, 3)                                     # (B,nc,H,Q)
    decay = _seg_exp(seg[..., :, None] - seg[..., None, :], clamp_decay)
    mask = torch.tril(torch.ones(Q, Q, dtype=torch.bool))
    M = torch.where(mask, CB * decay, torch.zeros((), dtype=acc))
    if ids is not None:
        M = M * (ids[:, :, :, None] == ids[:, :, None, :]).to(acc)[:, :, None]
    M = M * dt_c.to(acc).permute(0, 2, 1, 3)[..., None, :]
    y_diag = torch.einsum("bchls,bcshp->bclhp", M, xx)
    y = y_off + y_diag
    if D is not None:
        Dv = D.to(acc)
        y = y + (Dv[None, None, None, :, None] if Dv.ndim == 1 else Dv[None, None, None]) * xx
    y = y.reshape(batch, nc * Q, H, P)[:, :L]
    if z is not None:
        y = y * F.silu(z.to(acc))
    return y


def chunk_state_varlen(B, x, dt_c, dA_cumsum, cu_seqlens, chunk_states, clamp_decay=True, acc=torch.float64):
    """State at the last step of every sequence of a packed batch row (batch 1):
    -> (nseq,H,P,N).  ``chunk_states`` (1,nc,H,P,N) are the states entering the chunks;
    the one entering the chunk of a sequence's last step counts only if the sequence
    began before that chunk (or at step 0: the row's initial state belongs to the first
    sequence).  Follows the routine behind
    ``mamba_chunk_scan_combined(..., cu_seqlens=, return_varlen_states=True)``
    (/root/reference/scripts/refresh_mamba_goldens.py:618-632)."""
    _, H, nc, Q = dt_c.shape
    G, N = B.shape[2], B.shape[3]
    per = H // G
    L = x.shape[1]
    xx = x.to(acc)[0]                                  # (L,H,P)
    Bh = B.to(acc)[0].repeat_interleave(per, dim=1)    # (L,H,N)
    dA = dA_cumsum.to(acc)[0]                          # (H,nc,Q)
    dtc = dt_c.to(acc)[0]
    cu = [int(v) for v in cu_seqlens]
    outs = []
    for i in range(len(cu) - 1):
        start, end = cu[i], min(cu[i + 1], L)
        st = torch.zeros(H, xx.shape[2], N, dtype=acc)
        if end > start:
            c = (end - 1) // Q
            last = dA[:, c, end - 1 - c * Q]           # (H,)
            if start < c * Q or start == 0:            # start == 0: the row's initial state belongs to the first sequence
                st = chunk_states.to(acc)[0, c] * torch.exp(last)[:, None, None]
            for t in range(max(start, c * Q), end):
                w = _seg_exp(last - dA[:, c, t - c * Q], clamp_decay) * dtc[:, c, t - c * Q]
                st = st + w[:, None, None] * xx[t][:, :, None] * Bh[t][:, None, :]
        outs.append(st)
    return torch.stack(outs, dim=0)


def ssd_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None,
                 initial_states=None, dt_softplus=False, dt_limit=(0.0, float("inf")),
                 clamp_decay=True, acc=torch.float64, seq_idx=None, cu_seqlens=None):
    """cumsum -> chunk_state -> state_passing -> chunk_scan; returns
    ``(y, final_states (B,H,P,N))``, and with ``cu_seqlens`` also the state at the end
    of every packed sequence."""
    dA_cs, dt_c = chunk_cumsum(dt, A, chunk_size, dt_bias, dt_softplus, dt_limit, acc)
    st = chunk_state(B, x, dt_c, dA_cs, clamp_decay, acc, seq_idx=seq_idx)
    entering, final = state_passing(st, dA_cs[..., -1], initial_states, acc, seq_idx=seq_idx, chunk_size=chunk_size)
    y = chunk_scan(B, C, x, dt_c, dA_cs, entering, D=D, z=z, clamp_decay=clamp_decay, acc=acc, seq_idx=seq_idx)
    if cu_seqlens is not None:
        return y, final, chunk_state_varlen(B, x, dt_c, dA_cs, cu_seqlens, entering, clamp_decay, acc)
    return y, final

"""State-space-duality (Mamba-2) operators on the GPU.

The reference repository ships no implementation of these (its
``ssd_chunk_scan`` is a diagonal recurrence, see :func:`ssm_amd.ops.ssd_chunk_scan`);
it only records their behaviour as vectors in ``tests/mamba_reference_cases.json``.
The functions below take the argument order of the calls that produced those
vectors (scripts/refresh_mamba_goldens.py:430-486, :591-604, :680-705) so that the
vectors can be replayed one to one.

Shapes: ``x, z, y (B, L, H, P)``; ``dt (B, L, H)``; ``A (H,)``; ``B, C (B, L, G, N)``;
``dt_out, dA_cumsum (B, H, nc, Q)`` float32; ``states (B, nc, H, P, N)``;
``final_states (B, H, P, N)`` float32, with ``nc = ceil(L / Q)``.
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from .. import _lib
from . import _contract as K


def _dims(batch, seqlen, heads, headdim, groups, nstate, chunk) -> _lib.SsdDims:
    return _lib.SsdDims(batch=batch, seqlen=seqlen, heads=heads, headdim=headdim, groups=groups,
                        nstate=nstate, chunk=chunk)


def _need(cond, msg):
    if not cond:
        raise ValueError(msg)


def chunk_cumsum(dt, A, chunk_size, dt_bias=None, dt_softplus=False, dt_limit=(0.0, float("inf"))):
    """Effective step and its chunk-wise running sum times ``A``.

    Args:
        dt: ``(B, L, H)`` raw steps.
        A: ``(H,)``.
        chunk_size: ``Q``.
        dt_bias: Optional ``(H,)`` added before ``softplus``.
        dt_softplus: Apply ``softplus`` to ``dt + dt_bias``.
        dt_limit: ``(min, max)`` clamp applied last.

    Returns:
        ``(dA_cumsum, dt_out)``, both ``(B, H, nc, Q)`` float32; steps past ``L`` in
        the last chunk have ``dt_out = 0``.
    """
    _need(dt.ndim == 3, "dt must have shape (B, L, H).")
    batch, seqlen, heads = (int(s) for s in dt.shape)
    _need(tuple(A.shape) == (heads,), "A must have shape (H,).")
    _need(dt_bias is None or tuple(dt_bias.shape) == (heads,), "dt_bias must have shape (H,).")
    Q = int(chunk_size)
    _need(Q > 0, "chunk_size must be positive.")
    K.check_float("dt", dt)
    dev = K.require_gpu(dt, A, dt_bias)
    nc = (seqlen + Q - 1) // Q
    dtc = K.cast_c(dt, dt.dtype)
    Af, bf = K.as_f32_vec(A), K.as_f32_vec(dt_bias)
    dA = torch.empty(batch, heads, nc, Q, dtype=torch.float32, device=dev)
    dto = torch.empty_like(dA)
    lo, hi = float(dt_limit[0]), float(dt_limit[1])
    args = _lib.SsdCumsumArgs(
        dt=_lib.ptr(dtc), A=_lib.ptr(Af), dt_bias=_lib.ptr(bf), dA_cumsum=_lib.ptr(dA), dt_out=_lib.ptr(dto),
        dims=_dims(batch, seqlen, heads, 1, 1, 1, Q), dt_dtype=_lib.dtype_enum(dtc.dtype),
        dt_softplus=int(bool(dt_softplus)), dt_min=lo if lo > -math.inf else -3.0e38,
        dt_max=hi if hi < math.inf else 3.0e38)
    _lib.call("ssm_ssd_chunk_cumsum", args, dev)
    return dA, dto


def bmm_chunk(a, b, chunk_size, seq_idx=None, causal=False, output_dtype=None, force_generic=False):
    """Per-chunk ``a b^T``: ``out[b, c, (g,) l, s] = <a[b, cQ+l, (g,)], b[b, cQ+s, (g,)]>``.

    Args:
        a, b: ``(B, L, K)`` or grouped ``(B, L, G, K)``.
        chunk_size: ``Q``.
        seq_idx: Optional ``(B, L)`` int sequence ids; products across sequences are 0.
        causal: Only ``s <= l`` is computed (the rest is returned as 0).
        output_dtype: dtype of the result (default: dtype of ``a``).

    Returns:
        ``(B, nc, Q, Q)`` or ``(B, nc, G, Q, Q)``.
    """
    _need(a.ndim in (3, 4) and a.shape == b.shape, "a and b must both be (B, L, K) or (B, L, G, K).")
    grouped = a.ndim == 4
    batch, seqlen = int(a.shape[0]), int(a.shape[1])
    groups = int(a.shape[2]) if grouped else 1
    kdim = int(a.shape[-1])
    Q = int(chunk_size)
    _need(Q > 0, "chunk_size must be positive.")
    K.check_float("a", a)
    K.check_float("b", b)
    dev = K.require_gpu(a, b, seq_idx)
    io = K.common_io_dtype([a, b])
    ac, bc = K.cast_c(a, io), K.cast_c(b, io)
    out_dt = output_dtype or a.dtype
    nc = (seqlen + Q - 1) // Q
    out = torch.empty((batch, nc, groups, Q, Q), dtype=out_dt, device=dev)
    si = None
    if seq_idx is not None:
        _need(tuple(seq_idx.shape) == (batch, seqlen), "seq_idx must have shape (B, L).")
        si = seq_idx.to(torch.int32).contiguous()
    args = _lib.SsdBmmArgs(a=_lib.ptr(ac), b=_lib.ptr(bc), seq_idx=_lib.ptr(si), out=_lib.ptr(out),
                           batch=batch, seqlen=seqlen, groups=groups, kdim=kdim, chunk=Q,
                           in_dtype=_lib.dtype_enum(io), out_dtype=_lib.dtype_enum(out_dt),
                           causal=int(bool(causal)), reserved=int(bool(force_generic)))
    _lib.call("ssm_ssd_bmm_chunk", args, dev)
    return out if grouped else out[:, :, 0]


def _ssd_shapes(x, B):
    _need(x.ndim == 4, "x must have shape (B, L, H, P).")
    _need(B.ndim == 4 and B.shape[0] == x.shape[0] and B.shape[1] == x.shape[1],
          "B and C must have shape (B, L, G, N).")
    batch, seqlen, heads, hdim = (int(s) for s in x.shape)
    groups, nstate = int(B.shape[2]), int(B.shape[3])
    _need(groups > 0 and heads % groups == 0, "ngroups must divide nheads.")
    return batch, seqlen, heads, hdim, groups, nstate


def _seq_idx_i32(seq_idx, batch, seqlen):
    """``seq_idx (B, L)`` as a contiguous int32 tensor (``None`` passes through)."""
    if seq_idx is None:
        return None
    _need(tuple(seq_idx.shape) == (batch, seqlen), "seq_idx must have shape (B, L).")
    _need(not seq_idx.dtype.is_floating_point, "seq_idx must hold integers.")
    return seq_idx.to(torch.int32).contiguous()


def _scale_arg(x_scale, dt):
    if x_scale is None:
        return None
    _need(x_scale.shape == dt.shape and x_scale.dtype == torch.float32 and x_scale.device == dt.device,
          "x_scale must be a float32 tensor of dt's shape (B, H, nc, Q).")
    return x_scale.contiguous()


def _row_scale_ok(x, Bm, Cm, chunk_size):
    """Whether ``chunk_state`` / ``chunk_scan`` take ``x_scale`` for these operands: the matrix-core kernels' shapes
    (bfloat16 tensors, whole chunks of a multiple of 32 up to 256 steps, a state size that is a multiple of 16, heads
    of 32 channels or a multiple of 64, which :func:`_lin_pass` cuts into pieces of 64)."""
    Q, seqlen, hdim, nstate = int(chunk_size), int(x.shape[1]), int(x.shape[-1]), int(Bm.shape[-1])
    return (x.dtype == torch.bfloat16 and Bm.dtype == x.dtype and Cm.dtype == x.dtype
            and seqlen % Q == 0 and Q % 32 == 0 and Q <= 256 and nstate % 16 == 0 and seqlen % 8 == 0
            and (hdim == 32 or hdim % 64 == 0))


def chunk_state(B, x, dt, dA_cumsum, states_dtype=torch.float32, force_generic=False, seq_idx=None, x_scale=None,
                x_reversed=False):
    """Contribution of each chunk to the state at its end.

    Args:
        B: ``(B, L, G, N)``.
        x: ``(B, L, H, P)``.
        dt: ``(B, H, nc, Q)`` float32 (``dt_out`` of :func:`chunk_cumsum`).
        dA_cumsum: ``(B, H, nc, Q)`` float32.
        states_dtype: dtype of the result.
        seq_idx: Optional ``(B, L)`` int sequence ids of a packed batch: steps of another
            sequence than the chunk's last step add nothing.
        x_scale: Optional ``(B, H, nc, Q)`` float32: ``x`` stands for ``x * x_scale`` rounded to ``x.dtype`` (only
            for calls :func:`_row_scale_ok` accepts).
        x_reversed: The call walks the sequence backwards in time (``B``, ``dt``, ``dA_cumsum`` given reversed) while
            ``x`` is given in forward time (same calls).

    Returns:
        ``states (B, nc, H, P, N)``.
    """
    batch, seqlen, heads, hdim, groups, nstate = _ssd_shapes(x, B)
    _need(dt.ndim == 4 and dt.shape == dA_cumsum.shape and dt.shape[0] == batch and dt.shape[1] == heads,
          "dt and dA_cumsum must have shape (B, H, nc, Q).")
    nc, Q = int(dt.shape[2]), int(dt.shape[3])
    _need(nc == (seqlen + Q - 1) // Q, "dt has the wrong number of chunks for this sequence length.")
    dev = K.require_gpu(B, x, dt, dA_cumsum, seq_idx)
    xc, Bc = K.cast_c(x, x.dtype), K.cast_c(B, B.dtype)
    K.check_float("x", xc)
    K.check_float("B", Bc)
    dtf, daf = K.as_f32_vec(dt), K.as_f32_vec(dA_cumsum)
    si = _seq_idx_i32(seq_idx, batch, seqlen)
    states = torch.empty(batch, nc, heads, hdim, nstate, dtype=states_dtype, device=dev)
    dims = _dims(batch, seqlen, heads, hdim, groups, nstate, Q)
    import ctypes
    nbytes = _lib.load().ssm_ssd_chunk_state_workspace_bytes(ctypes.byref(dims))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=dev)
    args = _lib.SsdChunkStateArgs(
        Bm=_lib.ptr(Bc), x=_lib.ptr(xc), dt=_lib.ptr(dtf), dA_cumsum=_lib.ptr(daf), states=_lib.ptr(states),
        workspace=_lib.ptr(ws), workspace_bytes=nbytes,
        dims=dims, x_dtype=_lib.dtype_enum(xc.dtype),
        b_dtype=_lib.dtype_enum(Bc.dtype), states_dtype=_lib.dtype_enum(states_dtype),
        reserved=int(bool(force_generic)), seq_idx=_lib.ptr(si), x_row_scale=_lib.ptr(_scale_arg(x_scale, dt)),
        x_time_reversed=int(bool(x_reversed)))
    _lib.call("ssm_ssd_chunk_state", args, dev)
    return states


def state_passing(states, dA_chunk_cumsum, initial_states=None, seq_idx=None, chunk_size=None):
    """Carry states across chunks: ``H_{c+1} = exp(dA_c) H_c + states_c``.

    Args:
        states: ``(B, nc, H, ...)`` per-chunk contributions (any trailing shape).
        dA_chunk_cumsum: ``(B, H, nc)``: ``dA_cumsum[..., -1]``.
        initial_states: Optional ``(B, H, ...)``.
        seq_idx: Optional ``(B, L)`` int sequence ids: the carried state is dropped where the
            id of a chunk's last step differs from that of the chunk before (the initial
            state belongs to id 0).  Needs ``chunk_size``.
        chunk_size: ``Q`` (only with ``seq_idx``).

    Returns:
        ``(states_passed, final_states)``: the state entering each chunk (shape and dtype
        of ``states``) and the state after the last chunk ``(B, H, ...)`` in float32.
    """
    _need(states.ndim >= 4, "states must have shape (B, nc, H, ...).")
    batch, nc, heads = (int(s) for s in states.shape[:3])
    trailing = tuple(int(s) for s in states.shape[3:])
    dim = 1
    for s_ in trailing:
        dim *= s_
    _need(tuple(dA_chunk_cumsum.shape) == (batch, heads, nc), "dA_chunk_cumsum must have shape (B, H, nc).")
    dev = K.require_gpu(states, dA_chunk_cumsum, initial_states, seq_idx)
    si, seqlen, Q = None, 0, 0
    if seq_idx is not None:
        _need(chunk_size is not None and int(chunk_size) > 0, "seq_idx needs chunk_size.")
        Q = int(chunk_size)
        _need(seq_idx.ndim == 2 and seq_idx.shape[0] == batch and (int(seq_idx.shape[1]) + Q - 1) // Q == nc,
              "seq_idx must have shape (B, L) with ceil(L / chunk_size) == nc.")
        seqlen = int(seq_idx.shape[1])
        si = _seq_idx_i32(seq_idx, batch, seqlen)
    sc = K.cast_c(states, states.dtype)
    K.check_float("states", sc)
    daf = K.as_f32_vec(dA_chunk_cumsum)
    init = None
    if initial_states is not None:
        _need(tuple(initial_states.shape) == (batch, heads) + trailing, "initial_states must have shape (B, H, ...).")
        init = K.as_f32_vec(initial_states)
    out = torch.empty_like(sc)
    final = torch.empty((batch, heads) + trailing, dtype=torch.float32, device=dev)
    args = _lib.SsdStatePassingArgs(
        states=_lib.ptr(sc), dA_chunk_last=_lib.ptr(daf), initial_states=_lib.ptr(init),
        states_out=_lib.ptr(out), final_states=_lib.ptr(final), batch=batch, nchunks=nc, heads=heads, dim=dim,
        states_dtype=_lib.dtype_enum(sc.dtype), seqlen=seqlen, chunk=Q, seq_idx=_lib.ptr(si))
    _lib.call("ssm_ssd_state_passing", args, dev)
    return out, final


def chunk_scan(B, C, x, dt, dA_cumsum, prev_states, D=None, z=None, CB=None, force_generic=False, seq_idx=None,
               out_f32=False, x_scale=None, dx_epilogue=None, x_reversed=False):
    """Outputs of every chunk from the state entering it.

    Args:
        B, C: ``(B, L, G, N)``.
        x: ``(B, L, H, P)``.
        dt, dA_cumsum: ``(B, H, nc, Q)`` float32.
        prev_states: ``(B, nc, H, P, N)`` state entering each chunk.
        D: Optional skip ``(H,)`` or ``(H, P)``.
        z: Optional gate ``(B, L, H, P)``.
        CB: Optional precomputed ``bmm_chunk(C, B, Q)`` (with the same ``seq_idx``).
        seq_idx: Optional ``(B, L)`` int sequence ids: the entering state only reaches steps
            whose id equals that of the last step of the chunk before (id 0 for the first
            chunk), and products across sequences inside a chunk are dropped.
        out_f32: Return ``y`` in float32 (the accumulators as they are) instead of ``x.dtype``.
        x_scale: As in :func:`chunk_state` (the skip term ``D x`` takes ``x`` as it is).
        x_reversed: As in :func:`chunk_state` (``C``, ``CB``, ``prev_states`` given reversed as well; not with ``D``).
        dx_epilogue: ``(x, dt_rows, D, out_dtype, round_dtx)`` -- the call is the gradient's time-reversed pass
            (``x`` here is ``dy`` reversed) and finishes ``dx`` itself instead of returning its result ``u``:
            returns ``(dx, xu, s1)`` as :func:`_bwd_dx` would from ``u`` (for calls :func:`_row_scale_ok` accepts
            with a head of 32 or 64 channels).

    Returns:
        ``y (B, L, H, P)`` in ``x.dtype`` (float32 with ``out_f32``).
    """
    batch, seqlen, heads, hdim, groups, nstate = _ssd_shapes(x, B)
    _need(C.shape == B.shape, "B and C must have the same shape.")
    _need(dt.ndim == 4 and dt.shape == dA_cumsum.shape and dt.shape[0] == batch and dt.shape[1] == heads,
          "dt and dA_cumsum must have shape (B, H, nc, Q).")
    nc, Q = int(dt.shape[2]), int(dt.shape[3])
    _need(tuple(prev_states.shape) == (batch, nc, heads, hdim, nstate),
          "prev_states must have shape (B, nc, H, P, N).")
    d_per_p = False
    if D is not None:
        _need(tuple(D.shape) in ((heads,), (heads, hdim)), "D must have shape (H,) or (H, P).")
        d_per_p = D.ndim == 2
    _need(z is None or z.shape == x.shape, "z must have the shape of x.")
    dev = K.require_gpu(B, C, x, dt, dA_cumsum, prev_states, D, z, seq_idx)
    si = _seq_idx_i32(seq_idx, batch, seqlen)
    if CB is None:
        CB = bmm_chunk(C, B, Q, seq_idx=si, causal=True,
                       output_dtype=x.dtype if x.dtype != torch.float32 else torch.float32, force_generic=force_generic)
    _need(tuple(CB.shape) == (batch, nc, groups, Q, Q), "CB must have shape (B, nc, G, Q, Q).")
    xc, Cc, zc = K.cast_c(x, x.dtype), K.cast_c(C, C.dtype), (K.cast_c(z, z.dtype) if z is not None else None)
    for name, t in (("x", xc), ("C", Cc), ("z", zc), ("CB", CB), ("prev_states", prev_states)):
        if t is not None:
            K.check_float(name, t)
    ps, cb = K.cast_c(prev_states, prev_states.dtype), K.cast_c(CB, CB.dtype)
    dtf, daf, Df = K.as_f32_vec(dt), K.as_f32_vec(dA_cumsum), K.as_f32_vec(D)
    y = dxo = None
    if dx_epilogue is None:
        y = torch.empty_like(xc, dtype=torch.float32) if out_f32 else torch.empty_like(xc)
    else:
        ex, edt, eD, eout, eround = dx_epilogue
        _need(ex.shape == xc.shape and ex.dtype == xc.dtype and ex.is_contiguous(), "dx_epilogue: x must match the operand.")
        _need(tuple(edt.shape) == (batch, seqlen, heads) and edt.dtype == torch.float32 and edt.is_contiguous(),
              "dx_epilogue: dt_rows must be a contiguous float32 (B, L, H) tensor.")
        _need(eout in (torch.float32, xc.dtype), "dx_epilogue: out_dtype is float32 or the operand's type.")
        eDf = K.as_f32_vec(eD)
        dxo = torch.empty(xc.shape, dtype=eout, device=dev)
        exu = torch.empty(batch, seqlen, heads, dtype=torch.float32, device=dev)
        es1 = torch.empty_like(exu)
    args = _lib.SsdChunkScanArgs(
        CB=_lib.ptr(cb), Cm=_lib.ptr(Cc), x=_lib.ptr(xc), z=_lib.ptr(zc), prev_states=_lib.ptr(ps),
        dt=_lib.ptr(dtf), dA_cumsum=_lib.ptr(daf), Dskip=_lib.ptr(Df), y=_lib.ptr(y),
        dims=_dims(batch, seqlen, heads, hdim, groups, nstate, Q), x_dtype=_lib.dtype_enum(xc.dtype),
        c_dtype=_lib.dtype_enum(Cc.dtype), cb_dtype=_lib.dtype_enum(cb.dtype),
        states_dtype=_lib.dtype_enum(ps.dtype), z_dtype=_lib.dtype_enum(zc.dtype) if zc is not None else 0,
        d_per_p=int(d_per_p), reserved=int(bool(force_generic)), seq_idx=_lib.ptr(si), y_f32=int(bool(out_f32)),
        x_row_scale=_lib.ptr(_scale_arg(x_scale, dt)), x_time_reversed=int(bool(x_reversed)))
    if dx_epilogue is not None:
        args.dx_x, args.dx_dt, args.dx_Dskip = _lib.ptr(ex), _lib.ptr(edt), _lib.ptr(eDf)
        args.dx_out, args.dx_xu, args.dx_s1 = _lib.ptr(dxo), _lib.ptr(exu), _lib.ptr(es1)
        args.dx_d_per_p = int(eD is not None and eD.ndim == 2)
        args.dx_out_f32 = int(eout == torch.float32)
        args.dx_round_dtx = int(bool(eround))
    _lib.call("ssm_ssd_chunk_scan", args, dev)
    return y if dx_epilogue is None else (dxo, exu, es1)


def chunk_state_varlen(B, x, dt, dA_cumsum, cu_seqlens, chunk_states):
    """State at the last step of every sequence of a packed batch row.

    Args:
        B: ``(1, L, G, N)``.
        x: ``(1, L, H, P)``.
        dt, dA_cumsum: ``(1, H, nc, Q)`` float32.
        cu_seqlens: ``(nseq + 1,)`` ints, increasing from 0: sequence ``i`` covers steps
            ``cu_seqlens[i] .. cu_seqlens[i+1] - 1``.
        chunk_states: ``(1, nc, H, P, N)`` state entering each chunk (from :func:`state_passing`
            with the matching ``seq_idx`` unless every sequence starts on a chunk boundary).

    Returns:
        ``states (nseq, H, P, N)`` float32.
    """
    batch, seqlen, heads, hdim, groups, nstate = _ssd_shapes(x, B)
    _need(batch == 1, "packed sequences need batch size 1.")
    _need(dt.ndim == 4 and dt.shape == dA_cumsum.shape and dt.shape[0] == 1 and dt.shape[1] == heads,
          "dt and dA_cumsum must have shape (1, H, nc, Q).")
    nc, Q = int(dt.shape[2]), int(dt.shape[3])
    _need(nc == (seqlen + Q - 1) // Q, "dt has the wrong number of chunks for this sequence length.")
    _need(tuple(chunk_states.shape) == (1, nc, heads, hdim, nstate), "chunk_states must have shape (1, nc, H, P, N).")
    _need(cu_seqlens.ndim == 1 and cu_seqlens.numel() >= 2 and not cu_seqlens.dtype.is_floating_point,
          "cu_seqlens must be a 1-D integer tensor of length nseq + 1.")
    dev = K.require_gpu(B, x, dt, dA_cumsum, cu_seqlens, chunk_states)
    nseq = int(cu_seqlens.numel()) - 1
    xc, Bc, cs = K.cast_c(x, x.dtype), K.cast_c(B, B.dtype), K.cast_c(chunk_states, chunk_states.dtype)
    for name, t in (("x", xc), ("B", Bc), ("chunk_states", cs)):
        K.check_float(name, t)
    dtf, daf = K.as_f32_vec(dt), K.as_f32_vec(dA_cumsum)
    cu = cu_seqlens.to(torch.int32).contiguous()
    out = torch.empty(nseq, heads, hdim, nstate, dtype=torch.float32, device=dev)
    args = _lib.SsdChunkStateVarlenArgs(
        Bm=_lib.ptr(Bc), x=_lib.ptr(xc), dt=_lib.ptr(dtf), dA_cumsum=_lib.ptr(daf), chunk_states=_lib.ptr(cs),
        cu_seqlens=_lib.ptr(cu), states=_lib.ptr(out), dims=_dims(1, seqlen, heads, hdim, groups, nstate, Q),
        nseq=nseq, x_dtype=_lib.dtype_enum(xc.dtype), b_dtype=_lib.dtype_enum(Bc.dtype),
        states_dtype=_lib.dtype_enum(cs.dtype))
    _lib.call("ssm_ssd_chunk_state_varlen", args, dev)
    return out


def _fused_ok(x, dt, B, C, z, D, batch, seqlen, heads, hdim, groups, nstate, Q):
    """Whether the one-pass kernel covers this call (bf16 or fp16 tensors of one type on the GPU and a
    shape ``ssm_ssd_combined_supported`` accepts)."""
    if Q <= 0 or seqlen % Q != 0:
        return False
    tensors = [x, B, C] + ([z] if z is not None else [])
    if x.dtype not in (torch.bfloat16, torch.float16) or any(t.dtype != x.dtype for t in tensors) or not x.is_cuda:
        return False
    dims = _dims(batch, seqlen, heads, hdim, groups, nstate, Q)
    return bool(_lib.load().ssm_ssd_combined_supported(dims, _lib.dtype_enum(x.dtype)))


def _rows_in_place(t):
    """``(tensor, row stride)`` for a ``(B, L, G, N)`` operand of the one-pass kernel: the tensor itself with the
    distance in elements between consecutive steps when its ``(G, N)`` blocks are dense, follow each other at one
    stride through batch and time, and start 16-byte aligned (a slice of wider rows); else a dense copy and 0."""
    b, l, g, n = t.shape
    sb, sl, sg, sn = t.stride()
    ok = (sn == 1 and (g == 1 or sg == n) and sl >= g * n and sl % 8 == 0 and (b == 1 or sb == l * sl)
          and t.data_ptr() % 16 == 0)
    return (t, int(sl)) if ok and not t.is_contiguous() else (K.cast_c(t, t.dtype), 0)


def _ssd_fused(x, dt, A, B, C, Q, D, z, dt_bias, initial_states, dt_softplus, dt_limit, return_final_states, shape,
               seq_idx=None):
    batch, seqlen, heads, hdim, groups, nstate = shape
    si = _seq_idx_i32(seq_idx, batch, seqlen)
    d_per_p = False
    if D is not None:
        _need(tuple(D.shape) in ((heads,), (heads, hdim)), "D must have shape (H,) or (H, P).")
        d_per_p = D.ndim == 2
    _need(z is None or z.shape == x.shape, "z must have the shape of x.")
    _need(tuple(A.shape) == (heads,), "A must have shape (H,).")
    _need(dt_bias is None or tuple(dt_bias.shape) == (heads,), "dt_bias must have shape (H,).")
    dev = K.require_gpu(x, dt, A, B, C, D, z, dt_bias, initial_states)
    xc = K.cast_c(x, x.dtype)
    # B and C cut out of wider rows (the two halves of one projection) are read where they are
    (Bc, b_row), (Cc, c_row) = _rows_in_place(B), _rows_in_place(C)
    zc = K.cast_c(z, z.dtype) if z is not None else None
    dtc = K.cast_c(dt, dt.dtype)
    K.check_float("dt", dtc)
    Af, Df, bf, init = K.as_f32_vec(A), K.as_f32_vec(D), K.as_f32_vec(dt_bias), K.as_f32_vec(initial_states)
    if d_per_p and Df.data_ptr() % 16:          # a view into a larger buffer: the kernel reads (H, P) factors as 16-byte vectors
        Df = Df.clone()
    dims = _dims(batch, seqlen, heads, hdim, groups, nstate, Q)
    nbytes = int(_lib.load().ssm_ssd_combined_workspace_bytes(dims))
    work = torch.empty(nbytes + 256, dtype=torch.uint8, device=dev)
    off = (-work.data_ptr()) % 256
    y = torch.empty_like(xc)
    final = torch.empty(batch, heads, hdim, nstate, dtype=torch.float32, device=dev) if return_final_states else None
    args = _lib.SsdCombinedArgs(
        x=_lib.ptr(xc), dt=_lib.ptr(dtc), A=_lib.ptr(Af), dt_bias=_lib.ptr(bf), Bm=_lib.ptr(Bc), Cm=_lib.ptr(Cc),
        Dskip=_lib.ptr(Df), z=_lib.ptr(zc), initial_states=_lib.ptr(init), y=_lib.ptr(y),
        final_states=_lib.ptr(final), workspace=work.data_ptr() + off, workspace_bytes=nbytes, dims=dims,
        io_dtype=_lib.dtype_enum(xc.dtype), dt_dtype=_lib.dtype_enum(dtc.dtype),
        dt_softplus=int(bool(dt_softplus)), d_per_p=int(d_per_p),
        dt_min=float(dt_limit[0]), dt_max=float(dt_limit[1]), seq_idx=_lib.ptr(si), b_row_stride=b_row,
        c_row_stride=c_row)
    _lib.call("ssm_ssd_combined_fwd", args, dev)
    if return_final_states:
        return y, final
    return y


def ssd_combined(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                 dt_softplus=False, dt_limit=(0.0, float("inf")), return_final_states=False,
                 states_dtype=None, force_generic=False, fused=None, seq_idx=None, cu_seqlens=None,
                 return_varlen_states=False):
    """Mamba-2 SSD, differentiable in ``x, dt, A, B, C, D, z, dt_bias, initial_states`` (gradients:
    :func:`ssd_combined_backward`).  bf16 and fp16 calls whose shape the one-pass kernel covers run
    ``ssm_ssd_combined_fwd``; everything else runs
    ``chunk_cumsum -> bmm_chunk, chunk_state -> state_passing -> chunk_scan``.

    Args:
        x: ``(B, L, H, P)``.
        dt: ``(B, L, H)``.
        A: ``(H,)`` (negative for a decaying system).
        B, C: ``(B, L, G, N)``.
        chunk_size: ``Q``.
        D: Optional skip ``(H,)`` or ``(H, P)``.
        z: Optional gate ``(B, L, H, P)``.
        dt_bias: Optional ``(H,)``.
        initial_states: Optional ``(B, H, P, N)``.
        dt_softplus: Apply ``softplus`` to ``dt + dt_bias``.
        dt_limit: ``(min, max)`` clamp of the effective step.
        return_final_states: Also return the state after the last token.
        states_dtype: dtype of the per-chunk states kept in HBM between the kernels
            (default: ``x.dtype``; the recurrence itself accumulates in float32).
        fused: ``None`` picks the one-pass kernel when it covers the call, ``False`` never uses it,
            ``True`` requires it (``ValueError`` if the call is not covered).  The values of ``A`` play no
            part in the choice and are never read on the host: the kernel looks at the sign of a head's
            ``A`` itself and treats a growing state as the five kernels do (decays inside a chunk bounded
            by 1, the carried state growing freely).
        seq_idx: Optional ``(B, L)`` int sequence ids of a packed batch (ids start at 0):
            no state and no product crosses from one sequence into the next.  The five kernels
            mask exactly.  The one-pass kernel (picked for bfloat16 calls it covers) and the
            backward separate sequences by an extra decay of ``2**-64`` at every first step
            instead: what crosses a boundary is scaled by 5e-20.
        cu_seqlens: Optional ``(nseq + 1,)`` sequence boundaries of a packed batch row
            (batch size 1), only used for ``return_varlen_states``.
        return_varlen_states: Also return the state at the last step of every sequence,
            ``(nseq, H, P, N)`` float32 (needs ``cu_seqlens``).  Differentiable in ``x, dt, A, B,
            dt_bias, initial_states`` when ``seq_idx`` changes exactly at the inner entries of
            ``cu_seqlens`` (:func:`varlen_states_backward`).

    Returns:
        ``y (B, L, H, P)`` in ``x.dtype``; with ``return_final_states`` and / or
        ``return_varlen_states`` a tuple ``(y[, final_states (B, H, P, N)][, varlen_states])``.
    """
    Q = int(chunk_size)
    seqlen = int(x.shape[1]) if x.ndim == 4 else 0
    if (x.ndim == 4 and x.dtype in (torch.bfloat16, torch.float16) and Q > 0 and seqlen % Q != 0 and not force_generic
            and float(dt_limit[0]) <= 0.0 and dt.ndim == 3):
        # The matrix-core kernels take whole chunks.  Steps of size zero neither decay the state nor add to
        # it, so a ragged end is filled up with them (zeros for x, B, C, z) and the extra rows of y dropped;
        # gradients flow through the padding and the slice.
        pad = (Q - seqlen % Q) % Q
        tpad = lambda t: None if t is None else torch.nn.functional.pad(t, (0, 0) * (t.ndim - 2) + (0, pad))
        if dt_softplus:
            dt_fill = torch.full_like(dt[:, :1], float("-inf")).expand(-1, pad, -1)     # softplus(-inf) = 0
        elif dt_bias is not None:
            # raw step + bias must be exactly zero: in float32 (a 16-bit -bias would leave bias - round(bias), a
            # small step that lets the state decay over the padding)
            dt = dt.to(torch.float32)
            dt_fill = (-dt_bias.detach().to(torch.float32))[None, None].expand(dt.shape[0], pad, -1)
        else:
            dt_fill = torch.zeros_like(dt[:, :1]).expand(-1, pad, -1)
        sp = None
        if seq_idx is not None:
            sp = torch.cat([seq_idx, seq_idx[:, -1:].expand(-1, pad)], dim=1)
        out = ssd_combined(tpad(x), torch.cat([dt, dt_fill], dim=1), A, tpad(B), tpad(C), Q, D=D, z=tpad(z),
                           dt_bias=dt_bias, initial_states=initial_states, dt_softplus=dt_softplus,
                           dt_limit=dt_limit, return_final_states=return_final_states, states_dtype=states_dtype,
                           force_generic=force_generic, fused=fused, seq_idx=sp, cu_seqlens=cu_seqlens,
                           return_varlen_states=return_varlen_states)
        if isinstance(out, tuple):
            return (out[0][:, :seqlen],) + tuple(out[1:])
        return out[:, :seqlen]
    tensors = (x, dt, A, B, C, D, z, dt_bias, initial_states)
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        from ._autograd import SsdCombinedFn, SsdVarlenStatesFn
        _need(not return_varlen_states or cu_seqlens is not None, "return_varlen_states needs cu_seqlens.")
        si = None if seq_idx is None else _seq_idx_i32(seq_idx, int(x.shape[0]), int(x.shape[1]))
        limit = (float(dt_limit[0]), float(dt_limit[1]))
        y, final = SsdCombinedFn.apply(x, dt, A, B, C, int(chunk_size), D, z, dt_bias, initial_states,
                                       bool(dt_softplus), limit, states_dtype, bool(force_generic), fused, si)
        outs = (y, final) if return_final_states else (y,)
        if return_varlen_states:
            # a second node of the graph: its gradients add to those of y and the final state
            outs += (SsdVarlenStatesFn.apply(x, dt, A, B, int(chunk_size), dt_bias, initial_states,
                                             bool(dt_softplus), limit, states_dtype, bool(force_generic), si,
                                             cu_seqlens),)
        return outs[0] if len(outs) == 1 else outs
    return _ssd_combined_forward(x, dt, A, B, C, chunk_size, D=D, z=z, dt_bias=dt_bias,
                                 initial_states=initial_states, dt_softplus=dt_softplus, dt_limit=dt_limit,
                                 return_final_states=return_final_states, states_dtype=states_dtype,
                                 force_generic=force_generic, fused=fused, seq_idx=seq_idx, cu_seqlens=cu_seqlens,
                                 return_varlen_states=return_varlen_states)


def _ssd_combined_forward(x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None, initial_states=None,
                          dt_softplus=False, dt_limit=(0.0, float("inf")), return_final_states=False,
                          states_dtype=None, force_generic=False, fused=None, seq_idx=None, cu_seqlens=None,
                          return_varlen_states=False):
    """The forward of :func:`ssd_combined` (same arguments); runs no autograd bookkeeping."""
    batch, seqlen, heads, hdim, groups, nstate = _ssd_shapes(x, B)
    _need(C.shape == B.shape, "B and C must have the same shape.")
    _need(tuple(dt.shape) == (batch, seqlen, heads), "dt must have shape (B, L, H).")
    _need(initial_states is None or tuple(initial_states.shape) == (batch, heads, hdim, nstate),
          "initial_states must have shape (B, H, P, N).")
    Q = int(chunk_size)
    _need(not return_varlen_states or cu_seqlens is not None, "return_varlen_states needs cu_seqlens.")
    _need(cu_seqlens is None or batch == 1, "cu_seqlens describes one packed batch row: batch size must be 1.")
    if x.dtype in (torch.bfloat16, torch.float16) and hdim > 64 and hdim % 64 == 0 and not force_generic:
        # Channels of a head do not interact: a head of 64k channels is k heads of 64 with the same step,
        # decay and group, which is the width the one-pass and matrix-core kernels are built for.  The
        # channel axis is innermost, so this is a view of x, z and the states.
        k = hdim // 64
        rep = lambda t: None if t is None else t.repeat_interleave(k, dim=-1)
        D2 = None if D is None else (D.repeat_interleave(k) if D.ndim == 1 else D.reshape(heads * k, 64))
        out = _ssd_combined_forward(
            x.reshape(batch, seqlen, heads * k, 64), rep(dt), rep(A), B, C, Q, D=D2,
            z=None if z is None else z.reshape(batch, seqlen, heads * k, 64), dt_bias=rep(dt_bias),
            initial_states=None if initial_states is None else initial_states.reshape(batch, heads * k, 64, nstate),
            dt_softplus=dt_softplus, dt_limit=dt_limit, return_final_states=return_final_states,
            states_dtype=states_dtype, fused=fused, seq_idx=seq_idx, cu_seqlens=cu_seqlens,
            return_varlen_states=return_varlen_states)
        outs = list(out) if isinstance(out, tuple) else [out]
        outs[0] = outs[0].reshape(batch, seqlen, heads, hdim)
        for i in range(1, len(outs)):                 # final states, per-sequence states: (.., H k, 64, N)
            outs[i] = outs[i].reshape(outs[i].shape[0], heads, hdim, nstate)
        return outs[0] if len(outs) == 1 else tuple(outs)
    can_fuse = not force_generic and fused is not False and not return_varlen_states and \
        _fused_ok(x, dt, B, C, z, D, batch, seqlen, heads, hdim, groups, nstate, Q)
    _need(can_fuse or not fused, "fused=True, but the one-pass kernel needs bf16 or fp16 x/B/C/z, headdim 64, "
          "chunk in {64,128,256}, nstate in {64,128} and seqlen % chunk == 0.")
    if can_fuse:
        return _ssd_fused(x, dt, A, B, C, Q, D, z, dt_bias, initial_states, dt_softplus, dt_limit,
                          return_final_states, (batch, seqlen, heads, hdim, groups, nstate), seq_idx=seq_idx)
    sdt = states_dtype or x.dtype
    dA, dtc = chunk_cumsum(dt, A, Q, dt_bias=dt_bias, dt_softplus=dt_softplus, dt_limit=dt_limit)
    states = chunk_state(B, x, dtc, dA, states_dtype=sdt, force_generic=force_generic, seq_idx=seq_idx)
    entering, final = state_passing(states, dA[:, :, :, -1].contiguous(), initial_states=initial_states,
                                    seq_idx=seq_idx, chunk_size=Q)
    y = chunk_scan(B, C, x, dtc, dA, entering, D=D, z=z, force_generic=force_generic, seq_idx=seq_idx)
    outs = [y]
    if return_final_states:
        outs.append(final)
    if return_varlen_states:
        outs.append(chunk_state_varlen(B, x, dtc, dA, cu_seqlens, entering))
    return outs[0] if len(outs) == 1 else tuple(outs)


def _varlen_states_forward(x, dt, A, B, chunk_size, dt_bias, initial_states, dt_softplus, dt_limit, states_dtype,
                           force_generic, seq_idx, cu_seqlens):
    """The per-sequence end states alone: ``chunk_cumsum -> chunk_state -> state_passing ->
    chunk_state_varlen``, the same kernels and the same dtype of the states between them as in
    :func:`_ssd_combined_forward`, so the values agree with its ``return_varlen_states`` output."""
    Q = int(chunk_size)
    dA, dtc = chunk_cumsum(dt, A, Q, dt_bias=dt_bias, dt_softplus=dt_softplus, dt_limit=dt_limit)
    states = chunk_state(B, x, dtc, dA, states_dtype=states_dtype or x.dtype, force_generic=force_generic,
                         seq_idx=seq_idx)
    entering, _ = state_passing(states, dA[:, :, :, -1].contiguous(), initial_states=initial_states,
                                seq_idx=seq_idx, chunk_size=Q)
    return chunk_state_varlen(B, x, dtc, dA, cu_seqlens, entering)


def _check_boundaries(seq_idx, cu, seqlen):
    """Gradients of the per-sequence end states are formed from ``cu_seqlens`` alone, so the sequences that
    ``seq_idx`` separates in the forward must be the same ones."""
    inner = sorted({v for v in cu[1:-1] if 0 < v < seqlen})
    if seq_idx is None:
        have = []
    else:
        row = seq_idx.reshape(-1, seqlen)[0]
        have = (torch.nonzero(row[1:] != row[:-1]).flatten() + 1).tolist()
    _need(have == inner, "gradients through the per-sequence end states need seq_idx to change exactly at the "
          "inner entries of cu_seqlens.")


def varlen_states_backward(dstates, x, dt, A, B, cu_seqlens, dt_bias=None, initial_states=None,
                           dt_softplus=False, dt_limit=(0.0, float("inf")), seq_idx=None):
    """Gradients of the per-sequence end states of a packed batch row (``return_varlen_states`` of
    :func:`ssd_combined`, the call at /root/reference/scripts/refresh_mamba_goldens.py:618-632).

    With ``w_t = exp(sum_{t < r < end} dt_r A)`` the end state of a sequence is
    ``sum_t w_t dt_t x_t (x) B_t`` over its steps, plus ``exp(sum_r dt_r A) * initial_states`` for the
    sequence that begins at step 0; this differentiates that sum sequence by sequence with float32
    tensor operations (a side output of packed batches: a few small products per sequence).

    Args:
        dstates: ``(nseq, H, P, N)`` gradient of the end states.
        x, dt, A, B, dt_bias, initial_states, dt_softplus, dt_limit, seq_idx: As given to the forward.
        cu_seqlens: ``(nseq + 1,)`` sequence boundaries.

    Returns:
        ``(dx, ddt, dA, dB, ddt_bias, dinitial_states)`` in float32 (the last two ``None`` without the input).
    """
    batch, seqlen, heads, hdim, groups, nstate = _ssd_shapes(x, B)
    _need(batch == 1, "cu_seqlens describes one packed batch row: batch size must be 1.")
    cu = [int(v) for v in cu_seqlens.tolist()]
    nseq = len(cu) - 1
    _need(tuple(dstates.shape) == (nseq, heads, hdim, nstate), "dstates must have shape (nseq, H, P, N).")
    _check_boundaries(seq_idx, cu, seqlen)
    per = heads // groups
    f32 = torch.float32
    Af = A.detach().to(f32)
    # The forward bounds the decays inside a chunk by 1 and lets the carried state grow across chunks, which is
    # not the plain sum this function differentiates; the two agree for a decaying system only.  (This path
    # already reads cu_seqlens on the host, so the look at A costs no further synchronisation.)
    _need(bool((Af <= 0).all()), "gradients through the per-sequence end states need A <= 0 on every head.")
    u = dt.detach().to(f32)[0]                                  # (L, H)
    if dt_bias is not None:
        u = u + dt_bias.detach().to(f32)
    sp = torch.nn.functional.softplus(u, threshold=20.0) if dt_softplus else u
    lo, hi = float(dt_limit[0]), float(dt_limit[1])
    dtp = sp.clamp(lo, hi)
    chain = ((sp >= lo) & (sp <= hi)).to(f32)                   # d dtp / d u
    if dt_softplus:
        chain = chain * torch.sigmoid(u)
    xf, Bf, G_all = x.detach()[0], B.detach()[0], dstates.detach().to(f32)
    dx = torch.zeros(1, seqlen, heads, hdim, device=x.device, dtype=f32)
    dB = torch.zeros(1, seqlen, groups, nstate, device=x.device, dtype=f32)
    ddtp = torch.zeros(seqlen, heads, device=x.device, dtype=f32)
    dA = torch.zeros(heads, device=x.device, dtype=f32)
    dinit = None if initial_states is None else torch.zeros_like(initial_states, dtype=f32)
    for i in range(nseq):
        a, e = cu[i], min(cu[i + 1], seqlen)
        if e <= a:
            continue
        G = G_all[i]                                            # (H, P, N)
        dts = dtp[a:e]
        cum = torch.cumsum(dts * Af, dim=0)
        w = torch.exp(cum[-1:] - cum)                           # decay from after step t to the end
        xs = xf[a:e].to(f32)
        Bh = Bf[a:e].to(f32).repeat_interleave(per, dim=1)      # (l, H, N)
        GB = torch.einsum("hpn,lhn->lhp", G, Bh)
        xG = torch.einsum("lhp,hpn->lhn", xs, G)
        coef = dts * w
        dx[0, a:e] = coef[..., None] * GB
        dB[0, a:e] = (coef[..., None] * xG).reshape(e - a, groups, per, nstate).sum(dim=2)
        sdot = (xs * GB).sum(dim=-1)                            # x_t' G B_t
        contrib = coef * sdot
        # dt_r A enters every term of an earlier step: the sum of those terms
        ddA = torch.cumsum(contrib, dim=0) - contrib
        if a == 0 and initial_states is not None:
            tot = torch.exp(cum[-1])                            # (H,)
            dinit[0] = tot[:, None, None] * G
            ddA = ddA + (tot * (G * initial_states.detach()[0].to(f32)).sum(dim=(1, 2)))[None]
        ddtp[a:e] = w * sdot + ddA * Af
        dA += (ddA * dts).sum(dim=0)
    ddt = (ddtp * chain)[None]
    dbias = None if dt_bias is None else ddt.sum(dim=(0, 1))
    return dx, ddt, dA, dB, dbias, dinit


def _lin_pass(x, w_c, dA_cs, Bm, Cm, init=None, want_entering=False, CB=None, x_scale=None, dx_epilogue=None,
              x_reversed=False):
    """``y_t = sum_{s<=t} exp(cs_t - cs_s) <C_t, B_s> w_s x_s + exp(cs_t) C_t . init`` and the state
    after the last step, through chunk_state -> state_passing -> chunk_scan (states in float32).

    Channels are independent of each other, so with bfloat16 operands a head dimension beyond 64 (the
    backward's passes that put the state axis in the channel role) is cut into pieces of 64, the width
    the matrix-core kernels are built for.  With ``want_entering`` the states entering the chunks
    ``(B, nc, H, P, N)`` come back as a third result.  ``x_scale (B, H, nc, Q)``: ``x`` stands for ``x * x_scale``
    rounded to its type (for calls :func:`_row_scale_ok` accepts).  ``dx_epilogue``: see :func:`chunk_scan`; the first
    result then is ``(dx, xu, s1)`` (heads of at most 64 channels).  ``x_reversed``: everything but ``x`` is given
    reversed in time, ``x`` in forward time (same calls)."""
    hd = int(x.shape[-1])
    if x.dtype == torch.bfloat16 and hd > 64 and hd % 64 == 0:
        Q = int(dA_cs.shape[3])
        CB = bmm_chunk(Cm, Bm, Q, causal=True, output_dtype=x.dtype)          # the same for every piece
        parts = [_lin_pass(x[..., k:k + 64].contiguous(), w_c, dA_cs, Bm, Cm,
                           None if init is None else init[:, :, k:k + 64].contiguous(), want_entering, CB=CB,
                           x_scale=x_scale, x_reversed=x_reversed)
                 for k in range(0, hd, 64)]
        out = (torch.cat([q[0] for q in parts], dim=-1), torch.cat([q[1] for q in parts], dim=2))
        return out + (torch.cat([q[2] for q in parts], dim=3),) if want_entering else out
    states = chunk_state(Bm, x, w_c, dA_cs, states_dtype=torch.float32, x_scale=x_scale, x_reversed=x_reversed)
    entering, final = state_passing(states, dA_cs[:, :, :, -1].contiguous(), initial_states=init)
    y = chunk_scan(Bm, Cm, x, w_c, dA_cs, entering, CB=CB, out_f32=True, x_scale=x_scale, dx_epilogue=dx_epilogue,
                   x_reversed=x_reversed)
    return (y, final, entering) if want_entering else (y, final)


def _elem_stages_ok(x, dout, z, hdim):
    """Whether the fused element-wise stages of the backward take this call: one dtype for ``x``, ``dout``
    and ``z``, and a head dimension of 4 * 2^k (at most 256)."""
    q = hdim // 4
    return (hdim % 4 == 0 and 1 <= q <= 64 and (q & (q - 1)) == 0 and dout.dtype == x.dtype
            and (z is None or z.dtype == x.dtype))


def _bwd_gate(dout, z, x, ypre, Df, cd, want_rev=True, w_dy=None, w_x=None, grads_io=False):
    """``ssm_ssd_bwd_gate``: ``(dy, dy_rev, dz, s2, dyx)``; with the per-row weights ``w_dy``, ``w_x (B, L, H)``
    also ``dy * w_dy`` and ``x * w_x`` in ``dy``'s type, as the sixth and seventh result."""
    batch, seqlen, heads, hdim = (int(v) for v in x.shape)
    dev = x.device
    dy = torch.empty(batch, seqlen, heads, hdim, dtype=cd, device=dev)
    dy_rev = torch.empty_like(dy) if want_rev else None
    dz = (torch.empty(batch, seqlen, heads, hdim, dtype=x.dtype if grads_io else torch.float32, device=dev)
          if z is not None else None)
    s2 = torch.empty(batch, seqlen, heads, dtype=torch.float32, device=dev)
    dyx = torch.empty_like(s2)
    dy_w = torch.empty_like(dy) if w_dy is not None else None
    x_w = torch.empty_like(dy) if w_x is not None else None
    args = _lib.SsdBwdGateArgs(
        dout=_lib.ptr(dout), z=_lib.ptr(z), x=_lib.ptr(x), ypre=_lib.ptr(ypre), Dskip=_lib.ptr(Df), dy=_lib.ptr(dy),
        dy_rev=_lib.ptr(dy_rev), dz=_lib.ptr(dz), s2=_lib.ptr(s2), dyx=_lib.ptr(dyx), batch=batch, seqlen=seqlen,
        heads=heads, headdim=hdim, io_dtype=_lib.dtype_enum(x.dtype), dy_dtype=_lib.dtype_enum(cd),
        d_per_p=int(Df is not None and Df.ndim == 2), w_dy=_lib.ptr(w_dy), w_x=_lib.ptr(w_x), dy_w=_lib.ptr(dy_w),
        x_w=_lib.ptr(x_w), dz_in_io_dtype=int(bool(grads_io)))
    _lib.call("ssm_ssd_bwd_gate", args, dev)
    if w_dy is not None or w_x is not None:
        return dy, dy_rev, dz, s2, dyx, dy_w, x_w
    return dy, dy_rev, dz, s2, dyx


def _bwd_dx(dout, z, x, u_rev, dte, Df, round_bf16, grads_io=False):
    """``ssm_ssd_bwd_dx``: ``(dx, xu, s1)``."""
    batch, seqlen, heads, hdim = (int(v) for v in x.shape)
    dev = x.device
    dx = torch.empty(batch, seqlen, heads, hdim, dtype=x.dtype if grads_io else torch.float32, device=dev)
    xu = torch.empty(batch, seqlen, heads, dtype=torch.float32, device=dev)
    s1 = torch.empty_like(xu)
    args = _lib.SsdBwdDxArgs(
        dout=_lib.ptr(dout), z=_lib.ptr(z), x=_lib.ptr(x), u_rev=_lib.ptr(u_rev), dt=_lib.ptr(dte), Dskip=_lib.ptr(Df),
        dx=_lib.ptr(dx), xu=_lib.ptr(xu), s1=_lib.ptr(s1), batch=batch, seqlen=seqlen, heads=heads, headdim=hdim,
        io_dtype=_lib.dtype_enum(x.dtype), d_per_p=int(Df is not None and Df.ndim == 2), round_bf16=int(bool(round_bf16)),
        dx_in_io_dtype=int(bool(grads_io)))
    _lib.call("ssm_ssd_bwd_dx", args, dev)
    return dx, xu, s1


def _bwd_db(v_rev, dte, groups):
    """``ssm_ssd_bwd_db``: ``dB (B, L, G, N)`` from the reversed pass output ``(B, L, H, N)``."""
    batch, seqlen, heads, nstate = (int(v) for v in v_rev.shape)
    dB = torch.empty(batch, seqlen, groups, nstate, dtype=torch.float32, device=v_rev.device)
    args = _lib.SsdBwdDbArgs(v_rev=_lib.ptr(v_rev), dt=_lib.ptr(dte), dB=_lib.ptr(dB), batch=batch, seqlen=seqlen,
                             heads=heads, groups=groups, nstate=nstate)
    _lib.call("ssm_ssd_bwd_db", args, v_rev.device)
    return dB


def _bwd_dcb(dy, x, dt_c, dA_cs, groups):
    """``ssm_ssd_bwd_dcb``: ``(B, nc, G, Q, Q)`` float32, the head-summed weighted ``<dy_l, x_s>`` of every chunk."""
    batch, seqlen, heads, hdim = (int(v) for v in x.shape)
    nc, Q = int(dA_cs.shape[2]), int(dA_cs.shape[3])
    out = torch.empty(batch, nc, groups, Q, Q, dtype=torch.float32, device=x.device)
    args = _lib.SsdBwdDcbArgs(dy=_lib.ptr(dy), x=_lib.ptr(x), dt=_lib.ptr(dt_c), dA_cumsum=_lib.ptr(dA_cs),
                              dCB=_lib.ptr(out), batch=batch, seqlen=seqlen, heads=heads, headdim=hdim, groups=groups,
                              chunk=Q)
    _lib.call("ssm_ssd_bwd_dcb", args, x.device)
    return out


def _bwd_dt(s1, s2, xu, dte, dt_raw, Af, dt_bias, W0, anchor, first, Q, dt_softplus, dt_limit):
    """``ssm_ssd_bwd_dt``: ``(ddt (B, L, H), dA (H,), dbias (H,))``."""
    batch, seqlen, heads = (int(v) for v in dte.shape)
    nc = seqlen // Q
    dev = dte.device
    f32 = dict(dtype=torch.float32, device=dev)
    ddt = torch.empty(batch, seqlen, heads, **f32)
    dA_p = torch.empty(batch, nc, heads, **f32)
    db_p = torch.empty_like(dA_p)
    lo, hi = float(dt_limit[0]), float(dt_limit[1])
    args = _lib.SsdBwdDtArgs(
        s1=_lib.ptr(s1), s2=_lib.ptr(s2), xu=_lib.ptr(xu), dt=_lib.ptr(dte), dt_raw=_lib.ptr(dt_raw), A=_lib.ptr(Af),
        dt_bias=_lib.ptr(dt_bias), q0=_lib.ptr(W0), anchor=_lib.ptr(anchor) if nc > 1 else None, first_step=_lib.ptr(first),
        ddt=_lib.ptr(ddt), dA_part=_lib.ptr(dA_p), dbias_part=_lib.ptr(db_p), batch=batch, seqlen=seqlen, heads=heads,
        chunk=Q, dt_dtype=_lib.dtype_enum(dt_raw.dtype), dt_softplus=int(bool(dt_softplus)),
        dt_min=lo if lo > -math.inf else -3.0e38, dt_max=hi if hi < math.inf else 3.0e38)
    _lib.call("ssm_ssd_bwd_dt", args, dev)
    return ddt, dA_p.sum(dim=(0, 1)), db_p.sum(dim=(0, 1))


def _scale_rows(x, w, out_dtype):
    """``ssm_ssd_scale_rows``: ``x * w[..., None]`` formed in float32 and rounded once to ``out_dtype``."""
    cols = int(x.shape[-1])
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    args = _lib.SsdScaleRowsArgs(x=_lib.ptr(x), w=_lib.ptr(w), out=_lib.ptr(out), rows=x.numel() // cols, cols=cols,
                                 x_dtype=_lib.dtype_enum(x.dtype), out_dtype=_lib.dtype_enum(out_dtype))
    _lib.call("ssm_ssd_scale_rows", args, x.device)
    return out


def _bwd_prep(dt, A, chunk_size, dt_bias, dt_softplus, dt_limit):
    """``ssm_ssd_bwd_prep``: ``(dA_cumsum, dt_out, dA_cumsum_rev)`` as ``(B, H, nc, Q)`` and ``(dt_rows, w_dy, w_x)``
    as ``(B, L, H)``, float32, for a sequence of whole chunks."""
    batch, seqlen, heads = (int(v) for v in dt.shape)
    Q = int(chunk_size)
    dev = dt.device
    dtc = K.cast_c(dt, dt.dtype)
    Af, bf = K.as_f32_vec(A), K.as_f32_vec(dt_bias)
    chunked = [torch.empty(batch, heads, seqlen // Q, Q, dtype=torch.float32, device=dev) for _ in range(3)]
    rows = [torch.empty(batch, seqlen, heads, dtype=torch.float32, device=dev) for _ in range(3)]
    lo, hi = float(dt_limit[0]), float(dt_limit[1])
    args = _lib.SsdBwdPrepArgs(
        dt=_lib.ptr(dtc), A=_lib.ptr(Af), dt_bias=_lib.ptr(bf), dA_cumsum=_lib.ptr(chunked[0]), dt_out=_lib.ptr(chunked[1]),
        dA_cumsum_rev=_lib.ptr(chunked[2]), dt_rows=_lib.ptr(rows[0]), w_dy=_lib.ptr(rows[1]), w_x=_lib.ptr(rows[2]),
        batch=batch, seqlen=seqlen, heads=heads, chunk=Q, dt_dtype=_lib.dtype_enum(dtc.dtype),
        dt_softplus=int(bool(dt_softplus)), dt_min=lo if lo > -math.inf else -3.0e38, dt_max=hi if hi < math.inf else 3.0e38)
    _lib.call("ssm_ssd_bwd_prep", args, dev)
    return (*chunked, *rows)


_ONES = {}


def _ones_like_cached(t):
    """A float32 tensor of ones with ``t``'s shape on its device, kept between calls (a read-only operand: the passes'
    step weights when the step is already in the operand)."""
    key = (tuple(t.shape), t.device)
    ones = _ONES.get(key)
    if ones is None:
        if len(_ONES) >= 8:
            _ONES.clear()
        ones = _ONES[key] = torch.ones(t.shape, dtype=torch.float32, device=t.device)
    return ones


def _bwd_states(ent_f, ent_r):
    """``ssm_ssd_bwd_states``: both stacks of chunk-boundary states as bfloat16 with chunks in time order, and the
    anchors ``<adjoint state, forward state>`` at the boundaries ``1..nc-1`` ``(B, nc-1, H)``."""
    batch, nc, heads, hdim, nstate = (int(v) for v in ent_f.shape)
    dev = ent_f.device
    f16 = torch.empty(ent_f.shape, dtype=torch.bfloat16, device=dev)
    r16 = torch.empty_like(f16)
    anchor = torch.empty(batch, max(nc - 1, 0), heads, dtype=torch.float32, device=dev)
    args = _lib.SsdBwdStatesArgs(entering_fwd=_lib.ptr(ent_f), entering_rev=_lib.ptr(ent_r), fwd_bf16=_lib.ptr(f16),
                                 rev_bf16=_lib.ptr(r16), anchor=_lib.ptr(anchor) if nc > 1 else None, batch=batch,
                                 nchunks=nc, heads=heads, dim=hdim * nstate)
    _lib.call("ssm_ssd_bwd_states", args, dev)
    return f16, r16, anchor


_BMM_F32_OUT = None       # whether this torch build's bmm forms float32 results from bfloat16 operands (probed once)


def _bmm_has_f32_out(device):
    global _BMM_F32_OUT
    if _BMM_F32_OUT is None:
        probe = torch.ones(1, 16, 16, dtype=torch.bfloat16, device=device)
        try:
            _BMM_F32_OUT = torch.bmm(probe, probe, out_dtype=torch.float32).dtype == torch.float32
        except (TypeError, RuntimeError, NotImplementedError):
            _BMM_F32_OUT = False
    return _BMM_F32_OUT


def _mm_f32(a, b):
    """Batched product of bfloat16 matrices with float32 accumulation and a float32 result.  Where the torch
    build has no ``out_dtype`` for ``bmm`` the operands are raised to float32 first, so the accuracy does not
    depend on the build; an error of the product itself (shapes, memory) surfaces as it is."""
    a3, b3 = a.reshape(-1, *a.shape[-2:]), b.reshape(-1, *b.shape[-2:])
    if _bmm_has_f32_out(a.device):
        out = torch.bmm(a3, b3, out_dtype=torch.float32)
    else:
        out = torch.bmm(a3.float(), b3.float())
    return out.view(*a.shape[:-1], b.shape[-1])


def _dB_dC_from_chunks(dyc, xc, Bc, Cc, dt_c, dA_cs, wdy, xw, f16, r16, groups):
    """``dB`` and ``dC`` ``(B, L, G, N)`` with the sum over a group's heads taken before the products with ``C`` and
    ``B`` (state-spaces/mamba ssd_combined.py, ``_chunk_scan_bwd_dcb`` / ``_chunk_state_bwd_db`` /
    ``_chunk_scan_bwd_dC``): inside a chunk both follow from one ``Q x Q`` matrix per group, ``dCB``; what crosses
    chunk boundaries is a product of the weighted ``x`` (``dy``) rows ``xw`` (``wdy``), all heads of the group side by
    side, with the adjoint (forward) states entering the chunk, ``r16`` (``f16``)."""
    batch, seqlen, heads, hdim = (int(v) for v in xc.shape)
    nc, Q = int(dA_cs.shape[2]), int(dA_cs.shape[3])
    nstate = int(Bc.shape[-1])
    per = heads // groups
    f32, bf = torch.float32, torch.bfloat16
    # the head-summed matrix is formed in float32 and rounded once: both products then run on the matrix cores with
    # float32 accumulation (a sum of Q terms whose roundings are independent)
    dCB = _bwd_dcb(dyc, xc, dt_c, dA_cs, groups).to(bf)                             # (B, nc, G, Q, Q)
    Bg = Bc.view(batch, nc, Q, groups, nstate).permute(0, 1, 3, 2, 4)               # (B, nc, G, Q, N)
    Cg = Cc.view(batch, nc, Q, groups, nstate).permute(0, 1, 3, 2, 4)
    dB = _mm_f32(dCB.transpose(-1, -2), Cg)
    dC = _mm_f32(dCB, Bg)

    def rows(t):           # (B, L, H, P) -> (B, nc, G, Q, per * P)
        return t.view(batch, nc, Q, groups, per * hdim).permute(0, 1, 3, 2, 4)

    def states(e):         # (B, nc, H, P, N) bf16, chunks in time order -> (B, nc, G, per * P, N)
        return e.view(batch, nc, groups, per * hdim, nstate)

    # dC_l += sum_{h,p} (exp(cs_l) dy_l)[h,p] H_in[h,p,:];  dB_s += sum_{h,p} (dt_s exp(cs'_s) x_s)[h,p] G_in[h,p,:]
    dC = dC + _mm_f32(rows(wdy), states(f16))
    dB = dB + _mm_f32(rows(xw), states(r16))
    back = lambda t: t.permute(0, 1, 3, 2, 4).reshape(batch, seqlen, groups, nstate)
    return back(dB), back(dC)


def ssd_combined_backward(dout, dfinal, x, dt, A, B, C, chunk_size, D=None, z=None, dt_bias=None,
                          initial_states=None, dt_softplus=False, dt_limit=(0.0, float("inf")), seq_idx=None,
                          grads_in_input_dtype=False):
    """Gradients of :func:`ssd_combined` (outputs ``y`` and ``final_states``).

    With ``a_t = exp(dt_t A)``, ``H_t = a_t H_{t-1} + dt_t x_t (x) B_t`` and the adjoint state
    ``G_t = dy_t (x) C_t + a_{t+1} G_{t+1}``, every contraction is again a chunked scan of the forward
    kind and runs through the same three kernels with the operands in other roles:

    * ``u_t = G_t B_t`` (then ``dx = dt u + D dy``): time reversed, ``x <- dy``, ``B <- C``, ``C <- B``;
    * ``dB_t = dt_t G_t^T x_t``: time reversed, ``x <- C``, ``B <- dy``, ``C <- x`` (state and channel
      axes trade places);
    * ``dC_t = H_t^T dy_t``: forward in time, ``x <- dt B``, ``B <- x``, ``C <- dy``;
    * ``y`` before skip and gate (for ``dz`` and the scalar below): the forward itself.

    The decay of the reversed passes is that of the following step (``a_{t+1}``).  The per-step
    scalar ``q_t = a_t <G_t, H_{t-1}>`` that ``ddt`` and ``dA`` need follows from
    ``<G_t, H_t> = <G_{t-1}, H_{t-1}> - <dy_{t-1}, H_{t-1} C_{t-1}> + dt_t <x_t, u_t>``, a running sum of
    quantities the passes have already produced.  The element-wise steps between the passes are
    fused kernels where the shape allows, tensor operations otherwise.

    Packed sequences (``seq_idx``) need no masks here: the first step of a sequence simply has decay zero
    (a jump of ``-64 ln 2`` in the running sums handed to the passes, forward and reversed), and every
    formula above holds for any decay.

    Args:
        dout: ``(B, L, H, P)`` gradient of ``y``.
        dfinal: ``(B, H, P, N)`` gradient of ``final_states`` or ``None``.
        (others): the arguments of the forward.

    Returns:
        ``(dx, ddt, dA, dB, dC, dD, dz, ddt_bias, dinitial_states)`` in float32 (``None`` for absent inputs); with
        ``grads_in_input_dtype`` the two large ones, ``dx`` and ``dz``, come back in ``x.dtype`` where the fused
        element-wise stages write them (one rounding, as a cast afterwards would give).
    """
    batch, seqlen, heads, hdim, groups, nstate = _ssd_shapes(x, B)
    Q = int(chunk_size)
    per = heads // groups
    f32 = torch.float32
    Af = A.detach().to(f32)
    fused = _elem_stages_ok(x, dout, z, hdim)
    # (dense, 16-byte aligned: a view that starts elsewhere in a larger buffer is copied once, here)
    xd, dod = K.cast_c(x, x.dtype), K.cast_c(dout, dout.dtype)
    zd = None if z is None else K.cast_c(z, z.dtype)
    B, C = K.cast_c(B, B.dtype), K.cast_c(C, C.dtype)
    xf = None if fused else xd.to(f32)
    dof = None if fused else dod.to(f32)
    # The passes take their operands in the inputs' precision when that is bfloat16 (matrix-core kernels,
    # float32 accumulation and states); everything between the passes is float32 either way.
    cd = torch.bfloat16 if (x.dtype == torch.bfloat16 and B.dtype == torch.bfloat16 and C.dtype == torch.bfloat16) else f32
    xc, Bc, Cc = (xd, B.detach(), C.detach()) if cd != f32 else (xd.to(f32), B.detach().to(f32), C.detach().to(f32))
    Df = None if D is None else D.detach().to(f32).contiguous()
    Dx = 0.0 if (Df is None or fused) else (Df[None, None, :, None] if Df.ndim == 1 else Df[None, None]) * xf
    init = None if initial_states is None else initial_states.detach().to(f32)
    dfin = None if dfinal is None else dfinal.detach().to(f32).contiguous()

    def blh(t_c):                         # (B, H, nc, Q) -> (B, L, H)
        return t_c.permute(0, 2, 3, 1).reshape(batch, -1, heads)[:, :seqlen]

    # everything that follows from the raw steps alone: one launch for whole chunks without packed sequences
    prepared = seq_idx is None and seqlen % Q == 0
    if prepared:
        dA_cs, dt_c, dA_r, dte, w_dy, w_x = _bwd_prep(dt.detach(), Af, Q, None if dt_bias is None else dt_bias.detach(),
                                                      dt_softplus, dt_limit)
    else:
        dA_cs, dt_c = chunk_cumsum(dt.detach(), Af, Q, dt_bias=None if dt_bias is None else dt_bias.detach(),
                                   dt_softplus=dt_softplus, dt_limit=dt_limit)
        dte = blh(dt_c)                                               # effective step
    # y before skip and gate.  The step enters through the operand (x~ = dt x, rounded once) rather than as a
    # weight inside the kernels: then this pass and the reversed one below multiply the same rounded
    # C.B-times-decay blocks, and the running sum that gives q (a difference of their row and column sums)
    # sees each product twice with the same value instead of collecting the two passes' rounding noise.
    if prepared:
        ones_c = _ones_like_cached(dt_c)
    else:
        _, ones_c = chunk_cumsum(torch.ones_like(dte), torch.zeros_like(Af), Q)
    bnd = None
    if seq_idx is not None:
        sid = seq_idx.to(torch.int64)
        bnd = sid != torch.cat([torch.zeros_like(sid[:, :1]), sid[:, :-1]], dim=1)      # (B, L): first steps

        def jumps(first_steps):               # (B, L) bool -> (B, 1, nc, Q) running sums of the jumps per chunk
            nc_ = dA_cs.shape[2]
            f = torch.nn.functional.pad(first_steps.to(f32), (0, nc_ * Q - seqlen))
            return (f.view(batch, nc_, Q).cumsum(-1) * (-64.0 * math.log(2.0)))[:, None]

        dA_cs = dA_cs + jumps(bnd)
    dte = dte.contiguous()
    if fused and cd == torch.bfloat16 and xd.dtype == cd and _row_scale_ok(xd, Bc, Cc, Q):
        # the kernels round dt x as they stage it: the same operand without a tensor of x's size written and read
        ypre, _, ent_f = _lin_pass(xd, ones_c, dA_cs, Bc, Cc, init, want_entering=True, x_scale=dt_c)
    else:
        xt = _scale_rows(xd, dte, cd) if (fused and cd in (torch.float32, torch.bfloat16)) else (dte[..., None] * xd).to(cd)
        ypre, _, ent_f = _lin_pass(xt, ones_c, dA_cs, Bc, Cc, init, want_entering=True)
    # decay of the reversed passes: a'_tau = a_{t+1} with t = L - 1 - tau; weights 1 on real steps
    if not prepared:
        dts = torch.cat([dte[:, 1:], torch.zeros_like(dte[:, :1])], dim=1).flip(1).contiguous()
        dA_r, _ = chunk_cumsum(dts, Af, Q, dt_limit=(-math.inf, math.inf))
    if bnd is not None:                       # the reversed passes decay by the following step's factor
        dA_r = dA_r + jumps(torch.cat([bnd[:, 1:], torch.zeros_like(bnd[:, :1])], dim=1).flip(1))
    # dB and dC with the sum over a group's heads taken first (two small products per chunk)?
    chunked = (fused and cd == torch.bfloat16 and hdim in (32, 64) and Q % 32 == 0 and seqlen % Q == 0
               and (hdim * nstate) % 4 == 0 and xc.is_contiguous() and Bc.is_contiguous() and Cc.is_contiguous())
    dD = None
    wdy = xw = None
    # the reversed pass reads dy in forward time where its matrix-core kernels run: no reversed copy is written
    rev_in_place = fused and chunked and xd.dtype == cd and _row_scale_ok(xd, Bc, Cc, Q)
    if fused and chunked:
        # the rows of the two products across chunk boundaries leave the gate kernel with their weights on:
        # dy_l exp(cs_l) for dC, x_s dt_s exp(cs'_s) for dB, cs' the running sum of the reversed pass at that step
        # (the decay from s to the end of its chunk and over the step that follows)
        if not prepared:
            w_dy = torch.exp(blh(dA_cs)).contiguous()
            w_x = (dte * torch.exp(blh(dA_r)).flip(1)).contiguous()
        dyc, dyr, dz, s2, dyx, wdy, xw = _bwd_gate(dod, zd, xd, ypre.contiguous(), Df, cd, want_rev=not rev_in_place,
                                                     w_dy=w_dy, w_x=w_x, grads_io=grads_in_input_dtype)
    elif fused:
        dyc, dyr, dz, s2, dyx = _bwd_gate(dod, zd, xd, ypre.contiguous(), Df, cd, grads_io=grads_in_input_dtype)
    if fused:
        if Df is not None and Df.ndim == 1:
            dD = dyx.sum(dim=(0, 1))
        elif Df is not None:
            gate = 1.0 if zd is None else torch.nn.functional.silu(zd.to(f32))
            dD = (dod.to(f32) * gate * xd.to(f32)).sum(dim=(0, 1))
    else:
        if z is not None:
            zf = zd.to(f32)
            sg = torch.sigmoid(zf)
            dy = dof * zf * sg
            dz = dof * (ypre + Dx) * (sg * (1.0 + zf * (1.0 - sg)))
        else:
            dy, dz = dof, None
        if Df is not None:
            dD = (dy * xf).sum(dim=(0, 1, 3)) if Df.ndim == 1 else (dy * xf).sum(dim=(0, 1))
    if not fused:
        dyc = dy.to(cd)
        dyr = dyc.flip(1).contiguous()
    # the reversed pass finishes dx itself where its matrix-core kernel runs: u never goes through memory
    dx_in_pass = (fused and cd == torch.bfloat16 and xd.dtype == cd and hdim in (32, 64) and _row_scale_ok(xd, Bc, Cc, Q))
    epilogue = (xd, dte, Df, xd.dtype if grads_in_input_dtype else f32, True) if dx_in_pass else None
    u_r, Gfin, ent_r = _lin_pass(dyc if rev_in_place else dyr, ones_c, dA_r, Cc.flip(1).contiguous(),
                                 Bc.flip(1).contiguous(), dfin, want_entering=True, dx_epilogue=epilogue,
                                 x_reversed=rev_in_place)
    dinit = None
    if init is not None:
        dinit = torch.exp(dte[:, 0] * Af[None])[:, :, None, None] * Gfin
        if bnd is not None:
            dinit = dinit * (~bnd[:, 0]).to(f32)[:, None, None, None]
    if dx_in_pass:
        dx, xu, s1 = u_r
    elif fused:
        dx, xu, s1 = _bwd_dx(dod, zd, xd, u_r.contiguous(), dte, Df, cd == torch.bfloat16,
                             grads_io=grads_in_input_dtype)
    else:
        u = u_r.flip(1)
        dx = dte[..., None] * u + (0.0 if Df is None else (Df[None, None, :, None] if Df.ndim == 1 else Df[None, None]) * dy)
    anchor_in = None
    if chunked:
        f16, r16, anchor_in = _bwd_states(ent_f.contiguous(), ent_r.contiguous())
        dB, dC = _dB_dC_from_chunks(dyc, xc, Bc, Cc, dt_c, dA_cs, wdy, xw, f16, r16, groups)
    else:
        Bh = Bc.repeat_interleave(per, dim=2) if per > 1 else Bc
        Ch = Cc.repeat_interleave(per, dim=2) if per > 1 else Cc
        v_r, _ = _lin_pass(Ch.flip(1).contiguous(), ones_c, dA_r, dyr, xc.flip(1).contiguous(),
                           None if dfin is None else dfin.transpose(2, 3).contiguous())
        if nstate % 4 == 0:
            dB = _bwd_db(v_r.contiguous(), dte, groups)
        else:
            dB = (dte[..., None] * v_r.flip(1)).view(batch, seqlen, groups, per, nstate).sum(3)
        dCh, _ = _lin_pass(Bh.contiguous(), dt_c, dA_cs, xc, dyc.contiguous(),
                           None if init is None else init.transpose(2, 3).contiguous())
        dC = dCh.view(batch, seqlen, groups, per, nstate).sum(3)
    if not fused:
        xu = (xf * u).sum(-1)                                             # (B, L, H)
        s1 = (xt.to(f32) * u).sum(-1)                  # with the rounded operand of the pass for y
        s2 = (dyc.to(f32) * ypre).sum(-1)              # the same rounded dy that the pass for u saw
    W0 = (dinit * init).sum(dim=(2, 3)) if init is not None else torch.zeros(batch, heads, dtype=f32, device=x.device)
    nc = (seqlen + Q - 1) // Q
    if anchor_in is not None and s1.is_contiguous() and s2.is_contiguous() and xu.is_contiguous():
        # the running sum behind ddt and dA, anchored at every chunk boundary on the two passes' float32 states
        # there (see below), the chain through softplus and clamp, and the sums for dA and the bias: one launch
        first = None if bnd is None else bnd.to(torch.uint8).contiguous()
        ddt, dA, dbias = _bwd_dt(s1, s2, xu, dte, dt.detach().contiguous(), Af.contiguous(),
                                 None if dt_bias is None else dt_bias.detach().to(f32).contiguous(),
                                 W0.contiguous() if init is not None else None, anchor_in, first, Q, dt_softplus, dt_limit)
        return dx, ddt, dA, dB, dC, dD, dz, (dbias if dt_bias is not None else None), (dinit if init is not None else None)
    if seqlen % Q == 0 and nc > 1:
        # q at the first step of every chunk straight from the two passes' states at the chunk boundary
        # (a_t <G_t, H_{t-1}>, float32), and from there the running sum inside the chunk only: what the
        # two passes round differently then adds up over one chunk instead of the whole sequence.
        a_first = torch.exp(dte[:, ::Q] * Af[None, None])                           # (B, nc, H)
        if bnd is not None:
            a_first = a_first * (~bnd[:, ::Q]).to(f32)[..., None]
        if anchor_in is not None:
            anchor = anchor_in                                                     # (B, nc-1, H): chunks 1..
        else:
            anchor = (ent_r.flip(1)[:, :-1] * ent_f[:, 1:]).sum(dim=(3, 4))
        anchor = torch.cat([W0[:, None], a_first[:, 1:] * anchor], dim=1)
        dq = (s1 - s2).view(batch, nc, Q, heads)
        q = (anchor[:, :, None] + dq.cumsum(2) - dq).reshape(batch, seqlen, heads)
    else:
        left = torch.cat([torch.zeros_like(s2[:, :1]), s2[:, :-1]], dim=1)
        q = W0[:, None] + (s1 - left).cumsum(1) - s1
    ddte = Af[None, None] * q + xu
    dA = (dte * q).sum(dim=(0, 1))
    raw = dt.detach().to(f32) + (0.0 if dt_bias is None else dt_bias.detach().to(f32)[None, None])
    v = torch.nn.functional.softplus(raw) if dt_softplus else raw
    lo, hi = float(dt_limit[0]), float(dt_limit[1])
    ddt = ddte * (torch.sigmoid(raw) if dt_softplus else 1.0) * ((v >= lo) & (v <= hi)).to(f32)
    dbias = ddt.sum(dim=(0, 1)) if dt_bias is not None else None
    return dx, ddt, dA, dB, dC, dD, dz, dbias, (dinit if init is not None else None)

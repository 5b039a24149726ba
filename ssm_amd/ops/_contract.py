"""Host-side argument contract shared by the operator façade.

The checks and their ``ValueError`` behaviour follow the reference's Python
path (src/ssm/ops/python/reference.py; each function cites its lines) so that
code written against ``ssm.ops`` sees the same failures here.  Nothing in this
module touches a device.
"""

from __future__ import annotations

from typing import Iterable, Optional

import torch

SUPPORTED = (torch.float32, torch.bfloat16, torch.float16, torch.float64)


class DeviceError(RuntimeError):
    """Inputs are not all on one ROCm device (this backend has no CPU path)."""


def on_gpu(t) -> bool:
    return t.is_cuda


def require_gpu(*tensors: Optional[torch.Tensor]) -> torch.device:
    """All tensor arguments must live on the same ``cuda`` (ROCm) device.

    The reference dispatches on the same predicate
    (src/ssm/ops/__init__.py:116-122) but falls back to Python loops otherwise;
    this backend refuses instead of silently computing on the CPU."""
    devs = {t.device for t in tensors if isinstance(t, torch.Tensor)}
    if not devs:
        raise DeviceError("no tensor arguments")
    if len(devs) != 1:
        raise DeviceError(f"tensors live on different devices: {sorted(map(str, devs))}")
    dev = next(iter(devs))
    if dev.type != "cuda":
        raise DeviceError(
            f"ssm_amd runs on ROCm devices only; got tensors on '{dev}'. "
            "There is deliberately no CPU fallback.")
    return dev


def check_float(name: str, t: torch.Tensor) -> None:
    if t.dtype not in SUPPORTED:
        raise ValueError(
            f"{name} has dtype {t.dtype}; the HIP backend supports float32, bfloat16, float16 "
            "(accumulated in float32) and float64 (computed in float64).")


def f64_compute(primary: torch.Tensor, A: Optional[torch.Tensor] = None) -> bool:
    """Whether the reference would compute this call in float64: the compute type is the primary tensor's
    (16-bit types widen to float32), promoted with ``A``'s when ``A`` is not float32
    (src/ssm/ops/python/reference.py:9-19, :135-137).  Complex tensors are not supported."""
    for t in (primary, A):
        if t is not None and t.is_complex():
            raise ValueError("complex tensors are not supported by the HIP backend.")
    ct = torch.float32 if primary.dtype in (torch.float16, torch.bfloat16) else primary.dtype
    if A is not None and A.dtype != torch.float32 and A.dtype != ct:
        ct = torch.promote_types(torch.float32 if A.dtype in (torch.float16, torch.bfloat16) else A.dtype, ct)
    return ct == torch.float64


def narrow(*tensors: Optional[torch.Tensor]):
    """Float64 tensors of a call that computes in float32 (the reference casts every operand to the compute
    type, reference.py:139-160), as float32."""
    return tuple(t.to(torch.float32) if (t is not None and t.dtype == torch.float64) else t for t in tensors)


def common_io_dtype(tensors: Iterable[Optional[torch.Tensor]]) -> torch.dtype:
    """Activation dtype the kernel reads: the shared dtype, or fp32 if mixed
    (widening is exact, so mixed inputs keep the reference's fp32 arithmetic)."""
    dts = {t.dtype for t in tensors if t is not None}
    return next(iter(dts)) if len(dts) == 1 else torch.float32


def as_f32_vec(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    if t is None:
        return None
    return t.detach().to(torch.float32).contiguous()


def cast_c(t: Optional[torch.Tensor], dt: torch.dtype) -> Optional[torch.Tensor]:
    """``t`` as the kernels take an input: detached, of type ``dt``, contiguous and starting on a 16-byte boundary
    (a contiguous view that starts elsewhere in a larger buffer is copied: the vector accesses of the fast kernels
    need the boundary, and a copy costs less than the element-wise kernels would)."""
    if t is None:
        return None
    t = t.detach()
    if t.dtype != dt:
        t = t.to(dt)
    if not t.is_contiguous():
        t = dense_copy(t)
    return t if t.data_ptr() % 16 == 0 else t.clone()


def dense_copy(t: torch.Tensor) -> torch.Tensor:
    """``t.contiguous()``.  A ``(B, C, L)``-shaped view on the GPU whose memory runs channels innermost -- the
    ``delta = F.linear(...).permute(0, 2, 1)`` and ``z = gate.permute(0, 2, 1)`` that the reference's block passes to
    the scan (src/ssm/modules/mamba1.py:223-228) -- goes through ``ssm_rows_to_bcl``, a tiled transposing copy
    (about 20 us for 8 x 1536 x 2048 bfloat16 where torch's strided copy takes 106)."""
    if t.ndim == 3 and t.is_cuda and t.element_size() in (2, 4) and not t.is_complex():
        batch, chans, length = t.shape
        sb, sc, sl = t.stride()
        if (sc == 1 and length > 1 and chans % 4 == 0 and sl >= chans and sl % 4 == 0 and sb % 4 == 0
                and (batch == 1 or sb >= (length - 1) * sl + chans) and t.data_ptr() % (4 * t.element_size()) == 0):
            from .. import _lib
            out = torch.empty(t.shape, dtype=t.dtype, device=t.device)
            args = _lib.RowsToBclArgs(src=_lib.ptr(t), dst=_lib.ptr(out), src_batch_stride=int(sb),
                                      src_row_stride=int(sl), batch=int(batch), channels=int(chans),
                                      seqlen=int(length), element_size=t.element_size())
            _lib.call("ssm_rows_to_bcl", args, t.device)
            return out
    return t.contiguous()


# ----------------------------------------------------------- selective scan

def scan_projection_kind(name: str, p: torch.Tensor, batch: int, dim: int, nstate: int,
                         length: int) -> tuple[int, int]:
    """-> (kind, groups) for a B/C argument (reference.py:22-56)."""
    from .._lib import PROJ_BDN, PROJ_BGNL, PROJ_DN

    if p.dim() == 2:
        if tuple(p.shape) != (dim, nstate):
            raise ValueError(f"{name} must have shape (D, N).")
        return PROJ_DN, 1
    if p.dim() == 3:
        if tuple(p.shape) != (batch, dim, nstate):
            raise ValueError(f"{name} must have shape (B, D, N) when 3-D.")
        return PROJ_BDN, 1
    if p.dim() == 4:
        if p.shape[0] != batch or p.shape[-1] != length:
            raise ValueError(f"{name} must have shape (B, G, N, L) when 4-D.")
        groups = int(p.shape[1])
        if groups == 0 or dim % groups != 0:
            raise ValueError("Group dimension must divide D.")
        if p.shape[2] != nstate:
            raise ValueError(f"{name} has mismatched state dimension.")
        return PROJ_BGNL, groups
    raise ValueError(f"Unsupported rank for {name}.")


def check_selective_scan(u, delta, A, B, C, D, z, dt_bias):
    """Shape contract of ``selective_scan`` (reference.py:124-165)."""
    if u.ndim != 3 or delta.ndim != 3:
        raise ValueError("u and delta must have shape (B, D, L).")
    batch, dim, length = (int(s) for s in u.shape)
    if tuple(delta.shape) != (batch, dim, length):
        raise ValueError("delta must match the shape of u.")
    if A.ndim < 1:
        raise ValueError("A must have shape (D, N).")
    nstate = int(A.shape[-1])
    if tuple(A.shape) != (dim, nstate):
        raise ValueError("A must have shape (D, N).")
    bk = scan_projection_kind("B", B, batch, dim, nstate, length)
    ck = scan_projection_kind("C", C, batch, dim, nstate, length)
    if D is not None and tuple(D.shape) != (dim,):
        raise ValueError("D must have shape (D,).")
    if z is not None and tuple(z.shape) != (batch, dim, length):
        raise ValueError("z must have shape (B, D, L).")
    if dt_bias is not None and tuple(dt_bias.shape) != (dim,):
        raise ValueError("dt_bias must have shape (D,).")
    for name, t in (("u", u), ("delta", delta), ("A", A), ("B", B), ("C", C), ("D", D), ("z", z),
                    ("dt_bias", dt_bias)):
        if t is not None:
            check_float(name, t)
    if batch == 0 or dim == 0 or length == 0 or nstate == 0:
        raise ValueError("selective_scan needs non-empty B, D, L and N.")
    return batch, dim, length, nstate, bk, ck


# ------------------------------------------------------ selective state step

def step_projection_kind(name: str, p: torch.Tensor, batch: int, dim: int, nstate: int) -> tuple[int, int]:
    """-> (kind, groups).  A 3-D tensor whose second axis is not ``D`` is the
    grouped ``(B, G, N)`` form (reference.py:252-272)."""
    from .._lib import PROJ_BDN, PROJ_BGNL, PROJ_DN

    if p.dim() == 3 and p.shape[0] == batch and p.shape[1] != dim:
        groups = int(p.shape[1])
        if groups == 0 or dim % groups != 0:
            raise ValueError(f"{name} group dimension must divide D.")
        if p.shape[2] != nstate:
            raise ValueError(f"{name} must have matching state dimension.")
        return PROJ_BGNL, groups
    if p.dim() == 2:
        if tuple(p.shape) != (dim, nstate):
            raise ValueError(f"{name} must have shape (D, N).")
        return PROJ_DN, 1
    if p.dim() == 3:
        if tuple(p.shape) != (batch, dim, nstate):
            raise ValueError(f"{name} must have shape (B, D, N) when 3-D.")
        return PROJ_BDN, 1
    if p.dim() == 4:
        # the reference broadcasts through its scan helper with L == 1
        if p.shape[0] != batch or p.shape[-1] != 1:
            raise ValueError(f"{name} must have shape (B, G, N, L) when 4-D.")
        groups = int(p.shape[1])
        if groups == 0 or dim % groups != 0:
            raise ValueError("Group dimension must divide D.")
        if p.shape[2] != nstate:
            raise ValueError(f"{name} has mismatched state dimension.")
        return PROJ_BGNL, groups
    raise ValueError(f"Unsupported rank for {name}.")


def check_state_step(state, x, dt, A, B, C, D, z, dt_bias):
    """Shape contract of ``selective_state_step`` (reference.py:231-291)."""
    if state.ndim != 3:
        raise ValueError("state must have shape (B, D, N).")
    if x.ndim != 2 or dt.ndim != 2:
        raise ValueError("x and dt must have shape (B, D).")
    batch, dim, nstate = (int(s) for s in state.shape)
    if tuple(x.shape) != (batch, dim) or tuple(dt.shape) != (batch, dim):
        raise ValueError("x and dt must match the first two dimensions of state.")
    if tuple(A.shape) != (dim, nstate):
        raise ValueError("A must have shape (D, N).")
    bk = step_projection_kind("B", B, batch, dim, nstate)
    ck = step_projection_kind("C", C, batch, dim, nstate)
    if D is not None and tuple(D.shape) != (dim,):
        raise ValueError("D must have shape (D,).")
    if z is not None and tuple(z.shape) != (batch, dim):
        raise ValueError("z must have shape (B, D).")
    if dt_bias is not None and tuple(dt_bias.shape) != (dim,):
        raise ValueError("dt_bias must have shape (D,).")
    for name, t in (("state", state), ("x", x), ("dt", dt), ("A", A), ("B", B), ("C", C), ("D", D),
                    ("z", z), ("dt_bias", dt_bias)):
        if t is not None:
            check_float(name, t)
    if batch == 0 or dim == 0 or nstate == 0:
        raise ValueError("selective_state_step needs non-empty B, D and N.")
    return batch, dim, nstate, bk, ck


# ------------------------------------------------------------ depthwise conv

def check_conv(x, weight, bias, activation, channels_last=None):
    """Layout detection and shape contract of ``dw_causal_conv``
    (reference.py:483-533): channels-first is tested first.  ``channels_last`` (not in the
    reference) names the layout instead, for callers whose sequence length may equal the
    channel count."""
    if x.ndim != 3:
        raise ValueError("x must have shape (B, C, L) or (B, L, C).")
    chans = int(weight.shape[0]) if weight.ndim >= 1 else -1
    if channels_last is not None:
        channels_first = not channels_last
        if x.shape[1 if channels_first else 2] != chans:
            raise ValueError("weight channel dimension must match x in the layout named.")
    elif x.shape[1] == chans:
        channels_first = True
    elif x.shape[2] == chans:
        channels_first = False
    else:
        raise ValueError("weight channel dimension must match x.")
    if weight.ndim == 2:
        width = int(weight.shape[1])
    elif weight.ndim == 3:
        if weight.shape[1] != 1:
            raise ValueError("Expected depthwise weights with shape (C, 1, K).")
        width = int(weight.shape[2])
    else:
        raise ValueError("weight must have 2 or 3 dimensions.")
    if bias is not None and tuple(bias.shape) != (chans,):
        raise ValueError("bias must have shape (C,).")
    act = str(activation).lower()
    if act in ("silu", "swish"):
        silu = True
    elif act in ("identity", "none"):
        silu = False
    else:
        raise ValueError(f"Unsupported activation '{activation}'.")
    for name, t in (("x", x), ("weight", weight), ("bias", bias)):
        if t is not None:
            check_float(name, t)
    if channels_first:
        batch, _, length = (int(s) for s in x.shape)
    else:
        batch, length, _ = (int(s) for s in x.shape)
    if batch == 0 or chans == 0 or length == 0 or width == 0:
        raise ValueError("dw_causal_conv needs non-empty B, C, L and K.")
    return batch, chans, length, width, channels_first, silu


# ----------------------------------------------------------------- layer norm

def check_norm(x, weight, bias, residual):
    """Shape contract of ``fused_layer_norm`` (reference.py:565-572)."""
    if x.ndim != 3:
        raise ValueError("x must have shape (B, L, D).")
    hidden = int(x.shape[-1])
    if tuple(weight.shape) != (hidden,):
        raise ValueError("weight must match the last dimension of x.")
    if bias is not None and tuple(bias.shape) != (hidden,):
        raise ValueError("bias must match the last dimension of x.")
    if residual is not None and tuple(residual.shape) != tuple(x.shape):
        raise ValueError("residual must match the shape of x.")
    for name, t in (("x", x), ("weight", weight), ("bias", bias), ("residual", residual)):
        if t is not None:
            check_float(name, t)
    rows = int(x.shape[0]) * int(x.shape[1])
    if rows == 0 or hidden == 0:
        raise ValueError("fused_layer_norm needs a non-empty input.")
    return rows, hidden


# -------------------------------------------- diagonal chunk scan (ssd_chunk_scan)

def chunk_projection_kind(name, p, batch, seqlen, heads, proj) -> int:
    """-> kind of a B/C argument of ``ssd_chunk_scan`` (reference.py:59-84)."""
    from .._lib import CHUNK_BHP, CHUNK_BLHP, CHUNK_HP

    if p.dim() == 2:
        if tuple(p.shape) != (heads, proj):
            raise ValueError(f"{name} must have shape (H, P).")
        return CHUNK_HP
    if p.dim() == 3:
        if tuple(p.shape) != (batch, heads, proj):
            raise ValueError(f"{name} must be (B, H, P) when 3-D.")
        return CHUNK_BHP
    if p.dim() == 4:
        if tuple(p.shape) != (batch, seqlen, heads, proj):
            raise ValueError(f"{name} must have shape (B, L, H, P) when 4-D.")
        return CHUNK_BLHP
    raise ValueError(f"Unsupported rank for {name}.")


def check_chunk_scan(X, dt, A, B, C, chunk_size, D, z, initial_states):
    """Shape contract of ``ssd_chunk_scan`` (reference.py:346-411)."""
    if X.ndim != 4:
        raise ValueError("X must have shape (B, L, H, P).")
    if dt.ndim != 3:
        raise ValueError("dt must have shape (B, L, H).")
    batch, seqlen, heads, proj = (int(s) for s in X.shape)
    if tuple(dt.shape) != (batch, seqlen, heads):
        raise ValueError("dt must align with (B, L, H).")
    if A.ndim == 1:
        if A.shape[0] != heads:
            raise ValueError("A must have shape (H,) when 1-D.")
        a_per_p = False
    elif A.ndim == 2:
        if tuple(A.shape) != (heads, proj):
            raise ValueError("A must have shape (H, P) when 2-D.")
        a_per_p = True
    else:
        raise ValueError("A must be 1-D or 2-D.")
    bk = chunk_projection_kind("B", B, batch, seqlen, heads, proj)
    ck = chunk_projection_kind("C", C, batch, seqlen, heads, proj)
    d_per_p = False
    if D is not None:
        if D.ndim == 1:
            if D.shape[0] != heads:
                raise ValueError("D must have shape (H,).")
        elif D.ndim == 2:
            if tuple(D.shape) != (heads, proj):
                raise ValueError("D must have shape (H, P) when 2-D.")
            d_per_p = True
        else:
            raise ValueError("Unsupported rank for D.")
    z_per_p = False
    if z is not None:
        if z.ndim == 3:
            if tuple(z.shape) != (batch, seqlen, heads):
                raise ValueError("z must have shape (B, L, H) when 3-D.")
        elif z.ndim == 4:
            if tuple(z.shape) != (batch, seqlen, heads, proj):
                raise ValueError("z must have shape (B, L, H, P) when 4-D.")
            z_per_p = True
        else:
            raise ValueError("Unsupported rank for z.")
    if initial_states is not None and tuple(initial_states.shape) != (batch, heads, proj):
        raise ValueError("initial_states must have shape (B, H, P).")
    if int(chunk_size) <= 0:
        raise ValueError("chunk_size must be positive.")
    for name, t in (("X", X), ("dt", dt), ("A", A), ("B", B), ("C", C), ("D", D), ("z", z),
                    ("initial_states", initial_states)):
        if t is not None:
            check_float(name, t)
    if batch == 0 or seqlen == 0 or heads == 0 or proj == 0:
        raise ValueError("ssd_chunk_scan needs non-empty B, L, H and P.")
    return batch, seqlen, heads, proj, a_per_p, bk, ck, d_per_p, z_per_p


def sequence_lengths(seq_meta, batch: int, device) -> Optional[torch.Tensor]:
    """``seq_meta`` -> int32 device tensor of valid lengths, or ``None``.
    ``cu_seqlens`` (B+1) wins over ``seq_lens`` (B) (reference.py:413-428;
    list/tensor handling as src/ssm/ops/__init__.py:1460-1481).  No host sync."""
    if not seq_meta:
        return None
    if seq_meta.get("cu_seqlens") is not None:
        cu = torch.as_tensor(seq_meta["cu_seqlens"]).to(device=device, dtype=torch.long).flatten()
        if cu.numel() != batch + 1:
            raise ValueError("cu_seqlens must have length B + 1.")
        return (cu[1:] - cu[:-1]).to(torch.int32).contiguous()
    if seq_meta.get("seq_lens") is not None:
        sl = torch.as_tensor(seq_meta["seq_lens"]).to(device=device, dtype=torch.int32).flatten()
        if sl.numel() != batch:
            raise ValueError("seq_lens must have length B.")
        return sl.contiguous()
    raise ValueError("seq_meta must provide cu_seqlens or seq_lens.")

"""Inputs that are contiguous views starting at an odd offset inside a larger buffer (a parameter cut out of a flat
parameter vector, an activation cut out of a workspace): every operator, forward and backward, gives what it
gives for the same values in a buffer of their own.  Found the hard way: the one-pass SSD entry refused a per-head
skip vector at a 4-byte offset, and its backward sent a misaligned ``x`` to a kernel that does not take it."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ops():
    from ssm_amd import ops
    return ops


def own(t):
    return t.cuda()


def view(t, off=1):
    """The same values ``off`` elements into a larger buffer: 2 or 4 bytes off the 16-byte grid."""
    t = t.cuda()
    buf = torch.zeros(t.numel() + off, device="cuda", dtype=t.dtype)
    buf[off:] = t.reshape(-1)
    v = buf[off:].view(t.shape)
    assert v.data_ptr() % 16 != 0 and v.is_contiguous()
    return v


def same(a, b, dtype, what):
    # mostly the same bits; where a view takes another kernel than the aligned tensor (the state step's variants),
    # the same values to the last bits of the arithmetic
    bar = 2e-5 if dtype == torch.float32 else 1e-2
    for i, (x, y) in enumerate(zip(a, b)):
        assert x.shape == y.shape and x.dtype == y.dtype, f"{what}[{i}]"
        rms = float(y.double().pow(2).mean().sqrt()) + 1e-30
        err = float((x.double() - y.double()).abs().max())
        assert err <= bar * rms, f"{what}[{i}]: max err / rms {err / rms:.3e}"


def grads_of(fn, tensors, mk):
    lv = [None if t is None else mk(t).detach().requires_grad_() for t in tensors]
    out = fn(*lv)
    out = out if isinstance(out, tuple) else (out,)
    sum(o.float().square().sum() for o in out).backward()
    return [o.detach() for o in out] + [t.grad for t in lv if t is not None]


DTYPES = [torch.float32, torch.bfloat16]


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "bfloat16"])
def test_selective_scan_and_state_step(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(0)
    B, D, L, N = 2, 48, 512, 16
    u, dl, z = (torch.randn(B, D, L, generator=g).to(dtype) for _ in range(3))
    A, Dk, bias = -(torch.rand(D, N, generator=g) + 0.5), torch.randn(D, generator=g), torch.randn(D, generator=g)
    Bm, Cm = (torch.randn(B, 1, N, L, generator=g).to(dtype) for _ in range(2))
    fn = lambda u, dl, A, Bm, Cm, Dk, z, bias: ops.selective_scan(u, dl, A, Bm, Cm, D=Dk, z=z, dt_bias=bias, softplus=True,
                                                                 return_last_state=True)
    ts = (u, dl, A, Bm, Cm, Dk, z, bias)
    with torch.no_grad():
        for _ in range(2):          # the second call of a form goes through the remembered argument struct
            same(fn(*map(view, ts)), fn(*map(own, ts)), dtype, "scan")
    same(grads_of(fn, ts, view), grads_of(fn, ts, own), dtype, "scan with gradients")
    st = torch.randn(B, D, N, generator=g)
    x1, dt1, z1 = (torch.randn(B, D, generator=g).to(dtype) for _ in range(3))
    B1, C1 = (torch.randn(B, 1, N, generator=g).to(dtype) for _ in range(2))

    def step(mk):
        s = st.clone().cuda()
        y = ops.selective_state_step(s, mk(x1), mk(dt1), mk(A), mk(B1), mk(C1), D=mk(Dk), z=mk(z1), dt_bias=mk(bias))
        return y, s
    same(step(view), step(own), dtype, "state step")


@pytest.mark.parametrize("dtype", DTYPES, ids=["float32", "bfloat16"])
def test_diagonal_chunk_scan_conv_and_norm(dtype):
    ops = _ops()
    g = torch.Generator().manual_seed(1)
    B, L, H, P = 2, 512, 3, 64
    X, Bq, Cq, zq = (torch.randn(B, L, H, P, generator=g).to(dtype) for _ in range(4))
    dtq, Ah, Dh = torch.rand(B, L, H, generator=g) * 0.1, -(torch.rand(H, generator=g) + 0.5), torch.randn(H, generator=g)
    fn = lambda X, dtq, Ah, Bq, Cq, Dh, zq: ops.ssd_chunk_scan(X, dtq, Ah, Bq, Cq, 64, D=Dh, z=zq)
    same(grads_of(fn, (X, dtq, Ah, Bq, Cq, Dh, zq), view), grads_of(fn, (X, dtq, Ah, Bq, Cq, Dh, zq), own), dtype, "chunk scan")
    xc, w, cb = torch.randn(B, 48, L, generator=g).to(dtype), torch.randn(48, 4, generator=g), torch.randn(48, generator=g)
    same(grads_of(ops.dw_causal_conv, (xc, w, cb), view), grads_of(ops.dw_causal_conv, (xc, w, cb), own), dtype, "conv")
    xl = xc.transpose(1, 2).contiguous()
    same(grads_of(ops.dw_causal_conv_channels_last, (xl, w, cb), view),
         grads_of(ops.dw_causal_conv_channels_last, (xl, w, cb), own), dtype, "conv, channels last")
    xn, rn = (torch.randn(4, 33, 768, generator=g).to(dtype) for _ in range(2))
    wn, bn = torch.randn(768, generator=g), torch.randn(768, generator=g)
    for rms in (False, True):
        fn = lambda x, w, b, r: ops.fused_layer_norm_with_residual(x, w, b, residual=r, is_rms=rms)
        same(grads_of(fn, (xn, wn, bn, rn), view), grads_of(fn, (xn, wn, bn, rn), own), dtype, f"norm rms={rms}")


@pytest.mark.parametrize("fused", [True, False], ids=["one-pass", "five-kernels"])
def test_ssd_combined(fused):
    from ssm_amd.ops import ssd
    g = torch.Generator().manual_seed(2)
    H, P, N, Q, dtype = 2, 64, 64, 128, torch.bfloat16
    xs, zs = (torch.randn(1, 256, H, P, generator=g).to(dtype) for _ in range(2))
    Bs, Cs = (torch.randn(1, 256, 1, N, generator=g).to(dtype) for _ in range(2))
    dts, As = torch.rand(1, 256, H, generator=g) * 0.1, -(torch.rand(H, generator=g) + 0.5)
    Ds, bs = torch.randn(H, generator=g), torch.randn(H, generator=g)
    fn = lambda x, dt, A, B, C, D, z, b: ssd.ssd_combined(x, dt, A, B, C, Q, D=D, z=z, dt_bias=b, dt_softplus=True, fused=fused)
    ts = (xs, dts, As, Bs, Cs, Ds, zs, bs)
    same(grads_of(fn, ts, view), grads_of(fn, ts, own), dtype, "ssd_combined")


# ------------------------------------------------------------- (B, C, L) views of memory that runs channels innermost

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32, torch.int32, torch.int16])
@pytest.mark.parametrize("shape", [(2, 11, 8, 8, 0), (1, 300, 64, 128, 64), (3, 1000, 12, 40, 4), (2, 130, 68, 68, 0),
                                   (2, 257, 132, 264, 132), (2, 64, 6, 6, 0), (2, 129, 8, 16, 2), (8, 2048, 1536, 3072, 1536)],
                         ids=lambda s: "B{}L{}C{}of{}at{}".format(*s))
def test_dense_copy_of_a_view_of_rows(dtype, shape):
    """``dense_copy`` equals ``contiguous()`` bit for bit on every view: the tiled copy takes the ones whose channel
    count, strides and start are multiples of 4 elements, torch the others (6 channels; a start 2 elements in)."""
    from ssm_amd.ops import _contract as K
    batch, length, chans, wide, offset = shape
    g = torch.Generator(device="cuda").manual_seed(length)
    rows = torch.randint(-30000, 30000, (batch, length, wide), device="cuda", generator=g).to(dtype)
    v = rows[:, :, offset:offset + chans].permute(0, 2, 1)
    out = K.dense_copy(v)
    assert out.is_contiguous() and out.shape == v.shape and out.dtype == v.dtype
    assert torch.equal(out, v.contiguous())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_scan_on_permuted_views_equals_the_scan_on_dense_copies(dtype):
    """What the reference's block passes (src/ssm/modules/mamba1.py:223-247): ``delta`` and ``z`` as permuted views of
    (B, L, D) projections, ``z`` one half of a wider one.  Forward and backward equal the call on dense copies."""
    from tests.test_scan_fwd_gpu import make_inputs
    ops = _ops()
    batch, dim, length, nstate = 2, 48, 520, 16
    inp = {k: v.cuda() for k, v in make_inputs(5, batch, dim, length, nstate, dtype=dtype).items()}
    g = torch.Generator(device="cuda").manual_seed(2)
    delta_rows = torch.randn(batch, length, dim, device="cuda", generator=g).to(dtype)
    xz = torch.randn(batch, length, 2 * dim, device="cuda", generator=g).to(dtype)
    go = torch.randn(batch, dim, length, device="cuda", generator=g).to(dtype)
    res = []
    for dense in (False, True):
        d_leaf, z_leaf = delta_rows.clone().requires_grad_(), xz.clone().requires_grad_()
        delta, z = d_leaf.permute(0, 2, 1), z_leaf.chunk(2, dim=-1)[1].permute(0, 2, 1)
        if dense:
            delta, z = delta.contiguous(), z.contiguous()
        else:
            assert not delta.is_contiguous() and not z.is_contiguous()
        u = inp["u"].clone().requires_grad_()
        y = ops.selective_scan(u, delta, inp["A"], inp["B"], inp["C"], D=inp["D"], z=z, dt_bias=inp["dt_bias"], softplus=True)
        y.backward(go)
        res.append((y.detach(), u.grad, d_leaf.grad, z_leaf.grad))
    for a, b in zip(*res):
        assert torch.equal(a, b)

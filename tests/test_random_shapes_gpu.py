"""Seeded sweeps over shapes, element types and optional arguments that the other files do not list one by
one: every operator's values and gradients against the CPU oracle evaluated in float64.

Each case draws its shape and options from ``random.Random(seed)`` and its data from a torch generator, so a
failure names a case that can be rebuilt from the seed alone.  Bars (``_close``): every element within a relative
bound of itself plus a fraction of the root mean square of the expected tensor -- float32 tensors 1e-5 (values) /
1e-4 + 1e-5 (gradients), with the float32 oracle arbitrating elements beyond that (the kernel may be at most four
times as far from the float64 value as the float32 oracle is at its worst); 16-bit tensors 2e-2 + 4e-2 of the
rms (values) / 3e-2 + 6e-2 (gradients) and a mean error of at most 5e-3 / 1e-2 of the rms -- the float64 oracle
does not round its result to the element type, so a 16-bit output carries its own last-place rounding on top
of the accumulated error.  For the SSD the two gradients that are sums over the whole sequence with cancelling
terms (``dA``, the bias of the step) are measured against the sum of the magnitudes of their terms."""

import random

import pytest
import torch

from oracle import ops_oracle as O
from oracle import ssd_oracle as SO

pytestmark = pytest.mark.gpu

HALF = (torch.bfloat16, torch.float16)
CASES_PER_BLOCK = 12


def _ops():
    from ssm_amd import ops
    return ops


def _close(a, r64, what, half=False, grad=False, r32=None, rtol=None, atol_rms=None, mean_rms=None):
    """``a`` (from the GPU) against the float64 oracle's ``r64``, element by element: within ``rtol`` of the element
    itself plus ``atol_rms`` of the root mean square of the expected tensor (not of its largest element).
    16-bit calls (``half``): one rounding of the result plus the float32 arithmetic behind it, with a bound on
    the mean error an order of magnitude lower.  float32 calls: 1e-5 for values and 1e-4 for gradients; an element
    outside that still passes when the float32 oracle ``r32`` is itself that far from the float64 value somewhere
    (at most four times its largest error): two float32 sums of the same terms in different orders."""
    a = a.detach().double().cpu()
    r = r64.detach().double().cpu()
    assert a.shape == r.shape, (what, tuple(a.shape), tuple(r.shape))
    assert torch.isfinite(a).all(), what
    if r.numel() == 0:
        return
    rms = float(r.pow(2).mean().sqrt()) + 1e-30
    err = (a - r).abs()
    if half:
        rt, at, mt = (3e-2, 6e-2, 1e-2) if grad else (2e-2, 4e-2, 5e-3)
    else:
        rt, at, mt = (1e-4, 1e-5, None) if grad else (1e-5, 1e-5, None)
    rt = rt if rtol is None else rtol
    at = at if atol_rms is None else atol_rms
    mt = mt if mean_rms is None else mean_rms
    bar = rt * r.abs() + at * rms
    if r32 is not None:
        bar = torch.clamp(bar, min=4.0 * float((r32.detach().double().cpu() - r).abs().max()))
    worst = float((err / (bar + 1e-300)).max())
    assert worst <= 1.0, (what, "max err / rms %.3e" % (float(err.max()) / rms), "err / bar %.2f" % worst)
    if mt is not None:
        assert float(err.mean()) <= mt * rms, (what, "mean err / rms %.3e" % (float(err.mean()) / rms))


def _leaf(t, grad=True):
    if t is None:
        return None, None
    return (t.cuda().detach().requires_grad_(grad), t.double().detach().requires_grad_(grad))


def _values_and_gradients(fn_dev, fn_ref, ins, desc, half):
    """``fn_ref(acc, *tensors)`` is the oracle: float64 arithmetic with ``acc=torch.float64``, the reference's own
    float32 with ``acc=None`` (run for float32 calls only, to arbitrate)."""
    devs, refs = zip(*[_leaf(t) for t in ins])
    out_d, out_r = fn_dev(*devs), fn_ref(torch.float64, *refs)
    refs32 = out_32 = None
    if not half:
        refs32 = [None if t is None else t.detach().clone().requires_grad_(True) for t in ins]
        out_32 = fn_ref(None, *refs32)
    if not isinstance(out_d, tuple):
        out_d, out_r = (out_d,), (out_r,)
        out_32 = None if out_32 is None else (out_32,)
    for i, (a, r) in enumerate(zip(out_d, out_r)):
        _close(a, r, (desc, "output", i), half=half, r32=None if out_32 is None else out_32[i])
    g = torch.Generator().manual_seed(7)
    loss_d = loss_r = loss_32 = 0
    for i, (a, r) in enumerate(zip(out_d, out_r)):
        w = torch.randn(r.shape, generator=g, dtype=torch.float64).to(a.dtype).double()
        loss_d = loss_d + (a.double() * w.cuda()).sum()
        loss_r = loss_r + (r * w).sum()
        if out_32 is not None:
            loss_32 = loss_32 + (out_32[i] * w.float()).sum()
    loss_d.backward()
    loss_r.backward()
    if out_32 is not None:
        loss_32.backward()
    for i, (d, r) in enumerate(zip(devs, refs)):
        if d is None:
            continue
        assert d.grad is not None and r.grad is not None, (desc, "gradient", i)
        _close(d.grad, r.grad, (desc, "gradient", i), half=half, grad=True,
               r32=None if refs32 is None else refs32[i].grad)


def _scan_case(rng, seed):
    g = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    b, n = rng.randint(1, 3), rng.choice([1, 3, 8, 16, 16, 16, 24, 32])
    l = rng.choice([rng.randint(1, 40), 16 * rng.randint(1, 40), rng.randint(1, 700)])
    kind = rng.choice(["grouped", "grouped", "dn", "bdn", "perchan"])
    groups = rng.choice([1, 2, 3])
    d = groups * rng.choice([8, 16, 24, 48, 5])
    u = torch.randn(b, d, l, generator=g).to(dtype)
    delta = torch.randn(b, d, l, generator=g).to(dtype)
    A = -(torch.rand(d, n, generator=g) * 3 + 0.1)
    shape = {"grouped": (b, groups, n, l), "perchan": (b, d, n, l), "dn": (d, n), "bdn": (b, d, n)}[kind]
    pt = dtype if len(shape) == 4 else torch.float32
    Bm, Cm = torch.randn(*shape, generator=g).to(pt), torch.randn(*shape, generator=g).to(pt)
    D = torch.randn(d, generator=g) if rng.random() < 0.6 else None
    z = torch.randn(b, d, l, generator=g).to(dtype) if rng.random() < 0.6 else None
    bias = torch.randn(d, generator=g) * 0.5 if rng.random() < 0.6 else None
    sp = rng.random() < 0.7
    if not sp:                              # a raw step must be positive, or the state grows without bound
        delta, bias = delta.abs() * 0.3, None
    half = dtype in HALF
    desc = ("scan", seed, (b, d, l, n), kind, groups, str(dtype), D is not None, z is not None, bias is not None, sp)
    # a draw of its own (the cases above stay what they were): u, delta, z as the reference's block passes the last
    # two, (B, D, L)-shaped views of (B, L, D') rows (src/ssm/modules/mamba1.py:223-228)
    own = random.Random(seed ^ 0x6C1D)
    turned = [name for name in ("u", "delta", "z") if own.random() < 0.25]
    if turned:
        desc = desc + ("views of rows", tuple(turned))

    def as_given(name, t):
        """The leaf to differentiate and the view of it that the operator gets."""
        if t is None or name not in turned:
            return t, (lambda leaf: leaf)
        pad = own.choice([0, 0, 4, d])
        rows = torch.zeros(b, l, d + pad).to(t.dtype)
        rows[:, :, :d] = t.transpose(1, 2)
        return rows, (lambda leaf: leaf[:, :, :d].permute(0, 2, 1))

    (u, vu), (delta, vd), (z, vz) = as_given("u", u), as_given("delta", delta), as_given("z", z)
    look = lambda a: (vu(a[0]), vd(a[1]), *a[2:6], None if a[6] is None else vz(a[6]), a[7])
    _values_and_gradients(lambda *a: _ops().selective_scan(*look(a), softplus=sp, return_last_state=True),
                          lambda acc, *a: O.selective_scan(*look(a), softplus=sp, return_last_state=True, acc=acc),
                          [u, delta, A, Bm, Cm, D, z, bias], desc, half)


def _step_case(rng, seed):
    g = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    b, d, n = rng.randint(1, 9), rng.choice([4, 16, 40, 64, 100, 256]), rng.choice([1, 4, 16, 16, 32, 64, 128, 5])
    state = torch.randn(b, d, n, generator=g)
    x, dt = torch.randn(b, d, generator=g).to(dtype), torch.randn(b, d, generator=g).to(dtype)
    A = -(torch.rand(d, n, generator=g) * 3 + 0.1)
    kind = rng.choice(["grouped", "bdn", "dn"])
    grp = rng.choice([gg for gg in (1, 2, 4) if d % gg == 0 and gg != d])
    shape = {"grouped": (b, grp, n), "bdn": (b, d, n), "dn": (d, n)}[kind]
    pt = dtype if kind == "grouped" else torch.float32
    Bm, Cm = torch.randn(*shape, generator=g).to(pt), torch.randn(*shape, generator=g).to(pt)
    D = torch.randn(d, generator=g) if rng.random() < 0.6 else None
    z = torch.randn(b, d, generator=g).to(dtype) if rng.random() < 0.6 else None
    bias = torch.randn(d, generator=g) * 0.5 if rng.random() < 0.6 else None
    sp = rng.random() < 0.7
    if not sp:
        dt, bias = dt.abs() * 0.3, None
    desc = ("step", seed, (b, d, n), kind, str(dtype), D is not None, z is not None, bias is not None, sp)
    half = dtype in HALF

    devs, refs = zip(*[_leaf(t, grad=False) for t in [state, x, dt, A, Bm, Cm, D, z, bias]])
    new_state = devs[0].clone()
    y = _ops().selective_state_step(new_state, *devs[1:], softplus=sp)
    y_ref, state_ref = O.selective_state_step_functional(*refs, softplus=sp, acc=torch.float64)
    y_32 = s_32 = None
    if not half:
        y_32, s_32 = O.selective_state_step_functional(state, x, dt, A, Bm, Cm, D, z, bias, softplus=sp)
    _close(y, y_ref, (desc, "y"), half=half, r32=y_32)
    _close(new_state, state_ref, (desc, "state"), half=half, r32=s_32)


def _conv_case(rng, seed):
    g = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    b, c = rng.randint(1, 4), rng.choice([1, 8, 24, 64, 96, 100, 512, 1536])
    l = rng.choice([rng.randint(1, 64), rng.randint(1, 1500), 256])
    l += int(c == l)
    k = rng.choice([2, 3, 4, 4, 4, 5, 7])
    channels_last = rng.random() < 0.5
    x = torch.randn(*((b, l, c) if channels_last else (b, c, l)), generator=g).to(dtype)
    wshape = rng.choice([(c, k), (c, 1, k)])
    w = (torch.rand(*wshape, generator=g) - 0.5).to(rng.choice([dtype, torch.float32]))
    bias = (torch.randn(c, generator=g) * 0.1).to(w.dtype) if rng.random() < 0.7 else None
    act = rng.choice(["silu", "silu", "identity", None])
    desc = ("conv", seed, (b, c, l, k), channels_last, str(dtype), str(w.dtype), wshape, bias is not None, act)
    half = dtype in HALF
    fn = _ops().dw_causal_conv_channels_last if channels_last else _ops().dw_causal_conv

    def ref(acc, x, w, bias):
        if channels_last:
            return O.dw_causal_conv(x.transpose(1, 2), w, bias, activation=act, acc=acc).transpose(1, 2)
        return O.dw_causal_conv(x, w, bias, activation=act, acc=acc)

    # a draw of its own (the cases above stay what they were): the (B, C, L) input as the reference's blocks pass
    # it, a permuted view of (B, L, C') rows, C' = C or wider with the channels somewhere inside
    own = random.Random(seed ^ 0x2F6B)
    if not channels_last and own.random() < 0.3:
        wide = c + own.choice([0, 0, 4, c, 3])
        off = own.choice([o for o in (0, 4, wide - c, 1) if 0 <= o <= wide - c])
        rows = torch.randn(b, l, wide, generator=g).to(dtype)
        view = lambda t: t[:, :, off:off + c].permute(0, 2, 1)
        desc = desc + ("view of rows", wide, off)
        _values_and_gradients(lambda x, w, bias: fn(view(x), w, bias, activation=act),
                              lambda acc, x, w, bias: ref(acc, view(x), w, bias), [rows, w, bias], desc, half)
        return
    _values_and_gradients(lambda x, w, bias: fn(x, w, bias, activation=act), ref, [x, w, bias], desc, half)


def _norm_case(rng, seed):
    g = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    b, l = rng.randint(1, 3), rng.randint(1, 300)
    h = rng.choice([8, 64, 100, 768, 1000, 1024, 1536, 2048, 2560, 3000, 4096, 5120, 8192, 8 * rng.randint(1, 1200),
                    rng.randint(1, 3000)])
    x = torch.randn(b, l, h, generator=g).to(dtype)
    w = torch.randn(h, generator=g).to(rng.choice([dtype, torch.float32]))
    rms = rng.random() < 0.5
    bias = None if (rms and rng.random() < 0.7) else torch.randn(h, generator=g).to(w.dtype)
    res_fp32 = rng.random() < 0.6
    res = None if rng.random() < 0.3 else torch.randn(b, l, h, generator=g).to(torch.float32 if res_fp32 else dtype)
    prenorm = rng.random() < 0.8
    desc = ("norm", seed, (b, l, h), str(dtype), str(w.dtype), rms, bias is not None,
            None if res is None else str(res.dtype), prenorm, res_fp32)
    half = dtype in HALF
    kw = dict(is_rms=rms, prenorm=prenorm, residual_in_fp32=res_fp32)
    _values_and_gradients(lambda x, w, bias, res: _ops().fused_layer_norm_with_residual(x, w, bias, residual=res, **kw),
                          lambda acc, x, w, bias, res: O.fused_layer_norm_with_residual(x, w, bias, residual=res, acc=acc, **kw),
                          [x, w, bias, res], desc, half)


def _decode_case(rng, seed):
    """Three tokens through the fused decode step against window roll + tap sum + activation + oracle step."""
    g = torch.Generator().manual_seed(seed)
    io = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    b, d, n, K = rng.randint(1, 9), rng.choice([4, 16, 40, 64, 100, 256, 1024]), rng.choice([1, 4, 16, 16, 32, 64, 5]), rng.choice([2, 3, 4, 4, 7])
    grp = rng.choice([gg for gg in (1, 2, 4) if d % gg == 0 and gg != d])
    A = -(torch.rand(d, n, generator=g) * 3 + 0.1)
    D = torch.randn(d, generator=g) if rng.random() < 0.6 else None
    bias = torch.randn(d, generator=g) * 0.5 if rng.random() < 0.6 else None
    use_z, use_cb = rng.random() < 0.6, rng.random() < 0.7
    act = rng.choice(["silu", "silu", "identity"])
    w = torch.rand(d, K, generator=g) - 0.5
    cb = torch.randn(d, generator=g) * 0.1 if use_cb else None
    cs_ref = torch.randn(b, d, K, generator=g).to(io).float()
    st_ref = torch.randn(b, d, n, generator=g)
    cs, st = cs_ref.to(io).cuda(), st_ref.clone().cuda()
    desc = ("decode", seed, (b, d, n, K), grp, str(io), D is not None, use_z, bias is not None, use_cb, act)
    half = io != torch.float32
    dev = lambda t: None if t is None else t.cuda()
    for _ in range(3):
        x, dt = torch.randn(b, d, generator=g).to(io), torch.randn(b, d, generator=g).to(io)
        Bm, Cm = torch.randn(b, grp, n, generator=g).to(io), torch.randn(b, grp, n, generator=g).to(io)
        z = torch.randn(b, d, generator=g).to(io) if use_z else None
        cs_ref = torch.roll(cs_ref, -1, dims=-1)
        cs_ref[..., -1] = x.float()
        pre = (cs_ref * w).sum(-1) + (0.0 if cb is None else cb)
        xc = (torch.nn.functional.silu(pre) if act == "silu" else pre).to(io)
        y_ref, st_ref = O.selective_state_step_functional(st_ref.double(), xc, dt, A, Bm, Cm, D, z, bias, softplus=True,
                                                          acc=torch.float64)
        y = _ops().decode_step(cs, st, x.cuda(), dt.cuda(), A.cuda(), Bm.cuda(), Cm.cuda(), w.cuda(), conv_bias=dev(cb),
                               D=dev(D), z=dev(z), dt_bias=dev(bias), softplus=True, activation=act)
        assert torch.equal(cs.float().cpu(), cs_ref), desc
        # the convolution output is rounded to the element type before the update on both sides; float32: it is a
        # float32 tap sum on the GPU against a float32 tap sum here, so the update's input agrees to a rounding
        _close(y, y_ref, (desc, "y"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 2e-5)
        _close(st, st_ref, (desc, "state"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 2e-5)
        st_ref = st_ref.float()


def _mamba2_decode_case(rng, seed):
    """Three tokens through the Mamba-2 decode step against split + window conv + per-head oracle step."""
    g = torch.Generator().manual_seed(seed)
    io = rng.choice([torch.float32, torch.bfloat16, torch.float16])
    b, G = rng.randint(1, 5), rng.choice([1, 1, 2, 4])
    H, P = G * rng.choice([1, 2, 3, 6]), rng.choice([16, 32, 64, 64, 80, 128])
    N, K = rng.choice([16, 32, 64, 128, 128]), rng.choice([2, 3, 4, 4, 7])
    di, conv_dim = H * P, H * P + 2 * G * N
    A = -(torch.rand(H, generator=g) * 4.0 + 0.5)
    D = rng.choice([None, torch.randn(H, generator=g), torch.randn(H, P, generator=g)])
    bias = torch.randn(H, generator=g) - 2.0 if rng.random() < 0.7 else None
    gate = rng.random() < 0.7
    w = torch.rand(conv_dim, K, generator=g) - 0.5
    cb = torch.randn(conv_dim, generator=g) * 0.1 if rng.random() < 0.7 else None
    cs_ref = torch.randn(b, conv_dim, K, generator=g).to(io).float()
    st_ref = torch.randn(b, H, P, N, generator=g)
    cs, st = cs_ref.to(io).cuda(), st_ref.clone().cuda()
    desc = ("mamba2 decode", seed, (b, H, P, G, N, K), str(io), None if D is None else tuple(D.shape), bias is not None, gate, cb is not None)
    half = io != torch.float32
    dev = lambda t: None if t is None else t.cuda()
    Dflat = None if D is None else (D.repeat_interleave(P) if D.ndim == 1 else D.reshape(di))
    for _ in range(3):
        row = torch.randn(b, 2 * di + 2 * G * N + H, generator=g).to(io)
        z, xBC, dt = torch.split(row.float(), [di, conv_dim, H], dim=-1)
        cs_ref = torch.roll(cs_ref, -1, dims=-1)
        cs_ref[..., -1] = xBC
        act = torch.nn.functional.silu((cs_ref * w).sum(-1) + (0.0 if cb is None else cb))
        x, Bm, Cm = torch.split(act, [di, G * N, G * N], dim=-1)
        y_ref, flat = O.selective_state_step_functional(
            st_ref.reshape(b, di, N).double(), x.double(), dt.repeat_interleave(P, dim=-1).double(),
            A.repeat_interleave(P)[:, None].expand(di, N), Bm.reshape(b, G, N).double(), Cm.reshape(b, G, N).double(), Dflat,
            z.double() if gate else None, None if bias is None else bias.repeat_interleave(P), softplus=True, acc=torch.float64)
        st_ref = flat.reshape(b, H, P, N).float()
        y = _ops().mamba2_decode_step(row.cuda(), cs, st, w.cuda(), dev(cb), A.cuda(), D=dev(D), dt_bias=dev(bias), ngroups=G,
                                      softplus=True, gate=gate)
        assert torch.equal(cs.float().cpu(), cs_ref), desc
        _close(y, y_ref, (desc, "y"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 2e-5)
        _close(st, flat.reshape(b, H, P, N), (desc, "state"), rtol=1e-4, atol_rms=2e-5)


def _dscan_case(rng, seed):
    """The reference's diagonal ``ssd_chunk_scan`` with its optional arguments, values and gradients."""
    g = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.bfloat16, torch.float16, torch.float32])
    b, l, h, p = rng.choice([1, 2, 3]), rng.randint(1, 700), rng.choice([1, 2, 4, 5]), rng.choice([8, 64, 128, 192, 20])
    chunk = rng.choice([16, 64, 256])
    X = torch.randn(b, l, h, p, generator=g).to(dtype)
    dt = torch.rand(b, l, h, generator=g) * 0.2
    per_p = rng.random() < 0.3
    A = -(torch.rand(*((h, p) if per_p else (h,)), generator=g) * 4 + 0.1)
    kind = rng.choice(["blhp", "blhp", "hp", "bhp"])
    shape = {"blhp": (b, l, h, p), "hp": (h, p), "bhp": (b, h, p)}[kind]
    pt = dtype if kind == "blhp" else rng.choice([dtype, torch.float32])
    Bm, Cm = torch.randn(*shape, generator=g).to(pt), torch.randn(*shape, generator=g).to(pt)
    D = torch.randn(*((h, p) if per_p else (h,)), generator=g) if rng.random() < 0.5 else None
    z = torch.randn(b, l, h, p, generator=g).to(dtype) if rng.random() < 0.6 else None
    init = torch.randn(b, h, p, generator=g) if rng.random() < 0.5 else None
    lens = [rng.randint(0, l) for _ in range(b)] if rng.random() < 0.4 else None
    meta = {"seq_lens": lens} if lens else None
    desc = ("dscan", seed, (b, l, h, p), chunk, str(dtype), kind, str(pt), per_p, D is not None, z is not None, init is not None, lens)
    half = dtype in HALF
    _values_and_gradients(
        lambda X, dt, A, Bm, Cm, D, z, init: _ops().ssd_chunk_scan(X, dt, A, Bm, Cm, chunk, D=D, z=z, seq_meta=meta, initial_states=init),
        lambda acc, X, dt, A, Bm, Cm, D, z, init: O.ssd_chunk_scan(X, dt, A, Bm, Cm, chunk, D=D, z=z, seq_meta=meta,
                                                                   initial_states=init, acc=acc),
        [X, dt, A, Bm, Cm, D, z, init], desc, half)


@pytest.mark.parametrize("block", range(4))
@pytest.mark.parametrize("case", [_scan_case, _step_case, _conv_case, _norm_case, _decode_case, _mamba2_decode_case, _dscan_case],
                         ids=["scan", "step", "conv", "norm", "decode", "mamba2_decode", "dscan"])
def test_operator_over_random_shapes_matches_the_float64_oracle(case, block):
    for i in range(CASES_PER_BLOCK):
        seed = 10_000 * (block + 1) + i
        case(random.Random(seed), seed)


# dA of the SSD, per head, against the sum of the magnitudes of its terms dt_t q_t
DA_TERM_BAR_HALF, DA_TERM_BAR_F32 = 5e-2, 5e-4     # seen over 3 700 cases: 3.03e-2 (one head, packed sequences of 89, 70 and 96 steps) and 3.0e-4 at worst, medians 5e-4 and 3e-6


def _ssd_case(rng, seed):
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    b, Q = rng.choice([1, 2, 3]), rng.choice([16, 32, 64, 128, 256])
    l = rng.choice([Q * rng.randint(1, 4), rng.randint(1, 3 * Q)])
    g, per = rng.choice([1, 2]), rng.choice([1, 2, 3])
    h = g * per
    p, n = rng.choice([16, 32, 64, 64, 128, 192, 24]), rng.choice([16, 32, 64, 128, 48])
    use_z, use_init, softplus = rng.random() < 0.6, rng.random() < 0.4, rng.random() < 0.7
    use_D = rng.choice([None, "h", "hp"])
    cuts = sorted(rng.sample(range(1, l), min(l - 1, rng.randint(1, 3)))) if (rng.random() < 0.3 and l >= 4) else None
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(b, l, h, p, generator=gen).to(dtype)
    dt = torch.randn(b, l, h, generator=gen) * 0.5 if softplus else torch.rand(b, l, h, generator=gen) * 0.3
    A = -(torch.rand(h, generator=gen) + 0.2)
    Bm = (torch.randn(b, l, g, n, generator=gen) * 0.5).to(dtype)
    Cm = (torch.randn(b, l, g, n, generator=gen) * 0.5).to(dtype)
    D = None if use_D is None else (torch.randn(h, generator=gen) if use_D == "h" else torch.randn(h, p, generator=gen))
    z = torch.randn(b, l, h, p, generator=gen).to(dtype) if use_z else None
    bias = torch.randn(h, generator=gen) * 0.3 if softplus else None
    init = torch.randn(b, h, p, n, generator=gen) if use_init else None
    dout, dfin = torch.randn(b, l, h, p, generator=gen).to(dtype), torch.randn(b, h, p, n, generator=gen)
    desc = ("ssd", seed, str(dtype), (b, l, h, p, g, n), Q, use_z, use_init, softplus, use_D, cuts)
    vals = dict(x=x, dt=dt, A=A, B=Bm, C=Cm, D=D, z=z, dt_bias=bias, init=init)
    w = {k: (None if v is None else v.double().clone().requires_grad_(True)) for k, v in vals.items()}
    # A per step (the same value at every step): its gradient holds the terms dt_t q_t whose sum is dA
    A_steps = w["A"][None, None, :].expand(b, l, h).clone().detach().requires_grad_(True)
    bounds = [0] + (cuts or []) + [l]                 # a packed row is each of its sequences alone
    ys = []
    for si in range(len(bounds) - 1):
        lo, hi = bounds[si], bounds[si + 1]
        yy, fin64 = SO.ssd_sequential(w["x"][:, lo:hi], w["dt"][:, lo:hi], A_steps[:, lo:hi], w["B"][:, lo:hi], w["C"][:, lo:hi],
                                      D=w["D"], z=None if z is None else w["z"][:, lo:hi], dt_bias=w["dt_bias"],
                                      dt_softplus=softplus, initial_states=w["init"] if si == 0 else None)
        ys.append(yy)
    y64 = torch.cat(ys, 1)
    seq_idx = None
    if cuts:
        seq_idx = torch.zeros(b, l, dtype=torch.int32)
        for c in cuts:
            seq_idx[:, c:] += 1
        seq_idx = seq_idx.cuda()
    from ssm_amd.ops import ssd as S
    d = {k: (None if v is None else v.cuda().clone().requires_grad_(True)) for k, v in vals.items()}
    y, fin = S.ssd_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, D=d["D"], z=d["z"], dt_bias=d["dt_bias"],
                            initial_states=d["init"], dt_softplus=softplus, return_final_states=True, seq_idx=seq_idx)
    # float32 calls: the chunked form (differences of running sums under one exponential) against the step-by-step
    # recurrence; the running sum's own float32 rounding, times its size, is the floor
    half = dtype != torch.float32
    # 16-bit calls: an output element sums products of rounded operands with a carried state that is itself rounded
    # to 16 bits once per chunk; over some hundred more seeds than the ones kept here two cases had a single
    # element (of 10^5..10^6) at 1.25 and 1.34 times the bar of an element-wise operator, so the SSD's values take
    # the gradients' bar (3e-2 of the element + 6e-2 of the rms, mean error 1e-2 of the rms)
    # 16 bits: the bar of the chunk_scan stage below (sums of products of operands rounded to 16 bits; one element in
    # 8 700 later cases lay at 0.13 of the rms where 0.03 of its value + 0.06 of the rms allowed 0.12)
    _close(y, y64, (desc, "y"), half=half, grad=half, rtol=None if half else 2e-4, atol_rms=8e-2 if half else 2e-4)
    _close(fin, fin64, (desc, "final state"), half=half, grad=half, rtol=None if half else 2e-4, atol_rms=None if half else 2e-4)
    ((y64 * dout.double()).sum() + (fin64 * dfin.double()).sum()).backward()
    ((y.float() * dout.cuda().float()).sum() + (fin.float() * dfin.cuda()).sum()).backward()
    mean_bar, max_bar = (2e-4, 2e-3) if dtype == torch.float32 else (2e-2, 0.3)
    w["A"].grad = A_steps.grad.sum(dim=(0, 1))
    dA_terms = A_steps.grad.abs().sum(dim=(0, 1))          # per head: sum over batch and time of |dt_t q_t|
    for k, v in vals.items():
        if v is None:
            continue
        want, got = w[k].grad, d[k].grad.float().cpu().double()
        assert torch.isfinite(got).all(), (desc, k)
        err = (got - want).abs()
        if k == "dt_bias":          # a sum of the step's gradients over batch and time: measure against its terms
            scale = w["dt"].grad.abs().sum(dim=(0, 1))
            # (15: one head in 3 700 cases lay at 10.03 of these units)
            bar = 15 * mean_bar * scale / max(1.0, (b * l) ** 0.5) + 1e-6 * scale + 1e-12
            assert bool((err <= bar).all()), (desc, k, "err / bar per head", (err / bar).tolist())
        elif k == "A":
            # the sum over time of step x running sum q: its terms cancel, so a head's own value is a poor
            # yardstick for the error of the sum; each head is measured against the sum of the magnitudes of its
            # own terms (what the 16-bit passes' running sum is worth per term: DA_TERM_BAR)
            bar = DA_TERM_BAR_F32 if dtype == torch.float32 else DA_TERM_BAR_HALF
            ratio = err / (dA_terms + 1e-30)
            assert bool((err <= bar * dA_terms + 1e-9).all()), (desc, k, "err / sum |terms| per head", ratio.tolist())
        else:
            rms = float(want.pow(2).mean().sqrt()) + 1e-30
            # a single element tens of times the rms carries the rounding of its own 16-bit value
            assert float(err.mean()) / rms < mean_bar, (desc, k, float(err.mean()) / rms)
            assert bool((err <= max_bar * rms + (0.0 if dtype == torch.float32 else 2e-2) * want.abs()).all()), (desc, k)


def _scan_wide_case(rng, seed):
    """Shapes of the size the specialised scan kernels are picked for (hundreds of channels per group, long rows,
    whole grids of workgroups).  Forward against the float64 oracle; backward -- the oracle's autograd takes
    minutes at these sizes -- against the general backward kernel on the same inputs, which the small shapes
    above pin against the oracle."""
    g = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    groups = rng.choice([1, 1, 2, 4])
    d = groups * rng.choice([48, 96, 192, 384, 768, 1536, 40, 200])
    if random.Random(seed ^ 0x5BD1).random() < 0.15:      # (drawn apart, so that the other seeds keep their cases)
        groups = d = rng.choice([48, 96, 200, 40])         # projections of their own per channel: (B, D, N, L)
    b, n = rng.randint(1, 8), rng.choice([16, 16, 16, 8, 4])
    l = rng.choice([16 * rng.randint(17, 160), 8 * rng.randint(33, 300), rng.randint(257, 2500)])
    while b * d * l > 6_000_000:
        if b > 1:
            b //= 2
        else:
            l //= 2
    u = torch.randn(b, d, l, generator=g).to(dtype)
    delta = torch.randn(b, d, l, generator=g).to(dtype)
    A = -(torch.rand(d, n, generator=g) * 3 + 0.1)
    bc = rng.choice([dtype, dtype, torch.float32])
    Bm, Cm = torch.randn(b, groups, n, l, generator=g).to(bc), torch.randn(b, groups, n, l, generator=g).to(bc)
    const = random.Random(seed ^ 0x7A3F)                   # (drawn apart again)
    kinds = None
    if const.random() < 0.15:                              # projections constant in time: (D, N) or (B, D, N)
        kinds = const.choice([("dn", "dn"), ("bdn", "bdn"), ("dn", "bdn"), ("bdn", "dn")])
        shape = {"dn": (d, n), "bdn": (b, d, n)}
        Bm, Cm = (torch.randn(*shape[k], generator=g).to(const.choice([torch.float32, bc])) for k in kinds)
    D = torch.randn(d, generator=g) if rng.random() < 0.7 else None
    z = torch.randn(b, d, l, generator=g).to(dtype) if rng.random() < 0.7 else None
    bias = torch.randn(d, generator=g) * 0.5 if rng.random() < 0.7 else None
    with_last = rng.random() < 0.5
    half = dtype in HALF
    desc = ("scan wide", seed, (b, d, l, n), groups, str(dtype), str(bc), D is not None, z is not None, bias is not None, with_last, kinds)
    dev = lambda t: None if t is None else t.cuda()
    with torch.no_grad():
        y64, last64 = O.selective_scan(u, delta, A, Bm, Cm, D, z, bias, softplus=True, return_last_state=True, acc=torch.float64)
        y, last = _ops().selective_scan(dev(u), dev(delta), dev(A), dev(Bm), dev(Cm), dev(D), dev(z), dev(bias), softplus=True,
                                        return_last_state=True)
    _close(y, y64, (desc, "y"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 2e-5)
    _close(last, last64, (desc, "last state"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 2e-5)
    go = torch.randn(b, d, l, generator=g).to(dtype).cuda()
    gl = torch.randn(b, d, n, generator=g).cuda() if with_last else None
    args = (go, gl, dev(u), dev(delta), dev(A), dev(Bm), dev(Cm), dev(D), dev(z), dev(bias), True)
    fast = _ops()._scan_backward(*args, tune_items=0)
    general = _ops()._scan_backward(*args, tune_items=1)
    for name, f, r in zip("u delta A B C D z dt_bias".split(), fast, general):
        assert (f is None) == (r is None), (desc, name)
        if r is None:
            continue
        # per-token gradients come back in the element type: one last place of a 16-bit value apart at most
        if half and name in ("u", "delta", "z"):
            _close(f.float(), r.float(), (desc, name), rtol=2.0 ** -7, atol_rms=1e-3)
        else:
            _close(f.float(), r.float(), (desc, name), rtol=3e-4, atol_rms=3e-4)


@pytest.mark.parametrize("block", range(3))
def test_scan_at_the_sizes_of_its_specialised_kernels_matches_the_float64_oracle(block):
    for i in range(4):
        seed = 50_000 * (block + 1) + i
        _scan_wide_case(random.Random(seed), seed)


def _model_case(rng, seed):
    """A small Mamba-2 or Mamba-1 stack of random block shape: dense forward over a prompt of random length,
    then cached steps, against the CPU oracle stack on the same weights (bars of tests/test_harness_gpu.py)."""
    from oracle import model_oracle as M
    from ssm_amd.harness import Mamba1Config, Mamba1LM, Mamba2Config, Mamba2LM
    kind = rng.choice(["mamba2", "mamba2", "mamba1"])
    vocab, layers, conv = rng.choice([97, 300, 512]), rng.choice([1, 2, 3]), rng.choice([2, 3, 4, 4])
    if kind == "mamba1":
        cfg = Mamba1Config(d_model=rng.choice([64, 128, 192]), n_layer=layers, expand=2, d_state=rng.choice([8, 16, 16]),
                           d_conv=conv, vocab_size=vocab)
        model = Mamba1LM(cfg, seed=seed % 1000)
    else:
        headdim = rng.choice([32, 64, 64])
        d_model = headdim * rng.choice([1, 2, 3])
        heads = 2 * d_model // headdim
        cfg = Mamba2Config(d_model=d_model, n_layer=layers, expand=2, headdim=headdim, d_state=rng.choice([16, 64, 128]),
                           ngroups=rng.choice([gg for gg in (1, 2) if heads % gg == 0]), d_conv=conv,
                           chunk_size=rng.choice([32, 64, 128, 256]), vocab_size=vocab)
        model = Mamba2LM(cfg, seed=seed % 1000)
    b, prompt, steps = rng.randint(1, 3), rng.choice([1, 2, rng.randint(3, 300), 128, 256]), rng.randint(1, 4)
    # the reference's layout rule for the convolution reads a sequence exactly as long as there are channels as
    # channels-first, and the oracle follows it: keep the oracle's sequence off that length
    steps += int(prompt + steps == (cfg.d_inner if kind == "mamba1" else cfg.conv_dim))
    tokens = torch.randint(0, vocab, (b, prompt + steps), generator=torch.Generator().manual_seed(seed)).cuda()
    desc = ("model", seed, kind, cfg, b, prompt, steps)
    if kind == "mamba1":
        w = M.weights_to_cpu(model, M.MAMBA1_LAYER_TENSORS)
        ref = M.mamba1_forward(w, tokens.cpu(), d_state=cfg.d_state, dt_rank=cfg.rank, eps=cfg.eps)
    else:
        w = M.weights_to_cpu(model, M.MAMBA2_LAYER_TENSORS)
        ref = M.mamba2_forward(w, tokens.cpu(), d_inner=cfg.d_inner, nheads=cfg.nheads, headdim=cfg.headdim,
                               d_state=cfg.d_state, ngroups=cfg.ngroups, eps=cfg.eps)
    ref = ref.float()
    rms = float(ref.pow(2).mean().sqrt())

    def close(got, want, what):
        got = got.float().cpu()
        assert torch.isfinite(got).all(), (desc, what)
        err = (got - want).abs()
        # one logit in a few hundred cases of narrow stacks is 7 % of the rms off, the mean 1.2 %: bars a little
        # wider than for the fixed shapes, far below what a wrong split or order of operations gives (100 %)
        assert bool((err <= 3e-2 * want.abs() + 1e-1 * rms).all()), (desc, what, float(err.max()), rms)
        assert float(err.mean()) < 1.5e-2 * rms, (desc, what, "mean", float(err.mean()), rms)

    with torch.no_grad():
        logits, cache = model.forward(tokens[:, :prompt], return_cache=True)
        close(logits, ref[:, :prompt], "dense forward")
        for t in range(prompt, prompt + steps):
            close(model.step(tokens[:, t], cache), ref[:, t], "cached step at %d" % t)


@pytest.mark.parametrize("block", range(3))
def test_small_stacks_of_random_shape_match_the_oracle_stack(block):
    for i in range(6):
        seed = 40_000 * (block + 1) + i
        _model_case(random.Random(seed), seed)


def _ssd_stages_case(rng, seed):
    """Each stage of the SSD on its own, fed with the float64 oracle's result of the stage before, so that no
    stage's error hides behind another's: running sums, chunk products, chunk states, state passing, chunk
    outputs, and the per-sequence end states of a packed row."""
    from ssm_amd.ops import ssd as S
    gen = torch.Generator().manual_seed(seed)
    dtype = rng.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
    b, Q = rng.choice([1, 1, 2, 3]), rng.choice([16, 32, 64, 128, 256])
    l = rng.choice([Q * rng.randint(1, 4), rng.randint(1, 3 * Q)])
    g, per = rng.choice([1, 2]), rng.choice([1, 2, 3])
    h = g * per
    p, n = rng.choice([16, 32, 64, 64, 24]), rng.choice([16, 32, 64, 128, 48])
    softplus, use_z, use_init = rng.random() < 0.7, rng.random() < 0.6, rng.random() < 0.5
    use_D = rng.choice([None, "h", "hp"])
    cuts = sorted(rng.sample(range(1, l), min(l - 1, rng.randint(1, 3)))) if (rng.random() < 0.4 and l >= 4) else None
    x = torch.randn(b, l, h, p, generator=gen).to(dtype)
    dt = torch.randn(b, l, h, generator=gen) * 0.5 if softplus else torch.rand(b, l, h, generator=gen) * 0.3
    A = -(torch.rand(h, generator=gen) + 0.2)
    Bm = (torch.randn(b, l, g, n, generator=gen) * 0.5).to(dtype)
    Cm = (torch.randn(b, l, g, n, generator=gen) * 0.5).to(dtype)
    D = None if use_D is None else (torch.randn(h, generator=gen) if use_D == "h" else torch.randn(h, p, generator=gen))
    z = torch.randn(b, l, h, p, generator=gen).to(dtype) if use_z else None
    bias = torch.randn(h, generator=gen) * 0.3 if softplus else None
    init = torch.randn(b, h, p, n, generator=gen) if use_init else None
    seq_idx = None
    if cuts:
        seq_idx = torch.zeros(b, l, dtype=torch.int32)
        for c in cuts:
            seq_idx[:, c:] += 1
    desc = ("ssd stages", seed, str(dtype), (b, l, h, p, g, n), Q, softplus, use_z, use_init, use_D, cuts)
    dev = lambda t: None if t is None else t.cuda()
    half = dtype != torch.float32
    sid = dev(seq_idx)

    cs64, dtc64 = SO.chunk_cumsum(dt, A, Q, dt_bias=bias, dt_softplus=softplus)
    cs, dtc = S.chunk_cumsum(dev(dt), dev(A), Q, dt_bias=dev(bias), dt_softplus=softplus)
    _close(cs, cs64, (desc, "chunk_cumsum"), rtol=1e-5, atol_rms=1e-5)
    _close(dtc, dtc64, (desc, "chunk_cumsum dt"), rtol=1e-5, atol_rms=1e-5)
    cs32, dtc32 = cs64.float().cuda(), dtc64.float().cuda()

    causal = rng.random() < 0.5
    cb64 = SO.bmm_chunk(Cm, Bm, Q, seq_idx=seq_idx, causal=causal)
    cb = S.bmm_chunk(dev(Cm), dev(Bm), Q, seq_idx=sid, causal=causal, output_dtype=torch.float32)
    _close(cb, cb64, (desc, "bmm_chunk"), rtol=1e-5, atol_rms=1e-5)      # exact products of 16-bit values, float32 sums

    st64 = SO.chunk_state(Bm, x, dtc64, cs64, seq_idx=seq_idx)
    st = S.chunk_state(dev(Bm), dev(x), dtc32, cs32, seq_idx=sid)
    # (float32: the running sums arrive rounded to float32, which the exponentials of their differences magnify;
    #  worst of 1 070 cases 5.4e-5 of the rms)
    _close(st, st64, (desc, "chunk_state"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 1e-4)

    ent64, fin64 = SO.state_passing(st64, cs64[..., -1], initial_states=init, seq_idx=seq_idx, chunk_size=Q)
    ent, fin = S.state_passing(st64.float().cuda(), cs32[..., -1].contiguous(), initial_states=dev(init), seq_idx=sid, chunk_size=Q)
    _close(ent, ent64, (desc, "state_passing"), rtol=2e-5, atol_rms=2e-5)
    _close(fin, fin64, (desc, "state_passing final"), rtol=2e-5, atol_rms=2e-5)

    y64 = SO.chunk_scan(Bm, Cm, x, dtc64, cs64, ent64, D=D, z=z, seq_idx=seq_idx)
    y = S.chunk_scan(dev(Bm), dev(Cm), dev(x), dtc32, cs32, ent64.float().cuda(), D=dev(D), z=dev(z), seq_idx=sid)
    # (16-bit: two roundings of operands ahead of the output's own, as in the gradients: their bar on single elements;
    #  worst of 1 070 cases 7.6e-2 of the rms in one element, the mean error stays under 5e-3)
    _close(y, y64, (desc, "chunk_scan"), half=half, rtol=None if half else 1e-4, atol_rms=8e-2 if half else 1e-4)

    if cuts and b == 1:
        cu = torch.tensor([0] + cuts + [l], dtype=torch.int32)
        ends64 = SO.chunk_state_varlen(Bm, x, dtc64, cs64, cu, ent64)
        ends = S.chunk_state_varlen(dev(Bm), dev(x), dtc32, cs32, cu.cuda(), ent64.float().cuda())
        _close(ends, ends64, (desc, "chunk_state_varlen"), half=half, rtol=None if half else 1e-4, atol_rms=None if half else 2e-5)


@pytest.mark.parametrize("block", range(4))
def test_ssd_stages_over_random_shapes_match_the_float64_oracle_stage_by_stage(block):
    for i in range(CASES_PER_BLOCK):
        seed = 30_000 * (block + 1) + i
        _ssd_stages_case(random.Random(seed), seed)


@pytest.mark.parametrize("block", range(4))
def test_ssd_combined_over_random_shapes_matches_the_float64_recurrence(block):
    for i in range(CASES_PER_BLOCK):
        seed = 20_000 * (block + 1) + i
        _ssd_case(random.Random(seed), seed)

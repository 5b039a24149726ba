"""GPU parity of ``selective_state_step`` against the CPU oracle and the
upstream ``selective_state_update`` vectors."""

import pytest
import torch

from oracle import ops_oracle as O
from tests import fixtures as fx

pytestmark = pytest.mark.gpu

FP32_TOL = dict(rtol=1e-5, atol=1e-5)
HALF_TOL = dict(rtol=2e-2, atol=2e-3)


def dev(t):
    return None if t is None else t.cuda()


def _ops():
    from ssm_amd import ops
    return ops


def make(seed, batch, dim, nstate, io=torch.float32, st=torch.float32, bkind="bgn", ckind="bgn", groups=1,
         use_D=True, use_z=True, use_bias=True):
    g = torch.Generator().manual_seed(seed)
    state = torch.randn(batch, dim, nstate, generator=g).to(st)
    x = torch.randn(batch, dim, generator=g).to(io)
    dt = torch.randn(batch, dim, generator=g).to(io)
    z = torch.randn(batch, dim, generator=g).to(io) if use_z else None
    A = -torch.arange(1, nstate + 1, dtype=torch.float32).repeat(dim, 1) * (1 + 0.1 * torch.rand(dim, nstate, generator=g))

    def proj(kind):
        if kind == "dn":
            return torch.randn(dim, nstate, generator=g).to(io)
        if kind == "bdn":
            return torch.randn(batch, dim, nstate, generator=g).to(io)
        return torch.randn(batch, groups, nstate, generator=g).to(io)

    Bm, Cm = proj(bkind), proj(ckind)
    D = torch.randn(dim, generator=g) if use_D else None
    bias = torch.randn(dim, generator=g) - 3.0 if use_bias else None
    return dict(state=state, x=x, dt=dt, A=A, B=Bm, C=Cm, D=D, z=z, dt_bias=bias)


def run_both(inp, softplus=True):
    st_ref = inp["state"].clone()
    y_ref = O.selective_state_step(st_ref, inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"],
                                   z=inp["z"], dt_bias=inp["dt_bias"], softplus=softplus)
    st = dev(inp["state"].clone())
    y = _ops().selective_state_step(st, dev(inp["x"]), dev(inp["dt"]), dev(inp["A"]), dev(inp["B"]),
                                    dev(inp["C"]), D=dev(inp["D"]), z=dev(inp["z"]),
                                    dt_bias=dev(inp["dt_bias"]), softplus=softplus)
    return (y.cpu(), st.cpu()), (y_ref, st_ref)


def test_upstream_baseline_vector():
    rec = fx.upstream("selective_state_update", "baseline_full")
    i = rec["inputs"]
    st = dev(i["state"].clone())
    y = _ops().selective_state_step(st, dev(i["x"]), dev(i["dt"]), dev(i["A"]), dev(i["B"][:, None].contiguous()),
                                    dev(i["C"][:, None].contiguous()), D=dev(i["D"]), z=dev(i["z"]),
                                    dt_bias=dev(i["dt_bias"]), softplus=True)
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(st.cpu(), rec["outputs"]["updated_state"], rtol=1e-4, atol=1e-5)


def test_upstream_grouped_heads_vector():
    rec = fx.upstream("selective_state_update", "grouped")
    i = rec["inputs"]
    b, h, d, n = i["state"].shape
    st = dev(i["state"].reshape(b, h * d, n).clone())
    y = _ops().selective_state_step(st, dev(i["x"].reshape(b, h * d)), dev(i["dt"].reshape(b, h * d)),
                                    dev(i["A"].reshape(h * d, n)), dev(i["B"]), dev(i["C"]),
                                    dt_bias=dev(i["dt_bias"].reshape(h * d)), softplus=False)
    torch.testing.assert_close(y.cpu().reshape(b, h, d), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(st.cpu().reshape(b, h, d, n), rec["outputs"]["updated_state"], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 3, 4), (4, 512, 16), (3, 40, 17), (2, 64, 64), (2, 8, 256), (5, 7, 6)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("kinds", [("bgn", "bgn"), ("dn", "dn"), ("bdn", "bgn"), ("bgn", "dn")])
def test_fp32_matches_oracle(shape, kinds):
    b, d, n = shape
    inp = make(sum(shape), b, d, n, bkind=kinds[0], ckind=kinds[1])
    (y, st), (yr, sr) = run_both(inp)
    torch.testing.assert_close(y, yr, **FP32_TOL)
    torch.testing.assert_close(st, sr, **FP32_TOL)


@pytest.mark.parametrize("groups,dim", [(1, 8), (2, 8), (4, 8), (3, 6)])
def test_groups(groups, dim):
    inp = make(3, 3, dim, 16, groups=groups)
    (y, st), (yr, sr) = run_both(inp)
    torch.testing.assert_close(y, yr, **FP32_TOL)
    torch.testing.assert_close(st, sr, **FP32_TOL)


@pytest.mark.parametrize("io,st", [(torch.bfloat16, torch.float32), (torch.float16, torch.float32),
                                   (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16)])
def test_half_activations(io, st):
    inp = make(5, 4, 96, 16, io=io, st=st)
    (y, s), (yr, sr) = run_both(inp)
    assert y.dtype == io and s.dtype == st
    torch.testing.assert_close(y.float(), yr.float(), **HALF_TOL)
    tol = FP32_TOL if st == torch.float32 else HALF_TOL
    torch.testing.assert_close(s.float(), sr.float(), **tol)


@pytest.mark.parametrize("use_D,use_z,use_bias,softplus", [(False, False, False, False), (True, False, True, True),
                                                           (False, True, False, True)])
def test_optional_arguments(use_D, use_z, use_bias, softplus):
    inp = make(8, 2, 24, 8, use_D=use_D, use_z=use_z, use_bias=use_bias)
    if not softplus:
        inp["dt"] = inp["dt"].abs() * 0.1
    (y, st), (yr, sr) = run_both(inp, softplus=softplus)
    torch.testing.assert_close(y, yr, **FP32_TOL)
    torch.testing.assert_close(st, sr, **FP32_TOL)


@pytest.mark.parametrize("io,batch,dim,nstate,groups", [(torch.bfloat16, 8, 1536, 16, 1), (torch.float32, 3, 96, 8, 2),
                                                         (torch.float16, 5, 64, 12, 1), (torch.bfloat16, 2, 40, 6, 1)])
def test_rows_cut_out_of_wider_rows_are_taken_as_they_are(io, batch, dim, nstate, groups):
    """z, B and C as slices of one projected row per batch entry (what a decoding block has): the kernel reads them
    in place through their batch strides; same result as dense copies, and the wrapper makes no copy when the
    slices are 8-byte aligned (an odd offset falls back to one)."""
    inp = make(21, batch, dim, nstate, io=io, st=torch.float32, groups=groups)
    gn = groups * nstate
    for lead in (8, 3):
        wide = torch.cat([torch.zeros(batch, lead).to(io), inp["z"], inp["B"].reshape(batch, gn),
                          inp["C"].reshape(batch, gn), torch.zeros(batch, 5).to(io)], dim=1).cuda()
        z = wide[:, lead:lead + dim]
        Bm = wide[:, lead + dim:lead + dim + gn].reshape(batch, groups, nstate)
        Cm = wide[:, lead + dim + gn:lead + dim + 2 * gn].reshape(batch, groups, nstate)
        assert not z.is_contiguous() and Bm.data_ptr() == wide.data_ptr() + (lead + dim) * wide.element_size()
        st = dev(inp["state"].clone())
        plan = _ops().StepPlan(st, dev(inp["x"]), dev(inp["dt"]), dev(inp["A"]), Bm, Cm, dev(inp["D"]), z,
                               dev(inp["dt_bias"]), True)
        in_place = plan.keep["z"].data_ptr() == z.data_ptr() and plan.keep["B"].data_ptr() == Bm.data_ptr()
        y = plan.run()
        st2 = dev(inp["state"].clone())
        y2 = _ops().selective_state_step(st2, dev(inp["x"]), dev(inp["dt"]), dev(inp["A"]), dev(inp["B"]), dev(inp["C"]),
                                         D=dev(inp["D"]), z=dev(inp["z"]), dt_bias=dev(inp["dt_bias"]), softplus=True)
        torch.testing.assert_close(y, y2, rtol=0, atol=0)
        torch.testing.assert_close(st, st2, rtol=0, atol=0)
        row_bytes_ok = (wide.stride(0) * wide.element_size()) % 8 == 0
        offsets_ok = all(t.data_ptr() % 8 == 0 for t in (z, Bm, Cm))
        if row_bytes_ok and offsets_ok:
            assert in_place, "aligned slices should be read in place"


def test_repeated_steps_equal_scan_last_state():
    """L steps from a zero state reproduce selective_scan and its last_state."""
    from tests.test_scan_fwd_gpu import make_inputs
    ops = _ops()
    inp = make_inputs(21, 2, 16, 33, 16)
    g = {k: dev(v) for k, v in inp.items()}
    y, h = ops.selective_scan(g["u"], g["delta"], g["A"], g["B"], g["C"], D=g["D"], z=g["z"],
                              dt_bias=g["dt_bias"], softplus=True, return_last_state=True)
    st = torch.zeros(2, 16, 16, device="cuda")
    for t in range(33):
        yt = ops.selective_state_step(st, g["u"][:, :, t].contiguous(), g["delta"][:, :, t].contiguous(), g["A"],
                                      g["B"][..., t].contiguous(), g["C"][..., t].contiguous(), D=g["D"],
                                      z=g["z"][:, :, t].contiguous(), dt_bias=g["dt_bias"], softplus=True)
        torch.testing.assert_close(yt, y[:, :, t], **FP32_TOL)
    torch.testing.assert_close(st, h, **FP32_TOL)


def test_config2_shape_512_steps():
    """BASELINE config 2: B=64, D=5120, N=16, bf16 activations, fp32 state, grouped
    B/C (64,1,16).  512 in-place steps on the GPU; a channel slice is replayed on the
    CPU oracle (a linear slice is exact because channels are independent)."""
    ops = _ops()
    g = torch.Generator().manual_seed(2)
    Bsz, D, N, steps = 64, 5120, 16, 512
    state = torch.randn(Bsz, D, N, generator=g)
    A = -torch.arange(1, N + 1, dtype=torch.float32).repeat(D, 1)
    Dk = torch.ones(D)
    from ssm_amd.configs import inverse_softplus_dt
    bias = inverse_softplus_dt(D, g)
    idx = torch.arange(0, D, 640)
    st_gpu = state.cuda()
    st_ref = state[:, idx].clone()
    A_g, D_g, b_g = A.cuda(), Dk.cuda(), bias.cuda()
    check_at = {0, 1, 17, 255, 511}
    for s in range(steps):
        x = torch.randn(Bsz, D, generator=g).to(torch.bfloat16)
        z = torch.randn(Bsz, D, generator=g).to(torch.bfloat16)
        dt = torch.randn(Bsz, D, generator=g).to(torch.bfloat16)
        Bm = torch.randn(Bsz, 1, N, generator=g).to(torch.bfloat16)
        Cm = torch.randn(Bsz, 1, N, generator=g).to(torch.bfloat16)
        y = ops.selective_state_step(st_gpu, x.cuda(), dt.cuda(), A_g, Bm.cuda(), Cm.cuda(), D=D_g, z=z.cuda(),
                                     dt_bias=b_g, softplus=True)
        yr = O.selective_state_step(st_ref, x[:, idx], dt[:, idx], A[idx], Bm, Cm, D=Dk[idx], z=z[:, idx],
                                    dt_bias=bias[idx], softplus=True)
        if s in check_at:
            torch.testing.assert_close(y[:, idx.cuda()].float().cpu(), yr.float(), **HALF_TOL)
    torch.testing.assert_close(st_gpu[:, idx.cuda()].cpu(), st_ref, rtol=1e-4, atol=1e-4)


def test_config2_fused_decode_step_512_steps():
    """BASELINE config 2 with both of its states: B=64, D=5120, N=16, conv width 4, bf16 activations and
    window, fp32 SSM state, grouped B/C (64,1,16), 512 in-place fused decode steps (the call ``bench.py``
    times).  A channel slice is replayed on the CPU the way the reference's ``Mamba1.step`` does
    (``/root/reference/src/ssm/modules/mamba1.py:345-381``): roll the window, tap sum + bias, SiLU, then the
    oracle's state step.  The window holds copies of the inputs, so it is compared bit for bit."""
    ops = _ops()
    from ssm_amd.configs import inverse_softplus_dt
    g = torch.Generator().manual_seed(22)
    Bsz, D, N, K, steps = 64, 5120, 16, 4, 512
    state = torch.randn(Bsz, D, N, generator=g)
    window = torch.randn(Bsz, D, K, generator=g).to(torch.bfloat16)
    A = -torch.arange(1, N + 1, dtype=torch.float32).repeat(D, 1)
    Dk = torch.ones(D)
    bias = inverse_softplus_dt(D, g)
    w = torch.rand(D, K, generator=g) - 0.5
    cb = torch.randn(D, generator=g) * 0.02
    idx = torch.cat([torch.arange(0, D, 320), torch.tensor([1, 2, 3, D - 1])])
    idx_g = idx.cuda()
    st_gpu, win_gpu = state.cuda(), window.cuda()
    st_ref, win_ref = state[:, idx].clone(), window[:, idx].float()
    A_g, D_g, b_g, w_g, cb_g = A.cuda(), Dk.cuda(), bias.cuda(), w.cuda(), cb.cuda()
    check_at = {0, 1, 2, 3, 4, 17, 255, 511}
    for s in range(steps):
        x = torch.randn(Bsz, D, generator=g).to(torch.bfloat16)
        z = torch.randn(Bsz, D, generator=g).to(torch.bfloat16)
        dt = torch.randn(Bsz, D, generator=g).to(torch.bfloat16)
        Bm = torch.randn(Bsz, 1, N, generator=g).to(torch.bfloat16)
        Cm = torch.randn(Bsz, 1, N, generator=g).to(torch.bfloat16)
        y, xc = ops.decode_step(win_gpu, st_gpu, x.cuda(), dt.cuda(), A_g, Bm.cuda(), Cm.cuda(), w_g, conv_bias=cb_g,
                                D=D_g, z=z.cuda(), dt_bias=b_g, softplus=True, return_conv_out=True)
        win_ref = torch.roll(win_ref, -1, dims=-1)
        win_ref[..., -1] = x[:, idx].float()
        xc_ref = torch.nn.functional.silu((win_ref * w[idx]).sum(-1) + cb[idx]).to(torch.bfloat16)
        yr = O.selective_state_step(st_ref, xc_ref, dt[:, idx], A[idx], Bm, Cm, D=Dk[idx], z=z[:, idx],
                                    dt_bias=bias[idx], softplus=True)
        if s in check_at:
            torch.testing.assert_close(win_gpu[:, idx_g].float().cpu(), win_ref, rtol=0, atol=0)
            torch.testing.assert_close(xc[:, idx_g].float().cpu(), xc_ref.float(), **HALF_TOL)
            torch.testing.assert_close(y[:, idx_g].float().cpu(), yr.float(), **HALF_TOL)
    torch.testing.assert_close(win_gpu[:, idx_g].float().cpu(), win_ref, rtol=0, atol=0)
    # the convolution output is rounded to bf16 on both sides; where the two roundings fall on different
    # sides the state sees one bf16 ulp of xc times dt.B, which decays like the state itself
    torch.testing.assert_close(st_gpu[:, idx_g].cpu(), st_ref, rtol=2e-2, atol=2e-2)
    err = (st_gpu[:, idx_g].cpu() - st_ref).abs().mean() / st_ref.abs().mean()
    assert float(err) < 2e-3, float(err)


@pytest.mark.parametrize("io", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [2, 4, 7])
def test_fused_decode_step_equals_conv_window_then_state_step(io, K):
    """decode_step == (roll window, tap sum, SiLU) followed by selective_state_step,
    the sequence of tensor ops in the reference's Mamba1.step."""
    ops = _ops()
    g = torch.Generator().manual_seed(K)
    Bsz, D, N = 3, 40, 16
    inp = make(K, Bsz, D, N, io=io)
    conv_state = torch.randn(Bsz, D, K, generator=g).to(io)
    w = torch.rand(D, K, generator=g) - 0.5
    cb = torch.randn(D, generator=g) * 0.02
    # oracle: explicit window update on the CPU, then the oracle step
    cs_ref = torch.roll(conv_state.float(), -1, dims=-1)
    cs_ref[..., -1] = inp["x"].float()
    xc = torch.nn.functional.silu((cs_ref * w).sum(-1) + cb).to(io)
    st_ref = inp["state"].clone()
    y_ref = O.selective_state_step(st_ref, xc, inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                                   dt_bias=inp["dt_bias"], softplus=True)
    cs = conv_state.clone().cuda()
    st = inp["state"].clone().cuda()
    y, xc_gpu = ops.decode_step(cs, st, dev(inp["x"]), dev(inp["dt"]), dev(inp["A"]), dev(inp["B"]), dev(inp["C"]),
                                w.cuda(), conv_bias=cb.cuda(), D=dev(inp["D"]), z=dev(inp["z"]),
                                dt_bias=dev(inp["dt_bias"]), softplus=True, return_conv_out=True)
    tol = FP32_TOL if io == torch.float32 else HALF_TOL
    torch.testing.assert_close(cs.float().cpu(), cs_ref.to(io).float(), rtol=0, atol=0)
    torch.testing.assert_close(xc_gpu.float().cpu(), xc.float(), **tol)
    torch.testing.assert_close(y.float().cpu(), y_ref.float(), **tol)
    torch.testing.assert_close(st.cpu(), st_ref, **(FP32_TOL if io == torch.float32 else dict(rtol=2e-2, atol=2e-2)))


@pytest.mark.parametrize("io", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(2, 4, 64, 1, 64, 4), (3, 6, 32, 2, 16, 4), (1, 3, 80, 3, 128, 2), (2, 8, 64, 8, 32, 7)],
                         ids=lambda s: "B%d_H%d_P%d_G%d_N%d_K%d" % s)
def test_mamba2_decode_step_equals_window_conv_then_per_head_state_step(io, shape):
    """mamba2_decode_step over three consecutive tokens == splitting the projected row into z | xBC | dt,
    rolling the convolution window, tap sum + bias + SiLU, and the oracle's single-token update with the
    per-head dt, A, D spread over the head's channels (the tensor ops of the reference's Mamba2.step)."""
    ops = _ops()
    Bsz, H, P, G, N, K = shape
    g = torch.Generator().manual_seed(sum(shape))
    di, conv_dim = H * P, H * P + 2 * G * N
    A = -(torch.rand(H, generator=g) * 4.0 + 0.5)
    D = torch.randn(H, generator=g)
    bias = torch.randn(H, generator=g) - 2.0
    w = torch.rand(conv_dim, K, generator=g) - 0.5
    cb = torch.randn(conv_dim, generator=g) * 0.1
    cs_ref = torch.randn(Bsz, conv_dim, K, generator=g).to(io).float()
    st_ref = torch.randn(Bsz, H, P, N, generator=g)
    cs, st = cs_ref.to(io).cuda(), st_ref.clone().cuda()
    tol = FP32_TOL if io == torch.float32 else HALF_TOL
    for step in range(3):
        row = torch.randn(Bsz, 2 * di + 2 * G * N + H, generator=g).to(io)
        z, xBC, dt = torch.split(row.float(), [di, conv_dim, H], dim=-1)
        cs_ref = torch.roll(cs_ref, -1, dims=-1)
        cs_ref[..., -1] = xBC
        act = torch.nn.functional.silu((cs_ref * w).sum(-1) + cb)
        x, Bm, Cm = torch.split(act, [di, G * N, G * N], dim=-1)
        flat = st_ref.reshape(Bsz, di, N).clone()
        y_ref = O.selective_state_step(flat, x, dt.repeat_interleave(P, dim=-1),
                                       A.repeat_interleave(P)[:, None].expand(di, N), Bm.reshape(Bsz, G, N),
                                       Cm.reshape(Bsz, G, N), D=D.repeat_interleave(P), z=z,
                                       dt_bias=bias.repeat_interleave(P), softplus=True)
        st_ref = flat.reshape(Bsz, H, P, N)
        y, act_gpu = ops.mamba2_decode_step(row.cuda(), cs, st, w.cuda(), cb.cuda(), A.cuda(), D=D.cuda(),
                                            dt_bias=bias.cuda(), ngroups=G, softplus=True, gate=True,
                                            return_conv_out=True)
        assert y.dtype == io
        torch.testing.assert_close(cs.float().cpu(), cs_ref, rtol=0, atol=0)
        torch.testing.assert_close(act_gpu.cpu(), act, **FP32_TOL)
        torch.testing.assert_close(y.float().cpu(), y_ref.float(), **tol)
        torch.testing.assert_close(st.cpu(), st_ref, **FP32_TOL)


def test_mamba2_decode_step_options_and_errors():
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    Bsz, H, P, G, N, K = 2, 2, 64, 1, 16, 4
    di, conv_dim = H * P, H * P + 2 * G * N
    row = torch.randn(Bsz, 2 * di + 2 * G * N + H, generator=g)
    cs0 = torch.randn(Bsz, conv_dim, K, generator=g)
    st0 = torch.randn(Bsz, H, P, N, generator=g)
    w = torch.rand(conv_dim, K, generator=g) - 0.5
    A = -torch.rand(H, generator=g) - 0.5
    Dhp = torch.randn(H, P, generator=g)
    # no bias, no softplus, no gate, D per channel
    z, xBC, dt = torch.split(row, [di, conv_dim, H], dim=-1)
    win = torch.roll(cs0, -1, dims=-1)
    win[..., -1] = xBC
    act = torch.nn.functional.silu((win * w).sum(-1))
    x, Bm, Cm = torch.split(act, [di, G * N, G * N], dim=-1)
    flat = st0.reshape(Bsz, di, N).clone()
    y_ref = O.selective_state_step(flat, x, dt.repeat_interleave(P, dim=-1), A.repeat_interleave(P)[:, None].expand(di, N),
                                   Bm.reshape(Bsz, G, N), Cm.reshape(Bsz, G, N), D=Dhp.reshape(di), z=None,
                                   dt_bias=None, softplus=False)
    cs, st = cs0.clone().cuda(), st0.clone().cuda()
    y = ops.mamba2_decode_step(row.cuda(), cs, st, w.cuda(), None, A.cuda(), D=Dhp.cuda(), dt_bias=None, ngroups=G,
                               softplus=False, gate=False)
    torch.testing.assert_close(y.cpu(), y_ref, **FP32_TOL)
    torch.testing.assert_close(st.cpu(), flat.reshape(Bsz, H, P, N), **FP32_TOL)
    with pytest.raises(ValueError):
        ops.mamba2_decode_step(row[:, :-1].cuda(), cs, st, w.cuda(), None, A.cuda())
    with pytest.raises(ValueError):
        ops.mamba2_decode_step(row.cuda(), cs.to(torch.bfloat16), st, w.cuda(), None, A.cuda())
    with pytest.raises(ValueError):
        ops.mamba2_decode_step(row.cuda(), cs, st.to(torch.bfloat16), w.cuda(), None, A.cuda())
    bad_n = torch.zeros(Bsz, H, P, 12, device="cuda")
    with pytest.raises((ValueError, RuntimeError)):
        ops.mamba2_decode_step(torch.zeros(Bsz, 2 * di + 24 + H, device="cuda"),
                               torch.zeros(Bsz, di + 24, K, device="cuda"), bad_n, torch.zeros(di + 24, K, device="cuda"),
                               None, A.cuda())


@pytest.mark.parametrize("io", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K,act", [(4, "silu"), (2, "identity"), (7, "silu"), (1, "silu")])
def test_conv_window_step_follows_the_full_convolution(io, K, act):
    """Feeding a sequence token by token through conv_window_step (window starting at zero) gives the
    columns of dw_causal_conv over the whole sequence; x is read in place from a wider matrix."""
    ops = _ops()
    g = torch.Generator().manual_seed(K)
    Bsz, Cn, L = 3, 70, 9
    wide = torch.randn(Bsz, L, Cn + 5, generator=g).to(io)
    w = torch.rand(Cn, K, generator=g) - 0.5
    cb = torch.randn(Cn, generator=g) * 0.1
    xs = wide[:, :, 2:2 + Cn]
    x32 = torch.nn.functional.pad(xs.float().transpose(1, 2), (K - 1, 0))
    full = torch.nn.functional.conv1d(x32, w[:, None], cb, groups=Cn)
    if act == "silu":
        full = torch.nn.functional.silu(full)
    state = torch.zeros(Bsz, Cn, K, dtype=io).cuda()
    wide_gpu = wide.cuda()
    for t in range(L):
        out = ops.conv_window_step(state, wide_gpu[:, t, 2:2 + Cn], w.cuda(), cb.cuda(), activation=act)
        assert out.dtype == io
        torch.testing.assert_close(out.float().cpu(), full[:, :, t], **(FP32_TOL if io == torch.float32 else HALF_TOL))
    torch.testing.assert_close(state.float().cpu(), x32[:, :, -K:], rtol=0, atol=0)
    with pytest.raises(ValueError):
        ops.conv_window_step(state, wide_gpu[:, 0, :Cn - 1], w.cuda(), cb.cuda())
    with pytest.raises(ValueError):
        ops.conv_window_step(state, wide_gpu[:, 0, :Cn], w.cuda(), cb.cuda(), activation="relu")


# ---------------------------------------------------------------------------
# backward: gradients of (y, new_state) against float64 autograd through the
# CPU restatement of the step
# ---------------------------------------------------------------------------

def _oracle_grads(inp, softplus, gy, gs):
    names = ["state", "x", "dt", "A", "B", "C", "D", "z", "dt_bias"]
    leaves = {k: (inp[k].double().clone().requires_grad_(True) if inp.get(k) is not None else None) for k in names}
    y, new_state = O.selective_state_step_functional(
        leaves["state"], leaves["x"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], D=leaves["D"],
        z=leaves["z"], dt_bias=leaves["dt_bias"], softplus=softplus, acc=torch.float64)
    loss = (y.double() * gy.double()).sum() + (new_state.double() * gs.double()).sum()
    loss.backward()
    return {k: (v.grad if v is not None else None) for k, v in leaves.items()}


@pytest.mark.parametrize("kinds", [("dn", "dn"), ("bdn", "bgn"), ("bgn", "bdn"), ("bgn", "bgn")])
@pytest.mark.parametrize("softplus", [True, False])
def test_backward_matches_float64_autograd(kinds, softplus):
    batch, dim, nstate, groups = 3, 8, 6, 2
    inp = make(23, batch, dim, nstate, bkind=kinds[0], ckind=kinds[1], groups=groups)
    if not softplus:
        inp["dt"] = inp["dt"].abs() * 0.1
        inp["dt_bias"] = inp["dt_bias"].abs() * 0.01
    g = torch.Generator().manual_seed(5)
    gy = torch.randn(batch, dim, generator=g)
    gs = torch.randn(batch, dim, nstate, generator=g)
    want = _oracle_grads(inp, softplus, gy, gs)
    got = _ops()._state_step_backward(dev(gy), dev(gs), dev(inp["state"]), dev(inp["x"]), dev(inp["dt"]), dev(inp["A"]),
                                      dev(inp["B"]), dev(inp["C"]), dev(inp["D"]), dev(inp["z"]), dev(inp["dt_bias"]),
                                      softplus)
    for name, gval in zip(["state", "x", "dt", "A", "B", "C", "D", "z", "dt_bias"], got):
        torch.testing.assert_close(gval.cpu().double().reshape(want[name].shape), want[name], rtol=1e-4, atol=1e-5,
                                   msg=lambda m, n=name: f"grad {n}: {m}")


def test_backward_without_optional_inputs_and_with_missing_upstream_grads():
    inp = make(29, 2, 5, 4, bkind="dn", ckind="bdn", use_D=False, use_z=False, use_bias=False)
    g = torch.Generator().manual_seed(6)
    gy = torch.randn(2, 5, generator=g)
    want = _oracle_grads(inp, True, gy, torch.zeros(2, 5, 4))
    got = _ops()._state_step_backward(dev(gy), None, dev(inp["state"]), dev(inp["x"]), dev(inp["dt"]), dev(inp["A"]),
                                      dev(inp["B"]), dev(inp["C"]), None, None, None, True)
    assert got[6] is None and got[7] is None and got[8] is None
    for name, gval in zip(["state", "x", "dt", "A", "B", "C"], got[:6]):
        torch.testing.assert_close(gval.cpu().double(), want[name], rtol=1e-4, atol=1e-5)


def test_autograd_through_two_steps_matches_oracle():
    """Back-propagation through time: two updates of the same state tensor."""
    batch, dim, nstate = 2, 6, 4
    a = make(31, batch, dim, nstate, bkind="bgn", ckind="bgn", groups=2)
    b = make(32, batch, dim, nstate, bkind="bgn", ckind="bgn", groups=2)
    ops = _ops()

    def leaves_of(to, dtype):
        return {k: to(a[k]).to(dtype).requires_grad_(True) for k in ["x", "dt", "A", "B", "C", "D", "z", "dt_bias"]}

    # float64 oracle, functional chaining of the state
    lw = leaves_of(lambda t: t, torch.float64)
    y1, s1 = O.selective_state_step_functional(a["state"].double(), lw["x"], lw["dt"], lw["A"], lw["B"], lw["C"],
                                               D=lw["D"], z=lw["z"], dt_bias=lw["dt_bias"], softplus=True,
                                               acc=torch.float64)
    y2, s2 = O.selective_state_step_functional(s1, b["x"].double(), b["dt"].double(), lw["A"], b["B"].double(),
                                               b["C"].double(), D=lw["D"], z=b["z"].double(), dt_bias=lw["dt_bias"],
                                               softplus=True, acc=torch.float64)
    (y1.sum() + 2.0 * y2.sum() + s2.sum()).backward()

    # GPU, the in-place API
    lg = leaves_of(dev, torch.float32)
    state = dev(a["state"]).clone()
    z1 = ops.selective_state_step(state, lg["x"], lg["dt"], lg["A"], lg["B"], lg["C"], D=lg["D"], z=lg["z"],
                                  dt_bias=lg["dt_bias"], softplus=True)
    z2 = ops.selective_state_step(state, dev(b["x"]), dev(b["dt"]), lg["A"], dev(b["B"]), dev(b["C"]), D=lg["D"],
                                  z=dev(b["z"]), dt_bias=lg["dt_bias"], softplus=True)
    (z1.sum() + 2.0 * z2.sum() + state.sum()).backward()
    torch.testing.assert_close(state.detach().cpu().double(), s2.detach(), rtol=1e-5, atol=1e-5)
    for k in lw:
        torch.testing.assert_close(lg[k].grad.cpu().double(), lw[k].grad, rtol=1e-4, atol=1e-5,
                                   msg=lambda m, n=k: f"grad {n}: {m}")


def test_repeated_step_of_one_form_goes_through_the_remembered_struct():
    """The second step of a form (same shapes, element types, optional arguments) skips the validation and fills a
    remembered argument struct: the same bits as a prepared plan on the same values, new tensors each time; a call
    whose tensors need a copy first, and a form never seen, still go the long way."""
    from ssm_amd import ops
    g = torch.Generator().manual_seed(8)
    batch, dim, nstate = 4, 96, 16
    A = (-(torch.rand(dim, nstate, generator=g) + 0.5)).cuda()
    D, bias = torch.randn(dim, generator=g).cuda(), torch.randn(dim, generator=g).cuda()
    def token(seed):
        h = torch.Generator().manual_seed(seed)
        x, dt, z = (torch.randn(batch, dim, generator=h).to(torch.bfloat16).cuda() for _ in range(3))
        Bm, Cm = (torch.randn(batch, 1, nstate, generator=h).to(torch.bfloat16).cuda() for _ in range(2))
        return x, dt, z, Bm, Cm
    ops._STEP_FORMS.clear()
    state, ref_state = torch.zeros(batch, dim, nstate).cuda(), torch.zeros(batch, dim, nstate).cuda()
    for step in range(4):
        x, dt, z, Bm, Cm = token(step)
        y = ops.selective_state_step(state, x, dt, A, Bm, Cm, D, z=z, dt_bias=bias, softplus=True)
        assert len(ops._STEP_FORMS) == 1
        want = ops.StepPlan(ref_state, x, dt, A, Bm, Cm, D, z, bias, True).run()
        assert torch.equal(y, want) and torch.equal(state, ref_state), step
    x, dt, z, Bm, Cm = token(9)
    y = ops.selective_state_step(state, x.t().contiguous().t(), dt, A, Bm, Cm, D, z=z, dt_bias=bias, softplus=True)
    want = ops.StepPlan(ref_state, x, dt, A, Bm, Cm, D, z, bias, True).run()
    assert torch.equal(y, want) and torch.equal(state, ref_state)
    with pytest.raises(ValueError):
        ops.selective_state_step(state, x, dt, A[:, :8].contiguous(), Bm, Cm, D, z=z, dt_bias=bias, softplus=True)

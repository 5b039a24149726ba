"""GPU parity of the selective-scan backward pass: gradients from the HIP
kernels against autograd through the CPU oracle (fp32 and fp64) and against
the upstream-CUDA gradient vectors."""

import pytest
import torch

from oracle import ops_oracle as O
from tests import fixtures as fx
from tests.test_scan_fwd_gpu import make_inputs

pytestmark = pytest.mark.gpu

NAMES = ("u", "delta", "A", "B", "C", "D", "z", "dt_bias")


def _ops():
    from ssm_amd import ops
    return ops


def grads_both(inp, softplus=True, with_last=False, acc=None, seed=5):
    g = torch.Generator().manual_seed(seed)
    go = torch.randn(inp["u"].shape, generator=g).to(inp["u"].dtype)
    gl = torch.randn(inp["u"].shape[0], inp["u"].shape[1], inp["A"].shape[1], generator=g).to(inp["u"].dtype)
    res = []
    for where in ("gpu", "cpu"):
        leaves = {}
        for k in NAMES:
            v = inp[k]
            if v is None:
                leaves[k] = None
                continue
            v = v.clone()
            if where == "gpu":
                v = v.cuda()
            leaves[k] = v.requires_grad_(True)
        kw = dict(D=leaves["D"], z=leaves["z"], dt_bias=leaves["dt_bias"], softplus=softplus,
                  return_last_state=with_last)
        if where == "gpu":
            out = _ops().selective_scan(leaves["u"], leaves["delta"], leaves["A"], leaves["B"], leaves["C"], **kw)
        else:
            out = O.selective_scan(leaves["u"], leaves["delta"], leaves["A"], leaves["B"], leaves["C"], acc=acc, **kw)
        dev = "cuda" if where == "gpu" else "cpu"
        if with_last:
            y, last = out
            loss = (y.float() * go.to(dev).float()).sum() + (last.float() * gl.to(dev).float()).sum()
        else:
            loss = (out.float() * go.to(dev).float()).sum()
        loss.backward()
        res.append({k: (leaves[k].grad.detach().cpu() if leaves[k] is not None else None) for k in NAMES})
    return res


def compare(got, want, rtol, atol, scale_atol=True):
    for k in NAMES:
        if want[k] is None:
            assert got[k] is None
            continue
        w = want[k].float()
        a = atol * max(1.0, float(w.abs().max())) if scale_atol else atol
        torch.testing.assert_close(got[k].float(), w, rtol=rtol, atol=a, msg=lambda m, k=k: f"grad {k}: {m}")


@pytest.mark.parametrize("case,softplus", [("full", True), ("minimal", False), ("time_varying_3d", True)])
def test_upstream_gradient_vectors(case, softplus):
    rec = fx.upstream("selective_scan", case)
    i = rec["inputs"]
    Bm, Cm = i["B"], i["C"]
    if case == "time_varying_3d":
        Bm, Cm = Bm[:, None].contiguous(), Cm[:, None].contiguous()
    leaves = dict(u=i["u"], delta=i["delta"], A=i["A"], B=Bm, C=Cm, D=i.get("D"), z=i.get("z"),
                  dt_bias=i.get("delta_bias"))
    leaves = {k: (v.clone().cuda().requires_grad_(True) if v is not None else None) for k, v in leaves.items()}
    y = _ops().selective_scan(leaves["u"], leaves["delta"], leaves["A"], leaves["B"], leaves["C"], D=leaves["D"],
                              z=leaves["z"], dt_bias=leaves["dt_bias"], softplus=softplus)
    y.sum().backward()
    for name, gref in rec["gradients"].items():
        if gref is None:
            continue
        key = "dt_bias" if name == "delta_bias" else name
        got = leaves[key].grad.cpu()
        if case == "time_varying_3d" and name in ("B", "C"):
            got = got[:, 0]
        ok = torch.isfinite(gref)
        if ok.any():
            torch.testing.assert_close(got[ok], gref[ok], rtol=2e-4, atol=2e-5)


SHAPES = [(1, 1, 1, 1), (2, 3, 5, 4), (2, 8, 64, 16), (1, 4, 65, 3), (3, 6, 513, 16), (2, 32, 1024, 16),
          (1, 8, 1500, 7), (2, 4, 300, 40)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("kinds", [("bgnl", "bgnl"), ("dn", "dn"), ("bdn", "bgnl"), ("bgnl", "dn")])
def test_fp32_gradients_match_oracle(shape, kinds):
    b, d, l, n = shape
    inp = make_inputs(sum(shape), b, d, l, n, bkind=kinds[0], ckind=kinds[1])
    got, want = grads_both(inp)
    compare(got, want, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("shape,with_last", [((2, 32, 1024, 16), False), ((3, 6, 513, 16), True), ((1, 48, 2048, 16), False)],
                         ids=lambda v: str(v).replace(" ", ""))
def test_fp32_gradient_error_is_that_of_fp32_arithmetic(shape, with_last):
    """Which of two float32 results is right is settled by float64: for each of the eight gradients the kernel's
    error against the float64 oracle must not exceed four times the float32 oracle's own error against it (plus
    one part in a million of the gradient's size, for gradients the float32 oracle happens to hit exactly)."""
    b, d, l, n = shape
    inp = make_inputs(sum(shape) + 1, b, d, l, n)
    got, want32 = grads_both(inp, with_last=with_last)
    _, want64 = grads_both(inp, with_last=with_last, acc=torch.float64)
    for k in NAMES:
        if want64[k] is None:
            continue
        w64 = want64[k].double()
        ours = float((got[k].double() - w64).abs().max())
        theirs = float((want32[k].double() - w64).abs().max())
        floor = 1e-6 * float(w64.abs().max())
        assert ours <= 4.0 * theirs + floor, f"grad {k}: kernel error {ours:.3e}, float32 oracle error {theirs:.3e}"


@pytest.mark.parametrize("groups,dim", [(1, 8), (2, 8), (8, 8), (3, 6), (2, 96)])
def test_groups(groups, dim):
    inp = make_inputs(4, 2, dim, 200, 16, groups=groups)
    got, want = grads_both(inp)
    compare(got, want, rtol=1e-4, atol=2e-5)


def test_gradient_of_last_state():
    inp = make_inputs(6, 2, 8, 700, 16)
    got, want = grads_both(inp, with_last=True)
    compare(got, want, rtol=1e-4, atol=2e-5)


@pytest.mark.parametrize("use_D,use_z,use_bias,softplus", [(False, False, False, False), (True, False, True, True),
                                                           (False, True, False, True)])
def test_optional_arguments(use_D, use_z, use_bias, softplus):
    inp = make_inputs(3, 2, 4, 130, 8, use_D=use_D, use_z=use_z, use_bias=use_bias)
    if not softplus:
        inp["delta"] = inp["delta"].abs() * 0.1
    got, want = grads_both(inp, softplus=softplus)
    compare(got, want, rtol=1e-4, atol=2e-5)


def test_only_requested_inputs_get_gradients():
    inp = make_inputs(2, 1, 4, 40, 4)
    g = {k: (v.cuda() if v is not None else None) for k, v in inp.items()}
    g["u"].requires_grad_(True); g["A"].requires_grad_(True)
    y = _ops().selective_scan(g["u"], g["delta"], g["A"], g["B"], g["C"], D=g["D"], z=g["z"],
                              dt_bias=g["dt_bias"], softplus=True)
    y.sum().backward()
    assert g["u"].grad is not None and g["A"].grad is not None
    assert g["delta"].grad is None and g["B"].grad is None and g["z"].grad is None


def test_against_float64_oracle_and_bitwise_determinism():
    inp = make_inputs(9, 2, 16, 1024, 16)
    got, want64 = grads_both(inp, acc=torch.float64)
    compare(got, want64, rtol=2e-4, atol=2e-5)
    again, _ = grads_both(inp, acc=torch.float64)
    for k in NAMES:
        assert torch.equal(got[k], again[k]), k


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_half_inputs(dtype):
    inp = make_inputs(8, 2, 16, 600, 16, dtype=dtype)
    got, want = grads_both(inp)
    for k in ("u", "delta", "z", "B", "C"):
        assert got[k].dtype == dtype
    for k in ("A", "D", "dt_bias"):
        assert got[k].dtype == torch.float32
    # the oracle differentiates the same 16-bit inputs in fp32; outputs are rounded once
    from tests.closeness import half_close
    for k in NAMES:
        half_close(got[k], want[k], what=f"grad {k}", atol_rms=4e-2, mean_rms=5e-3)


def test_config1_shape_bf16_slice():
    """B=8, D=1536, L=2048, N=16, bf16, G=1: full-size backward on the GPU.  du, ddelta
    and the parameter gradients of a channel slice are compared with the oracle run on
    that slice; dB/dC (sums over all 1536 channels) are checked through linearity: the
    gradient of the full problem equals the sum of the gradients of two channel halves."""
    ops = _ops()
    inp = make_inputs(1, 8, 1536, 2048, 16, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(11)
    go = torch.randn(8, 1536, 2048, generator=g).to(torch.bfloat16)

    def run(sl):
        lv = {}
        for k in NAMES:
            v = inp[k]
            if k in ("u", "delta", "z"):
                v = v[:, sl]
            elif k in ("A", "D", "dt_bias"):
                v = v[sl]
            lv[k] = v.contiguous().cuda().requires_grad_(True)
        y = ops.selective_scan(lv["u"], lv["delta"], lv["A"], lv["B"], lv["C"], D=lv["D"], z=lv["z"],
                               dt_bias=lv["dt_bias"], softplus=True)
        y.backward(go[:, sl].contiguous().cuda())
        return {k: lv[k].grad for k in NAMES}

    full = run(slice(0, 1536))
    lo, hi = run(slice(0, 768)), run(slice(768, 1536))
    from tests.closeness import half_close
    for k in ("B", "C"):
        s = lo[k].float() + hi[k].float()          # three roundings to bf16 against one
        half_close(full[k], s, what=f"grad {k}: whole call against the sum of two halves", atol_rms=4e-2, mean_rms=8e-3)
    # a row's sums over the states run in an order that depends on the wave that owns the row, and the block shape
    # follows the channel count: the same row in the two calls agrees to one rounding of the 16-bit result
    a, b = full["u"][:, :768].float(), lo["u"].float()
    torch.testing.assert_close(a, b, rtol=2 ** -7, atol=1e-6 * float(b.abs().max()))
    assert float((a != b).float().mean()) < 1e-3
    # slice of 8 channels against the oracle
    idx = torch.arange(0, 1536, 192)
    sub = {k: (inp[k][:, idx] if k in ("u", "delta", "z") else inp[k][idx] if k in ("A", "D", "dt_bias") else inp[k])
           for k in NAMES}
    lv = {k: v.clone().requires_grad_(True) for k, v in sub.items()}
    y = O.selective_scan(lv["u"], lv["delta"], lv["A"], lv["B"], lv["C"], D=lv["D"], z=lv["z"],
                         dt_bias=lv["dt_bias"], softplus=True)
    y.backward(go[:, idx])
    for k in ("u", "delta", "z"):
        half_close(full[k][:, idx.cuda()], lv[k].grad, what=f"grad {k}", atol_rms=4e-2, mean_rms=5e-3)
    for k in ("A", "D", "dt_bias"):
        half_close(full[k][idx.cuda()], lv[k].grad, what=f"grad {k}", atol_rms=4e-2, mean_rms=5e-3)


# ------------------------------------------------------------------ the specialised kernel (16-bit activations)

def _bwd_direct(inp, go, gl, tune_items):
    from ssm_amd import ops
    dev = {k: (v.cuda() if v is not None else None) for k, v in inp.items()}
    return ops._scan_backward(go.cuda(), None if gl is None else gl.cuda(), dev["u"], dev["delta"], dev["A"], dev["B"],
                              dev["C"], dev["D"], dev["z"], dev["dt_bias"], True, tune_items=tune_items)


@pytest.mark.parametrize("shape,groups,use_z,with_last", [
    ((2, 48, 1040, 16), 1, True, True), ((1, 96, 512, 16), 2, True, False), ((2, 32, 1536, 9), 1, False, True),
    ((1, 16, 72, 16), 1, True, False), ((3, 48, 2048, 16), 3, True, False)], ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("dtype,bc_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32),
                                            (torch.float32, torch.float32)])
def test_specialised_backward_matches_general_kernel_and_oracle(shape, groups, use_z, with_last, dtype, bc_dtype):
    """Time-varying grouped B/C, groups that 16-channel blocks tile: the wave-per-row kernel
    (all states in turn, dB/dC summed in LDS under a skew) against the general kernel on the same inputs (both
    compute in float32 from the same 16-bit values: they agree to float32 rounding where the outputs are float32 and
    to one 16-bit rounding elsewhere) and against float64 autograd through the oracle."""
    b, d, l, n = shape
    inp = make_inputs(sum(shape), b, d, l, n, dtype=dtype, bc_dtype=bc_dtype, groups=groups, use_z=use_z)
    g = torch.Generator().manual_seed(3)
    go = torch.randn(b, d, l, generator=g).to(dtype)
    gl = torch.randn(b, d, n, generator=g) if with_last else None
    fast = _bwd_direct(inp, go, gl, 0)
    gen = _bwd_direct(inp, go, gl, 1)
    names = ("u", "delta", "A", "B", "C", "D", "z", "dt_bias")
    for k, f, r in zip(names, fast, gen):
        if r is None:
            assert f is None, k
            continue
        f, r = f.float().cpu(), r.float().cpu()
        scale = float(r.abs().max()) + 1e-30
        if k in ("u", "delta", "z") and dtype != torch.float32:
            torch.testing.assert_close(f, r, rtol=2e-2, atol=1e-3 * scale, msg=lambda m, k=k: f"grad {k} vs general kernel: {m}")
        else:
            torch.testing.assert_close(f, r, rtol=2e-4, atol=2e-5 * scale, msg=lambda m, k=k: f"grad {k} vs general kernel: {m}")
    # float64 autograd through the oracle on the same 16-bit values
    w = {k: (None if v is None else v.double().requires_grad_(True)) for k, v in inp.items()}
    out = O.selective_scan(w["u"], w["delta"], w["A"], w["B"], w["C"], D=w["D"], z=w["z"], dt_bias=w["dt_bias"],
                           softplus=True, return_last_state=with_last, acc=torch.float64)
    if with_last:
        ((out[0] * go.double()).sum() + (out[1] * gl.double()).sum()).backward()
    else:
        (out * go.double()).sum().backward()
    for k, f in zip(names, fast):
        if w[k] is None:
            continue
        want = w[k].grad
        scale = float(want.abs().max()) + 1e-30
        half = k in ("u", "delta", "z") and dtype != torch.float32
        tol = dict(rtol=2e-2, atol=4e-3 * scale) if half else dict(rtol=1e-3, atol=1e-4 * scale)
        torch.testing.assert_close(f.double().cpu(), want, **tol, msg=lambda m, k=k: f"grad {k} vs float64: {m}")


@pytest.mark.parametrize("shape,use_z,with_last", [((2, 24, 1040, 16), True, True), ((1, 7, 512, 16), True, False),
                                                   ((2, 5, 1536, 9), False, True), ((3, 10, 72, 4), True, False)],
                         ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("dtype,bc_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32),
                                            (torch.float32, torch.float32)])
def test_per_channel_projections_backward(shape, use_z, with_last, dtype, bc_dtype):
    """``B`` and ``C`` of shape ``(B, D, N, L)``, the reference Mamba1 module's own call
    (/root/reference/src/ssm/modules/mamba1.py:229-246): the wave-per-row kernel that writes ``dB`` and ``dC`` straight
    to their place, against the general kernel (test-hooks selector 1) and float64 autograd through the oracle, and
    through autograd with ``dB`` / ``dC`` written in the projections' own type."""
    b, d, l, n = shape
    inp = make_inputs(sum(shape) + 1, b, d, l, n, dtype=dtype, bc_dtype=bc_dtype, groups=d, use_z=use_z)
    g = torch.Generator().manual_seed(5)
    go = torch.randn(b, d, l, generator=g).to(dtype)
    gl = torch.randn(b, d, n, generator=g) if with_last else None
    fast = _bwd_direct(inp, go, gl, 0)
    gen = _bwd_direct(inp, go, gl, 1)
    names = ("u", "delta", "A", "B", "C", "D", "z", "dt_bias")
    for k, f, r in zip(names, fast, gen):
        if r is None:
            assert f is None, k
            continue
        assert f.dtype == r.dtype and f.shape == r.shape, k
        f, r = f.float().cpu(), r.float().cpu()
        scale = float(r.abs().max()) + 1e-30
        if k in ("u", "delta", "z") and dtype != torch.float32:
            torch.testing.assert_close(f, r, rtol=2e-2, atol=1e-3 * scale, msg=lambda m, k=k: f"grad {k} vs general kernel: {m}")
        else:
            torch.testing.assert_close(f, r, rtol=2e-4, atol=2e-5 * scale, msg=lambda m, k=k: f"grad {k} vs general kernel: {m}")
    w = {k: (None if v is None else v.double().requires_grad_(True)) for k, v in inp.items()}
    out = O.selective_scan(w["u"], w["delta"], w["A"], w["B"], w["C"], D=w["D"], z=w["z"], dt_bias=w["dt_bias"],
                           softplus=True, return_last_state=with_last, acc=torch.float64)
    if with_last:
        ((out[0] * go.double()).sum() + (out[1] * gl.double()).sum()).backward()
    else:
        (out * go.double()).sum().backward()
    # through autograd: dB and dC arrive in the projections' type, written so by the kernel
    lv = {k: (None if v is None else v.cuda().requires_grad_(True)) for k, v in inp.items()}
    res = _ops().selective_scan(lv["u"], lv["delta"], lv["A"], lv["B"], lv["C"], D=lv["D"], z=lv["z"],
                                dt_bias=lv["dt_bias"], softplus=True, return_last_state=with_last)
    if with_last:
        ((res[0].float() * go.cuda().float()).sum() + (res[1].float() * gl.cuda()).sum()).backward()
    else:
        (res.float() * go.cuda().float()).sum().backward()
    for k, f in zip(names, fast):
        if w[k] is None:
            continue
        want = w[k].grad
        scale = float(want.abs().max()) + 1e-30
        half = k in ("u", "delta", "z") and dtype != torch.float32
        tol = dict(rtol=2e-2, atol=4e-3 * scale) if half else dict(rtol=1e-3, atol=1e-4 * scale)
        torch.testing.assert_close(f.double().cpu(), want, **tol, msg=lambda m, k=k: f"grad {k} vs float64: {m}")
        ga = lv[k].grad
        assert ga.dtype == lv[k].dtype and ga.shape == lv[k].shape, k
        half_a = half or (k in ("B", "C") and bc_dtype != torch.float32)
        tol = dict(rtol=2e-2, atol=4e-3 * scale) if half_a else dict(rtol=1e-3, atol=1e-4 * scale)
        torch.testing.assert_close(ga.double().cpu(), want, **tol, msg=lambda m, k=k: f"autograd grad {k} vs float64: {m}")


def test_per_channel_projections_backward_needs_no_partial_sums():
    """The call's workspace holds the per-row sums of dA, dD and the bias only (the general kernel would need a
    float32 copy of dB and dC on top)."""
    from ssm_amd import _lib
    b, d, l, n = 2, 24, 1024, 16
    lib = _lib.load()
    general = lib.ssm_scan_bwd_workspace_bytes(b, d, l, n, _lib.PROJ_BGNL, _lib.PROJ_BGNL, d, d)
    x = torch.zeros(b, d, l, device="cuda")
    p = torch.zeros(b, d, n, l, device="cuda")
    args = _lib.ScanBwdArgs(u=x.data_ptr(), delta=x.data_ptr(), dout=x.data_ptr(), du=x.data_ptr(), ddelta=x.data_ptr(),
                            Bproj=p.data_ptr(), Cproj=p.data_ptr(), dB=p.data_ptr(), dC=p.data_ptr(), batch=b, dim=d, seqlen=l,
                            nstate=n, io_dtype=_lib.SSM_F32, bc_dtype=_lib.SSM_F32, b_kind=_lib.PROJ_BGNL, c_kind=_lib.PROJ_BGNL,
                            b_groups=d, c_groups=d)
    direct = lib.ssm_scan_bwd_per_row_workspace_bytes(args)
    assert 0 < direct <= 4 * b * d * (n + 2) + 3 * 256 and general >= 2 * 4 * b * d * n * l
    args.b_groups = args.c_groups = 1            # one group for all channels: not such a call
    assert lib.ssm_scan_bwd_per_row_workspace_bytes(args) == 0


def test_specialised_backward_is_bit_reproducible():
    inp = make_inputs(11, 2, 48, 1040, 16, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(4)
    go = torch.randn(2, 48, 1040, generator=g).to(torch.bfloat16)
    first = _bwd_direct(inp, go, None, 0)
    for _ in range(3):
        again = _bwd_direct(inp, go, None, 0)
        for a, b in zip(first, again):
            assert (a is None and b is None) or torch.equal(a, b)


def test_a_wave_that_gives_up_its_wait_poisons_dB_and_dC():
    """The wave-per-row kernel bounds its wait for the neighbouring wave's slot count; a wave that gives up
    writes NaN into its sums so that the caller cannot take them for gradients.  The test-hooks build cuts the
    bound to nothing (selector 2, include/ssm_amd_testing.h), so every wave gives up at once: the kernel still ends
    normally, dB and dC come back NaN, and the gradients that do not pass through the shared tiles are those of
    an ordinary call."""
    inp = make_inputs(12, 2, 48, 1040, 16, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(5)
    go = torch.randn(2, 48, 1040, generator=g).to(torch.bfloat16)
    good = _bwd_direct(inp, go, None, 0)
    bad = _bwd_direct(inp, go, None, 2)
    torch.cuda.synchronize()
    names = ("u", "delta", "A", "B", "C", "D", "z", "dt_bias")
    for k, a, b in zip(names, good, bad):
        if a is None:
            continue
        if k in ("B", "C"):
            assert bool(torch.isnan(b).any()), f"grad {k} must be poisoned"
            assert not bool(torch.isnan(a).any())
        else:
            assert torch.equal(a, b), k


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_conv_then_scan_forward_and_backward(dtype):
    """The step that configuration 1 times (conv, SiLU, scan with gate, skip and softplus; forward and backward
    through autograd) on a shape the oracle differentiates in seconds: gradients reach the conv's input, taps
    and bias through the scan's gradient of ``u``."""
    ops = _ops()
    inp = make_inputs(21, 2, 32, 300, 16, dtype=dtype)
    g = torch.Generator().manual_seed(22)
    x = torch.randn(2, 32, 300, generator=g).to(dtype)
    w, b = torch.rand(32, 4, generator=g) - 0.5, torch.randn(32, generator=g) * 0.02
    go = torch.randn(2, 32, 300, generator=g).to(dtype)
    names = ("x", "w", "b") + tuple(k for k in NAMES if k != "u")

    def run(where, acc):
        # the float64 value of the chain: the same inputs widened, so that nothing in between is rounded to float32
        put = (lambda t: t.cuda()) if where == "gpu" else ((lambda t: t.double()) if acc is not None else (lambda t: t))
        lv = dict(x=x, w=w, b=b, **{k: inp[k] for k in NAMES if k != "u"})
        lv = {k: put(v.detach().clone()).requires_grad_(True) for k, v in lv.items()}
        if where == "gpu":
            u = ops.dw_causal_conv(lv["x"], lv["w"], lv["b"], activation="silu")
            y = ops.selective_scan(u, lv["delta"], lv["A"], lv["B"], lv["C"], D=lv["D"], z=lv["z"],
                                   dt_bias=lv["dt_bias"], softplus=True)
        else:
            u = O.dw_causal_conv(lv["x"], lv["w"], lv["b"], activation="silu")
            y = O.selective_scan(u, lv["delta"], lv["A"], lv["B"], lv["C"], D=lv["D"], z=lv["z"],
                                 dt_bias=lv["dt_bias"], softplus=True)
        y.backward(put(go).to(y.dtype))
        return y.detach().cpu(), {k: lv[k].grad.detach().cpu() for k in names}

    y, got = run("gpu", None)
    from tests.closeness import fp32_close, half_close
    if dtype == torch.float32:
        y64, want64 = run("cpu", torch.float64)
        y32, want32 = run("cpu", None)
        fp32_close(y, y64, y32, what="y")
        for k in names:
            fp32_close(got[k], want64[k], want32[k], what=f"grad {k}")
    else:
        # the 16-bit path rounds the conv's output once before the scan reads it, as the oracle's chain does
        yr, want = run("cpu", None)
        half_close(y, yr, what="y")
        for k in names:
            half_close(got[k], want[k], what=f"grad {k}", atol_rms=4e-2, mean_rms=5e-3)


@pytest.mark.parametrize("shape,bkind,ckind,use_z,with_last", [
    ((2, 48, 1040, 16), "dn", "dn", True, True), ((1, 96, 512, 16), "bdn", "bdn", True, False),
    ((2, 32, 1536, 9), "dn", "bdn", False, True), ((1, 16, 72, 16), "bdn", "dn", True, False),
    ((3, 40, 2048, 16), "dn", "dn", True, False), ((1, 16, 1600, 16), "bdn", "dn", True, True),
    ((1, 8, 3712, 5), "dn", "dn", False, False)], ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("dtype,bc_dtype", [(torch.bfloat16, torch.float32), (torch.float16, torch.float16),
                                            (torch.float32, torch.float32)])
def test_constant_projections_backward(shape, bkind, ckind, use_z, with_last, dtype, bc_dtype):
    """``B`` and ``C`` of shape ``(D, N)`` or ``(B, D, N)`` (the reference's other accepted forms,
    /root/reference/src/ssm/ops/python/reference.py:22-56): the wave-per-row kernel with the projections and their
    sums in lanes, against the general kernel on the same inputs (test-hooks selector 1) and against float64 autograd
    through the oracle.  Sequences that fill chunks of 1024 steps (2048; 1600 and 3712 with a ragged last chunk) take
    the 16-steps-per-lane form, the others 8."""
    b, d, l, n = shape
    inp = make_inputs(sum(shape) + 2, b, d, l, n, dtype=dtype, bc_dtype=bc_dtype, bkind=bkind, ckind=ckind, use_z=use_z)
    g = torch.Generator().manual_seed(6)
    go = torch.randn(b, d, l, generator=g).to(dtype)
    gl = torch.randn(b, d, n, generator=g) if with_last else None
    fast = _bwd_direct(inp, go, gl, 0)
    gen = _bwd_direct(inp, go, gl, 1)
    names = ("u", "delta", "A", "B", "C", "D", "z", "dt_bias")
    for k, f, r in zip(names, fast, gen):
        if r is None:
            assert f is None, k
            continue
        assert f.dtype == r.dtype and f.shape == r.shape, k
        f, r = f.float().cpu(), r.float().cpu()
        scale = float(r.abs().max()) + 1e-30
        if k in ("u", "delta", "z") and dtype != torch.float32:
            torch.testing.assert_close(f, r, rtol=2e-2, atol=1e-3 * scale, msg=lambda m, k=k: f"grad {k} vs general kernel: {m}")
        else:
            torch.testing.assert_close(f, r, rtol=2e-4, atol=2e-5 * scale, msg=lambda m, k=k: f"grad {k} vs general kernel: {m}")
    w = {k: (None if v is None else v.double().requires_grad_(True)) for k, v in inp.items()}
    out = O.selective_scan(w["u"], w["delta"], w["A"], w["B"], w["C"], D=w["D"], z=w["z"], dt_bias=w["dt_bias"],
                           softplus=True, return_last_state=with_last, acc=torch.float64)
    if with_last:
        ((out[0] * go.double()).sum() + (out[1] * gl.double()).sum()).backward()
    else:
        (out * go.double()).sum().backward()
    for k, f in zip(names, fast):
        if w[k] is None:
            continue
        want = w[k].grad
        scale = float(want.abs().max()) + 1e-30
        half = k in ("u", "delta", "z") and dtype != torch.float32
        tol = dict(rtol=2e-2, atol=4e-3 * scale) if half else dict(rtol=1e-3, atol=1e-4 * scale)
        torch.testing.assert_close(f.double().cpu(), want, **tol, msg=lambda m, k=k: f"grad {k} vs float64: {m}")

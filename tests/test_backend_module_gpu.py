"""``ssm_amd.backend_module``: each of the ten functions the reference's façade calls on its compiled backend,
invoked with exactly the positional lists of the façade's call sites (src/ssm/ops/__init__.py of the reference:
autograd wrappers :317, :447, :595, :653, :809, :868, :978, :1017, :1148, :1204; direct calls :1289, :1395, :1516,
:1594, :1640), checked against the CPU oracle (forward) and autograd through the oracle (backward)."""

import pytest
import torch

from oracle import ops_oracle as O

pytestmark = pytest.mark.gpu

TOL = dict(rtol=1e-4, atol=2e-5)


def backend():
    from ssm_amd import backend_module
    return backend_module.load()


def cu(t):
    return None if t is None else t.cuda()


def leaves(d):
    return {k: (None if v is None else v.clone().requires_grad_(True)) for k, v in d.items()}


def close(got, want, what, scale=True):
    if want is None:
        assert got is None, what
        return
    a = TOL["atol"] * (max(1.0, float(want.abs().max())) if scale else 1.0)
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=TOL["rtol"], atol=a, msg=lambda m: f"{what}: {m}")


def scan_inputs(seed=0, b=2, d=8, l=600, n=16):
    g = torch.Generator().manual_seed(seed)
    return dict(u=torch.randn(b, d, l, generator=g), delta=torch.randn(b, d, l, generator=g),
                A=-(torch.rand(d, n, generator=g) * 4 + 0.5), B=torch.randn(b, 2, n, l, generator=g),
                C=torch.randn(b, 2, n, l, generator=g), D=torch.randn(d, generator=g),
                z=torch.randn(b, d, l, generator=g), dt_bias=torch.randn(d, generator=g) - 3.0)


def test_selective_scan_and_backward():
    be = backend()
    assert be.available and be.name == "hip"
    i = scan_inputs()
    # :317-329 / :1289-1303
    out = be.selective_scan(cu(i["u"]), cu(i["delta"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), cu(i["D"]), cu(i["z"]),
                            cu(i["dt_bias"]), True, True)
    y, last, cache = out
    w = leaves(i)
    yr, lr = O.selective_scan(w["u"], w["delta"], w["A"], w["B"], w["C"], D=w["D"], z=w["z"], dt_bias=w["dt_bias"],
                              softplus=True, return_last_state=True)
    close(y, yr.detach(), "y")
    close(last, lr.detach(), "last_state")
    assert cache.dtype == torch.float32 and tuple(cache.shape) == (2, 8, 2, 16)
    g = torch.Generator().manual_seed(9)
    go, gl = torch.randn(yr.shape, generator=g), torch.randn(lr.shape, generator=g)
    ((yr * go).sum() + (lr * gl).sum()).backward()
    # :447-462
    grads = be.selective_scan_backward(cu(go), cu(gl), cu(i["u"]), cu(i["delta"]), cu(i["A"]), cu(i["B"]), cu(i["C"]),
                                       cu(i["D"]), cu(i["z"]), cu(i["dt_bias"]), True, y, cache)
    assert len(grads) == 8
    for k, gk in zip(("u", "delta", "A", "B", "C", "D", "z", "dt_bias"), grads):
        assert gk.shape == i[k].shape and gk.dtype == i[k].dtype
        close(gk, w[k].grad, f"grad {k}")
    # without optional inputs, without last state, without cache
    y2, last2, _ = be.selective_scan(cu(i["u"]), cu(i["delta"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), None, None, None,
                                     True, False)
    assert last2 is None
    close(y2, O.selective_scan(i["u"], i["delta"], i["A"], i["B"], i["C"], softplus=True), "y without options")
    g2 = be.selective_scan_backward(cu(go), None, cu(i["u"]), cu(i["delta"]), cu(i["A"]), cu(i["B"]), cu(i["C"]),
                                    None, None, None, True, y2, None)
    assert g2[5] is None and g2[6] is None and g2[7] is None and g2[0] is not None


def test_selective_state_step_and_backward():
    be = backend()
    g = torch.Generator().manual_seed(1)
    b, d, n = 3, 12, 16
    i = dict(state=torch.randn(b, d, n, generator=g), x=torch.randn(b, d, generator=g), dt=torch.randn(b, d, generator=g),
             A=-(torch.rand(d, n, generator=g) + 0.5), B=torch.randn(b, 1, n, generator=g), C=torch.randn(b, 1, n, generator=g),
             D=torch.randn(d, generator=g), z=torch.randn(b, d, generator=g), dt_bias=torch.randn(d, generator=g) - 2.0)
    state = cu(i["state"]).clone()
    # :595-607 / :1395-1408
    y = be.selective_state_step(state, cu(i["x"]), cu(i["dt"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), cu(i["D"]), cu(i["z"]),
                                cu(i["dt_bias"]), True)
    w = leaves(i)
    yr, new_state = O.selective_state_step_functional(w["state"], w["x"], w["dt"], w["A"], w["B"], w["C"], D=w["D"],
                                                      z=w["z"], dt_bias=w["dt_bias"], softplus=True)
    close(y, yr.detach(), "y")
    close(state, new_state.detach(), "state updated in place")
    go, gs = torch.randn(yr.shape, generator=g), torch.randn(new_state.shape, generator=g)
    ((yr * go).sum() + (new_state * gs).sum()).backward()
    # :653-667
    grads = be.selective_state_step_backward(cu(go), cu(gs), cu(i["state"]), cu(i["x"]), cu(i["dt"]), cu(i["A"]),
                                             cu(i["B"]), cu(i["C"]), cu(i["D"]), cu(i["z"]), cu(i["dt_bias"]), True)
    assert len(grads) == 9
    for k, gk in zip(("state", "x", "dt", "A", "B", "C", "D", "z", "dt_bias"), grads):
        assert gk.shape == i[k].shape
        close(gk, w[k].grad, f"grad {k}")


def test_ssd_chunk_scan_and_backward():
    be = backend()
    g = torch.Generator().manual_seed(2)
    b, l, h, p = 2, 70, 3, 8
    i = dict(X=torch.randn(b, l, h, p, generator=g), dt=torch.rand(b, l, h, generator=g) * 0.2,
             A=-(torch.rand(h, p, generator=g) + 0.2), B=torch.randn(b, l, h, p, generator=g),
             C=torch.randn(b, h, p, generator=g), D=torch.randn(h, generator=g), z=torch.randn(b, l, h, generator=g),
             init=torch.randn(b, h, p, generator=g))
    seq_lens = torch.tensor([70, 41], dtype=torch.int64)
    # :809-822 / :1516-1531
    Y = be.ssd_chunk_scan(cu(i["X"]), cu(i["dt"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), 16, cu(i["D"]), cu(i["z"]),
                          cu(seq_lens), None, cu(i["init"]))
    w = leaves(i)
    Yr = O.ssd_chunk_scan(w["X"], w["dt"], w["A"], w["B"], w["C"], 16, D=w["D"], z=w["z"],
                          seq_meta={"seq_lens": seq_lens}, initial_states=w["init"])
    close(Y, Yr.detach(), "Y")
    go = torch.randn(Yr.shape, generator=g)
    (Yr * go).sum().backward()
    # :868-882
    grads = be.ssd_chunk_scan_backward(cu(go), cu(i["X"]), cu(i["dt"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), 16,
                                       cu(i["D"]), cu(i["z"]), cu(seq_lens), None, cu(i["init"]))
    assert len(grads) == 8
    for k, gk in zip(("X", "dt", "A", "B", "C", "D", "z", "init"), grads):
        assert gk.shape == i[k].shape
        close(gk, w[k].grad, f"grad {k}")
    # cu_seqlens instead of seq_lens, no optional tensors
    cu_seqlens = torch.tensor([0, 33, 103], dtype=torch.int64)
    Y2 = be.ssd_chunk_scan(cu(i["X"]), cu(i["dt"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), 32, None, None, None,
                           cu(cu_seqlens), None)
    close(Y2, O.ssd_chunk_scan(i["X"], i["dt"], i["A"], i["B"], i["C"], 32, seq_meta={"cu_seqlens": cu_seqlens}), "Y, cu_seqlens")


@pytest.mark.parametrize("channels_first", [True, False])
def test_dw_causal_conv_and_backward(channels_first):
    be = backend()
    g = torch.Generator().manual_seed(3)
    b, c, l, k = 2, 24, 200, 4
    x = torch.randn(b, c, l, generator=g) if channels_first else torch.randn(b, l, c, generator=g)
    i = dict(x=x, weight=torch.randn(c, k, generator=g), bias=torch.randn(c, generator=g))
    # :978-983 / :1594-1599
    y = be.dw_causal_conv(cu(i["x"]), cu(i["weight"]), cu(i["bias"]), "silu")
    w = leaves(i)
    yr = O.dw_causal_conv(w["x"], w["weight"], w["bias"], activation="silu")
    close(y, yr.detach(), "y")
    go = torch.randn(yr.shape, generator=g)
    (yr * go).sum().backward()
    # :1017-1023
    dx, dw, db = be.dw_causal_conv_backward(cu(go), cu(i["x"]), cu(i["weight"]), cu(i["bias"]), "silu")
    close(dx, w["x"].grad, "grad x")
    close(dw, w["weight"].grad, "grad weight")
    close(db, w["bias"].grad, "grad bias")
    dx2, dw2, db2 = be.dw_causal_conv_backward(cu(go), cu(i["x"]), cu(i["weight"]), None, "identity")
    assert db2 is None and dx2.shape == x.shape and dw2.shape == (c, k)


@pytest.mark.parametrize("is_rms,prenorm", [(True, True), (False, True), (False, False)])
def test_fused_layer_norm_and_backward(is_rms, prenorm):
    be = backend()
    g = torch.Generator().manual_seed(4)
    b, l, d = 2, 50, 96
    i = dict(x=torch.randn(b, l, d, generator=g), weight=1 + 0.1 * torch.randn(d, generator=g),
             bias=None if is_rms else 0.1 * torch.randn(d, generator=g), residual=torch.randn(b, l, d, generator=g))
    # :1148-1157 / :1640-1653
    y = be.fused_layer_norm(cu(i["x"]), cu(i["weight"]), cu(i["bias"]), cu(i["residual"]), is_rms, 1e-5, prenorm, True)
    w = leaves(i)
    yr = O.fused_layer_norm(w["x"], w["weight"], w["bias"], residual=w["residual"], is_rms=is_rms, eps=1e-5,
                            prenorm=prenorm, residual_in_fp32=True)
    close(y, yr.detach(), "y")
    go = torch.randn(yr.shape, generator=g)
    (yr * go).sum().backward()
    # :1204-1215
    dx, dw, db, dres = be.fused_layer_norm_backward(cu(go), cu(i["x"]), cu(i["weight"]), cu(i["bias"]),
                                                    cu(i["residual"]), is_rms, 1e-5, prenorm, True)
    close(dx, w["x"].grad, "grad x")
    close(dw, w["weight"].grad, "grad weight")
    close(db, None if is_rms else w["bias"].grad, "grad bias")
    close(dres, w["residual"].grad, "grad residual")
    dx2, dw2, db2, dres2 = be.fused_layer_norm_backward(cu(go), cu(i["x"]), cu(i["weight"]), None, None, is_rms, 1e-5,
                                                        prenorm, True)
    assert db2 is None and dres2 is None and dx2.shape == (b, l, d)


def test_contract_violations_are_value_errors():
    be = backend()
    i = scan_inputs(l=32)
    with pytest.raises(ValueError):
        be.selective_scan(cu(i["u"]), cu(i["delta"]), cu(i["A"])[:, :3], cu(i["B"]), cu(i["C"]), None, None, None, False, False)
    with pytest.raises(ValueError):
        be.dw_causal_conv(cu(i["u"]), torch.randn(8, 4).cuda(), None, "gelu")

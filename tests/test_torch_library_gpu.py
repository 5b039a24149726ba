"""``torch.ops.ssm_amd.*`` on the device: the registered operators run the HIP kernels (same values as the Python
façade), differentiate through their registered backward operators (same gradients as the façade's autograd
functions), and pass PyTorch's own consistency checks of a registration (schema, fake tensors, autograd)."""

import pytest
import torch

from ssm_amd import ops
from ssm_amd import torch_library  # noqa: F401  (registers the operators)
from tests.test_scan_fwd_gpu import make_inputs

pytestmark = pytest.mark.gpu

CHECKS = ("test_schema", "test_faketensor", "test_autograd_registration")


def _dev(t):
    return None if t is None else t.cuda()


def _scan_args(dtype, grad):
    inp = make_inputs(7, 2, 16, 272, 16, dtype=dtype)
    g = {k: _dev(v) for k, v in inp.items()}
    if grad:
        for v in g.values():
            v.requires_grad_(True)
    return g


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_selective_scan_through_the_dispatcher(dtype):
    g, h = _scan_args(dtype, True), _scan_args(dtype, True)
    y, last = torch.ops.ssm_amd.selective_scan(g["u"], g["delta"], g["A"], g["B"], g["C"], g["D"], g["z"], g["dt_bias"],
                                               True, True)
    yr, lr = ops.selective_scan(h["u"], h["delta"], h["A"], h["B"], h["C"], D=h["D"], z=h["z"], dt_bias=h["dt_bias"],
                                softplus=True, return_last_state=True)
    assert torch.equal(y, yr) and torch.equal(last, lr)
    w = torch.randn_like(y.float()).to(dtype)
    wl = torch.randn_like(last.float()).to(dtype)
    ((y.float() * w.float()).sum() + (last.float() * wl.float()).sum()).backward()
    ((yr.float() * w.float()).sum() + (lr.float() * wl.float()).sum()).backward()
    for k in g:
        assert g[k].grad is not None and g[k].grad.dtype == g[k].dtype, k
        torch.testing.assert_close(g[k].grad, h[k].grad, rtol=1e-6, atol=0, msg=lambda m, k=k: f"grad {k}: {m}")
    y2, none = torch.ops.ssm_amd.selective_scan(g["u"].detach(), g["delta"].detach(), g["A"].detach(), g["B"].detach(),
                                                g["C"].detach())
    assert none.numel() == 0 and y2.shape == y.shape


def test_state_step_updates_the_state_in_place():
    g = torch.Generator().manual_seed(3)
    state = torch.randn(3, 40, 16, generator=g).cuda()
    x, dt, z = (torch.randn(3, 40, generator=g).cuda() for _ in range(3))
    A = -(torch.rand(40, 16, generator=g) + 0.5).cuda()
    Bm, Cm = torch.randn(3, 1, 16, generator=g).cuda(), torch.randn(3, 1, 16, generator=g).cuda()
    s1, s2 = state.clone(), state.clone()
    y1 = torch.ops.ssm_amd.selective_state_step(s1, x, dt, A, Bm, Cm, None, z, None, True)
    y2 = ops.selective_state_step(s2, x, dt, A, Bm, Cm, z=z, softplus=True)
    assert torch.equal(y1, y2) and torch.equal(s1, s2) and not torch.equal(s1, state)


def test_chunk_scan_conv_and_norm_differentiate_through_the_dispatcher():
    g = torch.Generator().manual_seed(5)
    leaf = lambda *s: torch.randn(*s, generator=g).cuda().requires_grad_(True)
    # diagonal chunk scan
    X, Bm, Cm = leaf(2, 70, 2, 64), leaf(2, 70, 2, 64), leaf(2, 70, 2, 64)
    dt = (torch.rand(2, 70, 2, generator=g) * 0.2).cuda().requires_grad_(True)
    A = (-(torch.rand(2, generator=g) + 0.3)).cuda().requires_grad_(True)
    args = (X, dt, A, Bm, Cm)
    twins = tuple(t.detach().clone().requires_grad_(True) for t in args)
    Y = torch.ops.ssm_amd.ssd_chunk_scan(*args, 32)
    Yr = ops.ssd_chunk_scan(*twins, 32)
    assert torch.equal(Y, Yr)
    w = torch.randn_like(Y)
    (Y * w).sum().backward()
    (Yr * w).sum().backward()
    for a, b in zip(args, twins):
        torch.testing.assert_close(a.grad, b.grad, rtol=1e-6, atol=0)
    # convolution
    x, wt, bias = leaf(2, 24, 100), leaf(24, 4), leaf(24)
    tw = tuple(t.detach().clone().requires_grad_(True) for t in (x, wt, bias))
    y = torch.ops.ssm_amd.dw_causal_conv(x, wt, bias, "silu")
    yr = ops.dw_causal_conv(*tw, activation="silu")
    assert torch.equal(y, yr)
    y.square().sum().backward()
    yr.square().sum().backward()
    for a, b in zip((x, wt, bias), tw):
        torch.testing.assert_close(a.grad, b.grad, rtol=1e-6, atol=0)
    # residual add + RMSNorm
    x, wt, res = leaf(3, 5, 96), leaf(96), leaf(3, 5, 96)
    tw = tuple(t.detach().clone().requires_grad_(True) for t in (x, wt, res))
    y = torch.ops.ssm_amd.fused_layer_norm(x, wt, None, res, True, 1e-5, True, True)
    yr = ops.fused_layer_norm(tw[0], tw[1], None, residual=tw[2], is_rms=True, eps=1e-5, prenorm=True,
                              residual_in_fp32=True)
    assert torch.equal(y, yr)
    y.square().sum().backward()
    yr.square().sum().backward()
    for a, b in zip((x, wt, res), tw):
        torch.testing.assert_close(a.grad, b.grad, rtol=1e-5, atol=1e-6)


def test_registrations_pass_opcheck():
    g = _scan_args(torch.float32, True)
    torch.library.opcheck(torch.ops.ssm_amd.selective_scan.default,
                          (g["u"], g["delta"], g["A"], g["B"], g["C"], g["D"], g["z"], g["dt_bias"], True, True),
                          test_utils=CHECKS)
    gen = torch.Generator().manual_seed(1)
    x = torch.randn(2, 24, 100, generator=gen).cuda().requires_grad_(True)
    wt = torch.randn(24, 4, generator=gen).cuda().requires_grad_(True)
    torch.library.opcheck(torch.ops.ssm_amd.dw_causal_conv.default, (x, wt, None, "silu"), test_utils=CHECKS)
    state = torch.randn(3, 40, 16, generator=gen).cuda()
    v = lambda: torch.randn(3, 40, generator=gen).cuda()
    A = -(torch.rand(40, 16, generator=gen) + 0.5).cuda()
    Bm, Cm = torch.randn(3, 1, 16, generator=gen).cuda(), torch.randn(3, 1, 16, generator=gen).cuda()
    torch.library.opcheck(torch.ops.ssm_amd.selective_state_step.default, (state, v(), v(), A, Bm, Cm),
                          test_utils=("test_schema", "test_faketensor"))
    xn = torch.randn(3, 5, 96, generator=gen).cuda().requires_grad_(True)
    wn = torch.randn(96, generator=gen).cuda().requires_grad_(True)
    torch.library.opcheck(torch.ops.ssm_amd.fused_layer_norm.default, (xn, wn, None, None, True), test_utils=CHECKS)


def test_a_traced_graph_holds_one_node_per_operator_call():
    """What the registration is for (the reference's ``TORCH_LIBRARY`` block, src/ssm/ops/cpu/bindings.cpp:151-189):
    a function that calls the operators traces into a graph with one opaque node per call, forward and backward,
    and the compiled function gives the eager results."""
    from torch.fx.experimental.proxy_tensor import make_fx

    gen = torch.Generator().manual_seed(3)
    x = torch.randn(2, 24, 100, generator=gen).cuda().requires_grad_(True)
    wt = torch.randn(24, 4, generator=gen).cuda().requires_grad_(True)
    delta = torch.randn(2, 24, 100, generator=gen).cuda().requires_grad_(True)
    A = (-(torch.rand(24, 8, generator=gen) + 0.5)).cuda().requires_grad_(True)
    Bm = torch.randn(2, 1, 8, 100, generator=gen).cuda().requires_grad_(True)
    Cm = torch.randn(2, 1, 8, 100, generator=gen).cuda().requires_grad_(True)
    wn = torch.randn(24, generator=gen).cuda().requires_grad_(True)

    def block(x, wt, delta, A, Bm, Cm, wn):
        h = torch.ops.ssm_amd.dw_causal_conv(x, wt, None, "silu")
        y, _ = torch.ops.ssm_amd.selective_scan(h, delta, A, Bm, Cm, None, None, None, True, False)
        return torch.ops.ssm_amd.fused_layer_norm(y.transpose(1, 2), wn, None, None, True)

    args = (x, wt, delta, A, Bm, Cm, wn)
    graph = make_fx(block, tracing_mode="fake")(*args)
    targets = [n.target for n in graph.graph.nodes if n.op == "call_function"]
    for op in (torch.ops.ssm_amd.dw_causal_conv.default, torch.ops.ssm_amd.selective_scan.default,
               torch.ops.ssm_amd.fused_layer_norm.default):
        assert targets.count(op) == 1, targets

    eager = block(*args)
    grads = torch.autograd.grad(eager.square().sum(), args)
    compiled = torch.compile(block, backend="aot_eager", fullgraph=True)
    out = compiled(*args)
    assert torch.equal(out, eager)
    for a, b in zip(torch.autograd.grad(out.square().sum(), args), grads):
        assert torch.equal(a, b)


def test_fake_outputs_promise_the_strides_the_kernels_produce():
    """A compiler plans the consumers of an operator's output on the strides of its fake: for inputs that are views
    (a permuted projection, a half of a wider one, an expanded parameter) the fakes must still describe what comes
    back -- dense tensors, except the convolution's gradient of a view of rows, which lies in rows itself."""
    g = torch.Generator().manual_seed(11)
    wide = torch.randn(2, 96, 128, generator=g).to(torch.bfloat16).cuda()
    w, b = torch.randn(64, 4, generator=g).cuda(), torch.randn(64, generator=g).cuda()
    views = {"permuted half": wide[:, :, :64].permute(0, 2, 1), "permuted": wide.permute(0, 2, 1)[:, :64],
             "6 channels (copied)": wide[:, :, :6].permute(0, 2, 1), "dense": wide[:, :, :64].permute(0, 2, 1).contiguous()}
    for name, x in views.items():
        ww, bb = (w, b) if x.shape[1] == 64 else (w[:6].contiguous(), b[:6].contiguous())
        meta = lambda t: torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device="meta")
        y = torch.ops.ssm_amd.dw_causal_conv(x, ww, bb, "silu")
        ym = torch.ops.ssm_amd.dw_causal_conv(meta(x), meta(ww), meta(bb), "silu")
        assert y.stride() == ym.stride() and y.shape == ym.shape, name
        go = torch.randn_like(y)
        real = torch.ops.ssm_amd.dw_causal_conv_backward(go, x, ww, bb, "silu")
        fake = torch.ops.ssm_amd.dw_causal_conv_backward(meta(go), meta(x), meta(ww), meta(bb), "silu")
        for r, f in zip(real, fake):
            assert r.shape == f.shape and r.stride() == f.stride() and r.dtype == f.dtype, name
    # the scan on views: outputs and gradients are dense whatever the inputs' strides
    inp = make_inputs(7, 2, 16, 272, 16, dtype=torch.bfloat16)
    u = inp["u"].cuda().transpose(1, 2).contiguous().transpose(1, 2)          # (B, D, L) view of (B, L, D) memory
    rest = [inp[k].cuda() for k in ("delta", "A", "B", "C", "D", "z", "dt_bias")]
    meta = lambda t: torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device="meta")
    y, _ = torch.ops.ssm_amd.selective_scan(u, *rest, True, False)
    ym, _ = torch.ops.ssm_amd.selective_scan(meta(u), *[meta(t) for t in rest], True, False)
    assert y.stride() == ym.stride() and y.is_contiguous()

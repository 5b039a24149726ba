"""Every operator, forward and backward, captured in a HIP graph and replayed: no entry point allocates, clears
memory with a memset node or synchronises, so a captured call must give on every replay what the eager call gives on
the inputs of that moment.  Each graph is replayed three times on fresh input values, with eager work and
synchronisations in between, and every replay is compared with the eager result bit for bit."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _ops():
    from ssm_amd import ops
    return ops


def _check_replays(make_inputs, fn, what):
    """``make_inputs(seed)`` -> list of device tensors; ``fn(*inputs)`` -> tuple of result tensors."""
    static = [t.clone() for t in make_inputs(0)]
    fn(*static)                                   # warm-up outside the capture (lazy initialisation, forms remembered)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs = fn(*static)
    torch.cuda.current_stream().wait_stream(side)
    for seed in (1, 2, 3):
        fresh = make_inputs(seed)
        want = [o.clone() for o in fn(*fresh) if o is not None]      # eager work between the replays
        torch.cuda.synchronize()
        for s, f in zip(static, fresh):
            s.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        got = [o for o in outs if o is not None]
        assert len(got) == len(want)
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"{what}: result {i} of the replay with seed {seed} differs from the eager call"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_selective_scan_forward_and_backward(dtype):
    ops = _ops()
    B, D, L, N = 2, 96, 1024, 16

    def inputs(seed):
        g = torch.Generator().manual_seed(seed)
        u, dl, z, go = (torch.randn(B, D, L, generator=g).to(dtype).cuda() for _ in range(4))
        Bm, Cm = (torch.randn(B, 1, N, L, generator=g).to(dtype).cuda() for _ in range(2))
        A = (-(torch.rand(D, N, generator=g) + 0.5)).cuda()
        Dk, bias = torch.randn(D, generator=g).cuda(), torch.randn(D, generator=g).cuda()
        return [u, dl, A, Bm, Cm, Dk, z, bias, go]

    def fn(u, dl, A, Bm, Cm, Dk, z, bias, go):
        y, last = ops._scan_forward(u, dl, A, Bm, Cm, Dk, z, bias, True, True)
        grads = ops._scan_backward(go, None, u, dl, A, Bm, Cm, Dk, z, bias, True)
        return (y, last) + tuple(grads)

    _check_replays(inputs, fn, "selective_scan")


def test_state_step_updates_its_state_on_every_replay():
    ops = _ops()
    B, D, N = 4, 128, 16
    g = torch.Generator().manual_seed(0)
    A = (-(torch.rand(D, N, generator=g) + 0.5)).cuda()
    Bm, Cm = torch.randn(B, 1, N, generator=g).cuda(), torch.randn(B, 1, N, generator=g).cuda()
    x, dt = torch.randn(B, D, generator=g).cuda(), torch.randn(B, D, generator=g).cuda()
    state = torch.randn(B, D, N, generator=g).cuda()
    eager_state = state.clone()
    ops.selective_state_step(state.clone(), x, dt, A, Bm, Cm)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            y = ops.selective_state_step(state, x, dt, A, Bm, Cm)
    torch.cuda.current_stream().wait_stream(side)
    for step in range(4):
        x.normal_(generator=None)
        want = ops.selective_state_step(eager_state, x, dt, A, Bm, Cm)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want) and torch.equal(state, eager_state), f"step {step}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_chunk_scan_conv_and_norm_forward_and_backward(dtype):
    ops = _ops()
    B, L, H, P = 2, 512, 4, 64

    def scan_inputs(seed):
        g = torch.Generator().manual_seed(seed)
        X, Bq, Cq, zq, go = (torch.randn(B, L, H, P, generator=g).to(dtype).cuda() for _ in range(5))
        dt = (torch.rand(B, L, H, generator=g) * 0.1).cuda()
        A, Dk = (-(torch.rand(H, generator=g) + 0.5)).cuda(), torch.randn(H, generator=g).cuda()
        return [X, dt, A, Bq, Cq, Dk, zq, go]

    def scan_fn(X, dt, A, Bq, Cq, Dk, zq, go):
        Y = ops._dscan_forward(X, dt, A, Bq, Cq, 64, Dk, zq, None, None)
        return (Y,) + tuple(ops._dscan_backward(go, X, dt, A, Bq, Cq, 64, Dk, zq, None, None))

    _check_replays(scan_inputs, scan_fn, "ssd_chunk_scan")

    for cl in (False, True):
        def conv_inputs(seed):
            g = torch.Generator().manual_seed(seed)
            shape = (B, L, 96) if cl else (B, 96, L)
            x, go = (torch.randn(shape, generator=g).to(dtype).cuda() for _ in range(2))
            return [x, torch.randn(96, 4, generator=g).cuda(), torch.randn(96, generator=g).cuda(), go]

        def conv_fn(x, w, b, go):
            return (ops._conv_forward(x, w, b, "silu", channels_last=cl),) + tuple(ops._conv_backward(go, x, w, b, "silu", channels_last=cl))

        _check_replays(conv_inputs, conv_fn, f"dw_causal_conv, channels last {cl}")

    def norm_inputs(seed):
        g = torch.Generator().manual_seed(seed)
        x, r, go = (torch.randn(B, L, 768, generator=g).to(dtype).cuda() for _ in range(3))
        return [x, torch.randn(768, generator=g).cuda(), torch.randn(768, generator=g).cuda(), r, go]

    def norm_fn(x, w, b, r, go):
        y, ro, mean, rstd = ops._norm_forward(x, w, b, r, False, 1e-5, True, True, want_residual_out=True, want_stats=True)
        return (y, ro) + tuple(ops._norm_backward(go, x, w, r, mean, rstd, False, True, True, True))

    _check_replays(norm_inputs, norm_fn, "fused_layer_norm")


def test_ssd_combined_forward_and_backward():
    from ssm_amd.ops import ssd
    H, P, N, Q, L = 4, 64, 128, 256, 1024

    def inputs(seed):
        g = torch.Generator().manual_seed(seed)
        x, z, go = (torch.randn(1, L, H, P, generator=g).to(torch.bfloat16).cuda() for _ in range(3))
        Bm, Cm = (torch.randn(1, L, 1, N, generator=g).to(torch.bfloat16).cuda() for _ in range(2))
        dt = (torch.rand(1, L, H, generator=g) * 0.1).cuda()
        A, D = (-(torch.rand(H, generator=g) * 4 + 0.5)).cuda(), torch.randn(H, generator=g).cuda()
        return [x, dt, A, Bm, Cm, D, z, go]

    def fn(x, dt, A, Bm, Cm, D, z, go):
        y, final = ssd.ssd_combined(x, dt, A, Bm, Cm, Q, D=D, z=z, return_final_states=True)
        grads = ssd.ssd_combined_backward(go, None, x, dt, A, Bm, Cm, Q, D=D, z=z)
        return (y, final) + tuple(g for g in grads if g is not None)

    _check_replays(inputs, fn, "ssd_combined")


def test_the_reference_blocks_views_in_a_graph():
    """The calls of ``Mamba1.forward`` (/root/reference/src/ssm/modules/mamba1.py:203-247) on its views -- the
    convolution on a permuted half of a projection, read as it lies, and the scan on a permuted ``delta`` and ``z``,
    turned by the library's own copy kernel, with projections constant in time -- forward and backward inside one
    captured graph."""
    ops = _ops()
    B, L, D, N, dtype = 2, 1024, 96, 16, torch.bfloat16

    def inputs(seed):
        g = torch.Generator().manual_seed(seed)
        xz = torch.randn(B, L, 2 * D, generator=g).to(dtype).cuda()
        delta_rows = torch.randn(B, L, D, generator=g).to(dtype).cuda()
        w, cb = (torch.rand(D, 4, generator=g) - 0.5).cuda(), (torch.randn(D, generator=g) * 0.1).cuda()
        A = (-(torch.rand(D, N, generator=g) + 0.5)).cuda()
        Bm, Cm = torch.randn(D, N, generator=g).cuda(), torch.randn(D, N, generator=g).cuda()
        Dk, bias = torch.randn(D, generator=g).cuda(), torch.randn(D, generator=g).cuda()
        go = torch.randn(B, D, L, generator=g).to(dtype).cuda()
        return [xz, delta_rows, w, cb, A, Bm, Cm, Dk, bias, go]

    def fn(xz, delta_rows, w, cb, A, Bm, Cm, Dk, bias, go):
        projected, gate = xz.chunk(2, dim=-1)
        x = projected.permute(0, 2, 1)
        assert ops._conv_rows_view(x, True, 4) is not None
        u = ops._conv_forward(x, w, cb, "silu")
        delta, z = delta_rows.permute(0, 2, 1), gate.permute(0, 2, 1)
        y, last = ops._scan_forward(u, delta, A, Bm, Cm, Dk, z, bias, True, True)
        grads = ops._scan_backward(go, None, u, delta, A, Bm, Cm, Dk, z, bias, True)
        dx, dw, db = ops._conv_backward(grads[0], x, w, cb, "silu")
        return (u, y, last, dx, dw, db) + tuple(grads)

    _check_replays(inputs, fn, "the reference block's calls on views")

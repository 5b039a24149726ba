#!/usr/bin/env python3
"""Benchmark of the operator hot path on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

Headline workload (``config.workload``): ``selective_scan`` forward at the
Mamba-1 prefill shape B=8, D=1536, L=2048, N=16 with bf16 activations, fp32
state, one B/C group, D skip, z gate, dt_bias and softplus.  A "step" is one
forward pass over one batch of synthetic inputs already resident in HBM; four
input/output sets (about 0.8 GB) are rotated so that a step does not find the
previous step's data in the 256 MB last-level cache.

``value`` is algorithmic bytes per step / wall time per step (GB/s) over the K
timed steps.  ``roofline`` prices the same bytes against the kernel's own
average duration measured with HIP events on the launch stream.
``cpu_baseline`` times the CPU restatement of the reference's Python path
(``oracle/``) on a bounded slice of the same workload on this host.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


PROFILES = os.path.join(ROOT, "profiles")
CLOCK_GHZ = 2.4            # MI355X peak engine clock
SIMDS = 256 * 4


def _profile_rows(name):
    """Rows ``(kernel, counter, mean per dispatch)`` of a counter summary under profiles/ (the text
    ``rocprofv3 --pmc`` runs of this file were condensed to), or [] when the file is missing."""
    path = os.path.join(PROFILES, name)
    rows = []
    if not os.path.exists(path):
        return rows
    for line in open(path):
        parts = line.rstrip("\n").rsplit(None, 3)
        if len(parts) == 4 and parts[2].isdigit():
            try:
                rows.append((parts[0].strip(), parts[1], float(parts[3])))
            except ValueError:
                pass
    return rows


def headline_counters(kernel_substr="scan_fwd_fast_kernel"):
    """HBM traffic and vector-ALU instruction count of one launch of the headline kernel, from the counter
    summaries committed under profiles/ (``FETCH_SIZE`` and ``WRITE_SIZE`` in KiB, each scaled by what the same
    counter read for the 256 MiB copy of ``--copy-calibration`` in the same run).  A summary taken with another
    kernel than the one named here does not count: the figure is then ``None``."""
    out = {"traffic": None, "valu_insts": None, "source": None}
    fetch = _profile_rows("scan_fwd_bf16_headline_pmc_FETCH_SIZE.txt")
    write = _profile_rows("scan_fwd_bf16_headline_pmc_WRITE_SIZE.txt")
    sq = _profile_rows("scan_fwd_bf16_headline_pmc_SQ.txt")

    def pick(rows, counter, sub):
        for k, c, v in rows:
            if c == counter and sub in k:
                return k, v
        return None, None

    kf, f = pick(fetch, "FETCH_SIZE", kernel_substr)
    kw, w = pick(write, "WRITE_SIZE", kernel_substr)
    _, cf = pick(fetch, "FETCH_SIZE", "CUDAFunctorOnSelf_add")
    _, cw = pick(write, "WRITE_SIZE", "CUDAFunctorOnSelf_add")
    if None not in (f, w, cf, cw) and cf > 0 and cw > 0:
        copy_kib = 256.0 * 1024.0
        out["traffic"] = int(round((f * copy_kib / cf + w * copy_kib / cw) * 1024))
        out["source"] = f"profiles/scan_fwd_bf16_headline_pmc_{{FETCH,WRITE}}_SIZE.txt ({kf})"
    _, v = pick(sq, "SQ_INSTS_VALU", kernel_substr)
    out["valu_insts"] = v
    return out


def _event_ms(fn, iters):
    """Average duration (ms) of ``fn``'s GPU work, one event pair per call, on the
    current stream (the stream the kernels are launched on)."""
    pairs = []
    for i in range(iters):
        s = torch.cuda.Event(enable_timing=True)
        e = torch.cuda.Event(enable_timing=True)
        s.record()
        fn(i)
        e.record()
        pairs.append((s, e))
    torch.cuda.synchronize()
    times = sorted(s.elapsed_time(e) for s, e in pairs)
    return sum(times) / len(times), times[len(times) // 2]


def _graph_us(fn, calls=24, replays=5):
    """Average GPU time (us) of one ``fn(i)``: ``calls`` of them captured once in a HIP graph and replayed, so that
    the time between launches is the GPU's and not Python's (an operator whose kernel takes less than the ~20 us
    that its Python entry takes is otherwise timed by its caller)."""
    for i in range(3):
        fn(i)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(calls):
                fn(i)
    torch.cuda.current_stream().wait_stream(side)
    graph.replay()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(replays):
        graph.replay()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / replays / calls * 1e3


SPIN_UP_LAUNCHES = 300


def bench_scan_fwd(steps, warmup, dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16,
                   nsets=4, spin_up=SPIN_UP_LAUNCHES):
    from ssm_amd import configs
    from ssm_amd.ops import ScanPlan

    plans = []
    for s in range(nsets):
        inp = configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=s))
        plans.append(ScanPlan(inp["u"], inp["delta"], inp["A"], inp["B"], inp["C"], inp["D"], inp["z"],
                              inp["dt_bias"], True, True))
    elt = 2 if dtype != torch.float32 else 4
    nbytes = configs.scan_fwd_bytes(batch, dim, length, nstate, elt)

    # The device takes some tens of milliseconds of work to reach its clocks after idling (the first hundred
    # launches of a fresh process run up to 15 % slower): bring it there before the W warm-up steps.
    for i in range(spin_up):
        plans[i % nsets].run()
    torch.cuda.synchronize()
    for i in range(warmup):
        plans[i % nsets].run()
    torch.cuda.synchronize()
    # the K timed steps, bracketed on the host by the clock and on the launch stream by two HIP events
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(steps):
        plans[i % nsets].run()
    ev1.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    avg_ms = ev0.elapsed_time(ev1) / steps
    return dict(bytes=nbytes, wall_s=wall, kernel_ms=avg_ms, tokens=batch * length)


def _time_us(fn, iters=20, warmup=3):
    for i in range(warmup):
        fn(i)
    torch.cuda.synchronize()
    avg_ms, med_ms = _event_ms(fn, iters)
    return avg_ms * 1e3


def bench_scan_bwd(dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16):
    """Forward (with chunk checkpoints) + backward of the config-1 scan, all gradients."""
    from ssm_amd import configs, ops

    inp = configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=0))
    g = torch.Generator().manual_seed(1)
    go = torch.randn(batch, dim, length, generator=g).to(dtype).cuda()
    plan = ops.ScanPlan(inp["u"], inp["delta"], inp["A"], inp["B"], inp["C"], inp["D"], inp["z"], inp["dt_bias"],
                        True, False, want_chunk_states=True)
    plan.run()

    def bwd(i):
        ops._scan_backward(go, None, inp["u"], inp["delta"], inp["A"], inp["B"], inp["C"], inp["D"], inp["z"],
                           inp["dt_bias"], True, chunk_states=plan.chunk_states)
    us = _time_us(bwd, iters=30, warmup=100)      # a kernel of its own power profile: the clocks settle again
    elt = 2 if dtype != torch.float32 else 4
    nbytes = 7 * elt * batch * dim * length + 2 * elt * batch * nstate * length + 2 * 4 * batch * nstate * length
    return {"kernel_us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1),
            "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes}


def bench_mixer_config1(dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16, width=4):
    """BASELINE configuration 1 as one step: depthwise causal conv (width 4, SiLU) -> selective scan (per-token
    B/C, z gate, D skip, bias + softplus), forward and backward through autograd with a random upstream gradient,
    gradients for x, the conv weights, delta, A, B, C, D and the bias."""
    from ssm_amd import configs, ops

    inp = configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=0))
    g = torch.Generator().manual_seed(2)
    x = torch.randn(batch, dim, length, generator=g).to(dtype).cuda().requires_grad_()
    w = (torch.rand(dim, width, generator=g) - 0.5).cuda().requires_grad_()
    b = (torch.randn(dim, generator=g) * 0.02).cuda().requires_grad_()
    go = torch.randn(batch, dim, length, generator=g).to(dtype).cuda()
    leaves = [x, w, b] + [inp[k].requires_grad_() for k in ("delta", "A", "B", "C", "D", "dt_bias")]

    def step(_):
        u = ops.dw_causal_conv(x, w, b, activation="silu")
        y = ops.selective_scan(u, inp["delta"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                               dt_bias=inp["dt_bias"], softplus=True)
        y.backward(go)
        for t in leaves:
            t.grad = None

    us = _time_us(step, iters=20, warmup=30)
    return {"fwd_bwd_us": round(us, 1), "tokens_per_s": round(batch * length / us * 1e6, 1),
            "shape": f"B={batch} D={dim} L={length} N={nstate} K={width} {str(dtype).split('.')[-1]}: conv + scan, "
                     "forward + backward through autograd"}


def bench_conv(dtype=torch.bfloat16, batch=8, chans=1536, length=2048, width=4):
    """The convolution of config 1 in its three layouts, forward and backward, each timed inside a replayed HIP
    graph (the kernels take about as long as the Python entry): (B,C,L); channels last (B,L,C), the layout of the
    Mamba-2 block; and the (B,C,L)-shaped view of one half of a (B,L,2C) projection that the reference's Mamba-1
    block passes (src/ssm/modules/mamba1.py:203-215), read as it lies, y dense (B,C,L)."""
    from ssm_amd import ops

    g = torch.Generator().manual_seed(0)
    xs = [torch.randn(batch, chans, length, generator=g).to(dtype).cuda() for _ in range(3)]
    w = (torch.rand(chans, width, generator=g) - 0.5).cuda()
    b = (torch.randn(chans, generator=g) * 0.02).cuda()
    go = torch.randn(batch, chans, length, generator=g).to(dtype).cuda()
    elt = 2 if dtype != torch.float32 else 4
    fwd_us = _graph_us(lambda i: ops._conv_forward(xs[i % 3], w, b, "silu"))
    bwd_us = _graph_us(lambda i: ops._conv_backward(go, xs[i % 3], w, b, "silu"))
    fb, bb = 2 * elt * batch * chans * length, 3 * elt * batch * chans * length
    xl = [x.transpose(1, 2).contiguous() for x in xs]
    gl = go.transpose(1, 2).contiguous()
    cl_fwd_us = _graph_us(lambda i: ops._conv_forward(xl[i % 3], w, b, "silu"))
    cl_bwd_us = _graph_us(lambda i: ops._conv_backward(gl, xl[i % 3], w, b, "silu"))
    wide = [torch.randn(batch, length, 2 * chans, generator=g).to(dtype).cuda() for _ in range(3)]
    views = [p.chunk(2, dim=-1)[0].permute(0, 2, 1) for p in wide]
    assert ops._conv_rows_view(views[0], True, width) is not None
    rv_fwd_us = _graph_us(lambda i: ops._conv_forward(views[i % 3], w, b, "silu"))
    rv_bwd_us = _graph_us(lambda i: ops._conv_backward(go, views[i % 3], w, b, "silu"))
    frac = lambda nbytes, us: round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)
    # the dense (B,C,L) copy of such a view that the scan asks for (delta and z of the reference's Mamba1 block)
    from ssm_amd.ops import _contract
    copy_us = _graph_us(lambda i: _contract.dense_copy(views[i % 3]))
    torch_copy_us = _graph_us(lambda i: views[i % 3].contiguous(), calls=6, replays=2)
    return {"fwd_us": round(fwd_us, 1), "fwd_GBps": round(fb / fwd_us / 1e3, 1), "fwd_frac_hbm": frac(fb, fwd_us),
            "view_of_rows_dense_copy_us": round(copy_us, 1), "view_of_rows_dense_copy_frac_hbm": frac(fb, copy_us),
            "view_of_rows_dense_copy_by_torch_us": round(torch_copy_us, 1),
            "bwd_us": round(bwd_us, 1), "bwd_GBps": round(bb / bwd_us / 1e3, 1), "bwd_frac_hbm": frac(bb, bwd_us),
            "channels_last_fwd_us": round(cl_fwd_us, 1), "channels_last_bwd_us": round(cl_bwd_us, 1),
            "channels_last_fwd_frac_hbm": frac(fb, cl_fwd_us), "channels_last_bwd_frac_hbm": frac(bb, cl_bwd_us),
            "view_of_rows_fwd_us": round(rv_fwd_us, 1), "view_of_rows_bwd_us": round(rv_bwd_us, 1),
            "view_of_rows_fwd_frac_hbm": frac(fb, rv_fwd_us), "view_of_rows_bwd_frac_hbm": frac(bb, rv_bwd_us),
            "timing": "per call inside a replayed HIP graph of 24 calls (backward: the kernel and the fold of dweight)"}


def bench_norm(batch=16, length=2048, hidden=768):
    from ssm_amd import ops

    g = torch.Generator().manual_seed(0)
    xs = [torch.randn(batch, length, hidden, generator=g).to(torch.bfloat16).cuda() for _ in range(3)]
    rs = [torch.randn(batch, length, hidden, generator=g).cuda() for _ in range(3)]
    w = torch.randn(hidden, generator=g).cuda()
    us = _time_us(lambda i: ops._norm_forward(xs[i % 3], w, None, rs[i % 3], True, 1e-5, True, True,
                                              want_residual_out=True))
    nbytes = batch * length * hidden * (2 + 4 + 2 + 4)
    # backward: reads x, residual, dy and the row statistics, writes dx and dresidual (+ dw)
    _, _, mean, rstd = ops._norm_forward(xs[0], w, None, rs[0], True, 1e-5, True, True, want_stats=True)
    gs = [torch.randn(batch, length, hidden, generator=g).to(torch.bfloat16).cuda() for _ in range(3)]
    bus = _time_us(lambda i: ops._norm_backward(gs[i % 3], xs[0], w, rs[0], mean, rstd, True, True, False, True))
    bbytes = batch * length * hidden * (2 + 4 + 2 + 2 + 4)
    return {"fwd_us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1),
            "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes,
            "bwd_us": round(bus, 1), "bwd_GBps": round(bbytes / bus / 1e3, 1),
            "bwd_frac_hbm": round(bbytes / bus / 1e3 / HBM_PEAK_GBPS, 4),
            "shape": "x bf16 (16,2048,768) + fp32 residual -> y bf16 + fp32 residual_out, RMSNorm"}


def bench_dscan(batch=4, length=4096, heads=80, proj=64, chunk=256):
    """The reference's own "SSD chunk scan" (an element-wise recurrence per (b, h, p)) at the outer
    dimensions of config 3: bf16 X/z, per-token B/C of X's shape, per-head A and D."""
    from ssm_amd import ops

    g = torch.Generator().manual_seed(4)
    X = torch.randn(batch, length, heads, proj, generator=g).to(torch.bfloat16).cuda()
    dt = (torch.rand(batch, length, heads, generator=g) * 0.1).cuda()
    A = -(torch.rand(heads, generator=g) * 15 + 1).cuda()
    Bm = torch.randn(batch, length, heads, proj, generator=g).to(torch.bfloat16).cuda()
    Cm = torch.randn(batch, length, heads, proj, generator=g).to(torch.bfloat16).cuda()
    D = torch.ones(heads).cuda()
    z = torch.randn(batch, length, heads, proj, generator=g).to(torch.bfloat16).cuda()
    gy = torch.randn(batch, length, heads, proj, generator=g).to(torch.bfloat16).cuda()
    fus = _time_us(lambda i: ops._dscan_forward(X, dt, A, Bm, Cm, chunk, D, z, None, None), iters=10)
    # the backward as autograd runs it: the forward left the state entering every 64 steps, and the gradients of
    # X's shape come back in X's type
    _, table = ops._dscan_forward(X, dt, A, Bm, Cm, chunk, D, z, None, None, want_round_states=True)
    bus = _time_us(lambda i: ops._dscan_backward(gy, X, dt, A, Bm, Cm, chunk, D, z, None, None,
                                                 grads_in_input_dtype=True, round_states=table), iters=10)
    # and called on its own with float32 gradients (its own forward sweep first)
    sus = _time_us(lambda i: ops._dscan_backward(gy, X, dt, A, Bm, Cm, chunk, D, z, None, None), iters=10)
    el = batch * length * heads * proj
    fbytes = el * 2 * 5 + batch * length * heads * 4               # X, B, C, z in; Y out; dt
    bbytes = el * 2 * 6 + el * 2 * 4 + batch * length * heads * 8  # X, B, C, z, grad_y in; dX, dB, dC, dz out; dt, ddt
    sbytes = el * 2 * 6 + el * 2 + el * 4 * 3 + batch * length * heads * 8   # dB, dC, dz in float32
    out = {"fwd_us": round(fus, 1), "fwd_GBps": round(fbytes / fus / 1e3, 1),
           "fwd_frac_hbm": round(fbytes / fus / 1e3 / HBM_PEAK_GBPS, 4),
           "bwd_us": round(bus, 1), "bwd_GBps": round(bbytes / bus / 1e3, 1),
           "bwd_frac_hbm": round(bbytes / bus / 1e3 / HBM_PEAK_GBPS, 4),
           "bwd_alone_fp32_grads_us": round(sus, 1), "bwd_alone_fp32_grads_GBps": round(sbytes / sus / 1e3, 1),
           "shape": f"X (B={batch}, L={length}, H={heads}, P={proj}) bf16, chunk {chunk}"}
    del Bm, Cm, z, table
    # the call of the reference's own Mamba2 module (src/ssm/modules/mamba2.py:189-199): B, C, A, D are (H, P)
    # parameters, no gate, float32 activations (the module promotes half to float32); bf16 activations beside it
    Ap = -(torch.rand(heads, proj, generator=g) * 15 + 1).cuda()
    Bp, Cp = torch.randn(heads, proj, generator=g).cuda(), torch.randn(heads, proj, generator=g).cuda()
    Dp = torch.ones(heads, proj).cuda()
    for name, dtype in (("module_call_fp32", torch.float32), ("module_call_bf16", torch.bfloat16)):
        Xm, gm = X.to(dtype), gy.to(dtype)
        f = _time_us(lambda i: ops._dscan_forward(Xm, dt, Ap, Bp, Cp, chunk, Dp, None, None, None, want_round_states=True),
                     iters=10)
        _, table = ops._dscan_forward(Xm, dt, Ap, Bp, Cp, chunk, Dp, None, None, None, want_round_states=True)
        b = _time_us(lambda i: ops._dscan_backward(gm, Xm, dt, Ap, Bp, Cp, chunk, Dp, None, None, None,
                                                   grads_in_input_dtype=True, round_states=table), iters=10)
        e = Xm.element_size()
        fb = el * e * 2 + batch * length * heads * 4 + table.numel() * 4       # X in, Y out; dt; the table out
        bb = el * e * 3 + batch * length * heads * 8 + table.numel() * 4       # X, grad_y in, dX out; dt, ddt; the table in
        out[name] = {"fwd_us": round(f, 1), "fwd_frac_hbm": round(fb / f / 1e3 / HBM_PEAK_GBPS, 4),
                     "bwd_us": round(b, 1), "bwd_frac_hbm": round(bb / b / 1e3 / HBM_PEAK_GBPS, 4)}
    return out


def bench_decode(batch=64, dim=5120, nstate=16, width=4, steps=512):
    """Config 2: 512 consecutive in-place decode steps (fused conv window + state update),
    bf16 activations, fp32 SSM state, grouped B/C (64,1,16)."""
    from ssm_amd import configs, ops

    g = torch.Generator().manual_seed(2)
    ssm_state = torch.randn(batch, dim, nstate, generator=g).cuda()
    conv_state = torch.randn(batch, dim, width, generator=g).to(torch.bfloat16).cuda()
    A = -torch.arange(1, nstate + 1, dtype=torch.float32).repeat(dim, 1).cuda()
    D = torch.ones(dim).cuda()
    bias = configs.inverse_softplus_dt(dim, g).cuda()
    w = (torch.rand(dim, width, generator=g) - 0.5).cuda()
    cb = (torch.randn(dim, generator=g) * 0.02).cuda()
    nset = 8
    plans = []
    for _ in range(nset):
        x = torch.randn(batch, dim, generator=g).to(torch.bfloat16).cuda()
        z = torch.randn(batch, dim, generator=g).to(torch.bfloat16).cuda()
        dt = torch.randn(batch, dim, generator=g).to(torch.bfloat16).cuda()
        Bm = torch.randn(batch, 1, nstate, generator=g).to(torch.bfloat16).cuda()
        Cm = torch.randn(batch, 1, nstate, generator=g).to(torch.bfloat16).cuda()
        plans.append(ops.DecodePlan(conv_state, ssm_state, x, dt, A, Bm, Cm, w, cb, D, z, bias, True))
    for i in range(16):
        plans[i % nset].run()
    torch.cuda.synchronize()
    # eager launches from Python
    t0 = time.perf_counter()
    for i in range(steps):
        plans[i % nset].run()
    torch.cuda.synchronize()
    eager_us = (time.perf_counter() - t0) / steps * 1e6
    # the same 512 launches captured once in a HIP graph and replayed
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(steps):
                plans[i % nset].run()
    torch.cuda.current_stream().wait_stream(side)
    graph.replay()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(3):
        graph.replay()
    e.record()
    torch.cuda.synchronize()
    graph_us = s.elapsed_time(e) / 3 / steps * 1e3
    nbytes = 2 * 4 * batch * dim * nstate + 4 * 2 * batch * dim + 2 * 2 * batch * dim * width + 4 * dim * (nstate + 2 + width + 1)
    return {"us_per_step_graph": round(graph_us, 2), "us_per_step_eager": round(eager_us, 2), "steps": steps,
            "GBps_graph": round(nbytes / graph_us / 1e3, 1),
            "frac_hbm_graph": round(nbytes / graph_us / 1e3 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes}


def bench_ssd(batch=4, length=4096, heads=80, hdim=64, nstate=128, chunk=256):
    """Config 3: Mamba-2 SSD forward, bf16, returns y and final states."""
    from ssm_amd.ops import ssd

    g = torch.Generator().manual_seed(3)
    x = torch.randn(batch, length, heads, hdim, generator=g).to(torch.bfloat16).cuda()
    from ssm_amd import configs
    dt_bias = configs.inverse_softplus_dt(heads, g)
    dt = torch.nn.functional.softplus(torch.randn(batch, length, heads, generator=g) + dt_bias).cuda()
    A = -(torch.rand(heads, generator=g) * 15 + 1).cuda()
    Bm = torch.randn(batch, length, 1, nstate, generator=g).to(torch.bfloat16).cuda()
    Cm = torch.randn(batch, length, 1, nstate, generator=g).to(torch.bfloat16).cuda()
    D = torch.ones(heads).cuda()
    z = torch.randn(batch, length, heads, hdim, generator=g).to(torch.bfloat16).cuda()
    us = _time_us(lambda i: ssd.ssd_combined(x, dt, A, Bm, Cm, chunk, D=D, z=z, return_final_states=True), iters=10)
    nc = length // chunk
    flops = (2 * chunk * chunk * nstate * batch * nc + 2 * chunk * chunk * hdim * batch * nc * heads
             + 2 * 2 * chunk * nstate * hdim * batch * nc * heads)
    # the same call on float16 tensors (the one-pass kernel is compiled for both 16-bit types)
    x16, B16, C16, z16 = (t.to(torch.float16) for t in (x, Bm, Cm, z))
    us16 = _time_us(lambda i: ssd.ssd_combined(x16, dt, A, B16, C16, chunk, D=D, z=z16, return_final_states=True), iters=10)
    return {"us": round(us, 1), "TFLOPs": round(flops / us / 1e6, 1),
            "frac_mfma_bf16_peak": round(flops / us / 1e6 / 2500.0, 4), "dense_tile_flops": flops,
            "float16_us": round(us16, 1)}


def bench_ssd_train(batch=4, length=4096, heads=80, hdim=64, nstate=128, chunk=256):
    """Config 3 shape through the parts of the SSD path that are not the one-pass forward: forward +
    backward through autograd (the backward is four passes of the five-kernel pipeline with operands in
    other roles) and the forward over packed sequences (`seq_idx`, generic kernels)."""
    from ssm_amd.ops import ssd
    from ssm_amd import configs

    g = torch.Generator().manual_seed(3)
    x = torch.randn(batch, length, heads, hdim, generator=g).to(torch.bfloat16).cuda().requires_grad_()
    dt_bias = configs.inverse_softplus_dt(heads, g)
    dt = torch.nn.functional.softplus(torch.randn(batch, length, heads, generator=g) + dt_bias).cuda().requires_grad_()
    A = (-(torch.rand(heads, generator=g) * 15 + 1)).cuda().requires_grad_()
    Bm = torch.randn(batch, length, 1, nstate, generator=g).to(torch.bfloat16).cuda().requires_grad_()
    Cm = torch.randn(batch, length, 1, nstate, generator=g).to(torch.bfloat16).cuda().requires_grad_()
    D = torch.ones(heads).cuda().requires_grad_()
    z = torch.randn(batch, length, heads, hdim, generator=g).to(torch.bfloat16).cuda().requires_grad_()
    dy = torch.randn(batch, length, heads, hdim, generator=g).to(torch.bfloat16).cuda()

    def step(_):
        y = ssd.ssd_combined(x, dt, A, Bm, Cm, chunk, D=D, z=z)
        y.backward(dy)
        for t in (x, dt, A, Bm, Cm, D, z):
            t.grad = None

    fb_us = _time_us(step, iters=5, warmup=2)
    # four sequences of unequal length packed into every batch row
    cuts = [0, length // 8, length // 2, length // 2 + 300, length]
    seq_idx = torch.zeros(batch, length, dtype=torch.int32)
    for i in range(len(cuts) - 1):
        seq_idx[:, cuts[i]:cuts[i + 1]] = i
    seq_idx = seq_idx.cuda()
    with torch.no_grad():
        pk_us = _time_us(lambda i: ssd.ssd_combined(x, dt, A, Bm, Cm, chunk, D=D, z=z, seq_idx=seq_idx), iters=5, warmup=2)
    return {"fwd_bwd_us": round(fb_us, 1), "packed_fwd_us": round(pk_us, 1),
            "shape": f"B={batch} L={length} H={heads} P={hdim} N={nstate} Q={chunk} bf16; packed: 4 sequences per row"}


def bench_model(batch=16, prompt=2048, new_tokens=256):
    """BASELINE config 4: Mamba-2-130M-style stack (24 layers, d_model 768, d_state 128, tied embeddings,
    random weights, bf16): prefill of batch x prompt tokens, then greedy decoding on cached states with
    the step replayed as a HIP graph.  GEMMs are torch's; everything else is this package's kernels."""
    from ssm_amd.harness import Mamba2Config, Mamba2LM
    model = Mamba2LM(Mamba2Config(), seed=0)
    gen = torch.Generator().manual_seed(0)
    tokens = torch.randint(0, model.cfg.vocab_size, (batch, prompt), generator=gen).cuda()
    model.generate(tokens, 4)                                   # warm-up (kernel selection, graph capture path)
    best = None
    for _ in range(2):
        _, t = model.generate(tokens, new_tokens)
        if best is None or t["prefill_s"] + t["decode_s"] < best["prefill_s"] + best["decode_s"]:
            best = t
    return {"prefill_ms": round(best["prefill_s"] * 1e3, 2),
            "prefill_tokens_per_s": round(batch * prompt / best["prefill_s"], 1),
            "decode_ms_per_token": round(best["decode_s"] * 1e3 / (new_tokens - 1), 4),
            "decode_tokens_per_s": round(batch * (new_tokens - 1) / best["decode_s"], 1),
            "shape": f"batch {batch}, prompt {prompt}, {new_tokens} new tokens, 24 layers, d_model 768, "
                     "d_state 128, vocab 50280, bf16, random weights"}


def bench_model1(batch=8, prompt=2048, new_tokens=256):
    """Mamba-1-130M-style stack (24 layers, d_model 768, 1536 channels, 16 states, 4 taps: every mixer call has
    the shape of the headline scan workload), bf16, random weights: prefill through selective_scan with the
    state handed over, then greedy decoding on cached states with the step replayed as a HIP graph."""
    from ssm_amd.harness import Mamba1Config, Mamba1LM
    model = Mamba1LM(Mamba1Config(), seed=0)
    gen = torch.Generator().manual_seed(0)
    tokens = torch.randint(0, model.cfg.vocab_size, (batch, prompt), generator=gen).cuda()
    model.generate(tokens, 4)
    best = None
    for _ in range(2):
        _, t = model.generate(tokens, new_tokens)
        if best is None or t["prefill_s"] + t["decode_s"] < best["prefill_s"] + best["decode_s"]:
            best = t
    return {"prefill_ms": round(best["prefill_s"] * 1e3, 2),
            "prefill_tokens_per_s": round(batch * prompt / best["prefill_s"], 1),
            "decode_ms_per_token": round(best["decode_s"] * 1e3 / (new_tokens - 1), 4),
            "decode_tokens_per_s": round(batch * (new_tokens - 1) / best["decode_s"], 1),
            "shape": f"batch {batch}, prompt {prompt}, {new_tokens} new tokens, 24 layers, d_model 768, "
                     "d_state 16, vocab 50280, bf16, random weights"}


def bench_scan_facade(dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16):
    """The headline call through the drop-in entry ``ops.selective_scan`` (validation, dtype normalisation and
    output allocation inside the timed region) instead of a prepared plan: wall time per call over a queue of
    calls, and the kernel's share of it."""
    from ssm_amd import configs, ops
    sets = [configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=s)) for s in range(4)]

    def call(i):
        g = sets[i % 4]
        return ops.selective_scan(g["u"], g["delta"], g["A"], g["B"], g["C"], D=g["D"], z=g["z"],
                                  dt_bias=g["dt_bias"], softplus=True, return_last_state=True)
    # the input sets above were made on the host while the device idled: bring it back to its clocks first, as
    # the headline does (the first hundred launches after idling run up to 15 % slower)
    for i in range(SPIN_UP_LAUNCHES):
        call(i)
    torch.cuda.synchronize()
    n = 50
    t0 = time.perf_counter()
    for i in range(n):
        call(i)
    host = (time.perf_counter() - t0) / n
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / n
    return {"wall_us_per_call": round(wall * 1e6, 1), "host_us_per_call": round(host * 1e6, 1),
            "note": "host time is what the Python entry costs per call; it overlaps the previous call's kernel"}


def bench_scan_per_channel_bc(dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16):
    """The shape the reference's Mamba1 module calls with (src/ssm/modules/mamba1.py:229-247): B and C as
    (B, D, N, L), one group per channel, so the projections dominate the traffic."""
    from ssm_amd import configs
    from ssm_amd.ops import ScanPlan
    g = configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=0))
    gen = torch.Generator(device="cuda").manual_seed(1)
    Bm = torch.randn(batch, dim, nstate, length, generator=gen, device="cuda", dtype=torch.float32).to(dtype)
    Cm = torch.randn(batch, dim, nstate, length, generator=gen, device="cuda", dtype=torch.float32).to(dtype)
    plan = ScanPlan(g["u"], g["delta"], g["A"], Bm, Cm, g["D"], g["z"], g["dt_bias"], True, True)
    us = _time_us(lambda i: plan.run(), iters=10)
    elt = 2 if dtype != torch.float32 else 4
    nbytes = configs.scan_fwd_bytes(batch, dim, length, nstate, elt, groups=dim)
    # backward of the same call (a wave per row; dB and dC written straight to their place in B's own type)
    from ssm_amd.ops import _scan_backward
    cs_plan = ScanPlan(g["u"], g["delta"], g["A"], Bm, Cm, g["D"], g["z"], g["dt_bias"], True, False, want_chunk_states=True)
    cs_plan.run()
    go = torch.randn(batch, dim, length, generator=gen, device="cuda", dtype=torch.float32).to(dtype)
    bus = _time_us(lambda i: _scan_backward(go, None, g["u"], g["delta"], g["A"], Bm, Cm, g["D"], g["z"], g["dt_bias"], True,
                                            chunk_states=cs_plan.chunk_states, grads_in_input_dtype=True), iters=10)
    bbytes = 7 * elt * batch * dim * length + 4 * elt * batch * dim * nstate * length
    return {"kernel_us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1),
            "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes,
            "bwd_us": round(bus, 1), "bwd_GBps": round(bbytes / bus / 1e3, 1),
            "bwd_frac_hbm": round(bbytes / bus / 1e3 / HBM_PEAK_GBPS, 4), "bwd_algorithmic_bytes": bbytes,
            "shape": "B, C (8, 1536, 16, 2048) bf16: one B/C group per channel"}


def bench_scan_const_bc(dtype=torch.bfloat16, batch=8, dim=1536, length=2048, nstate=16):
    """Config 1's shape with projections constant in time, ``B`` and ``C`` of shape ``(D, N)`` (the reference's other
    accepted form, src/ssm/ops/python/reference.py:22-56; what its Mamba1 block's projections reduce to with the
    per-token gate outside the recurrence): forward, and backward from the forward's chunk states."""
    from ssm_amd import configs
    from ssm_amd.ops import ScanPlan, _scan_backward
    g = configs.to_device(configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=0))
    gen = torch.Generator(device="cuda").manual_seed(1)
    Bm = torch.randn(dim, nstate, generator=gen, device="cuda")
    Cm = torch.randn(dim, nstate, generator=gen, device="cuda")
    plan = ScanPlan(g["u"], g["delta"], g["A"], Bm, Cm, g["D"], g["z"], g["dt_bias"], True, True)
    us = _time_us(lambda i: plan.run(), iters=20, warmup=20)
    cs_plan = ScanPlan(g["u"], g["delta"], g["A"], Bm, Cm, g["D"], g["z"], g["dt_bias"], True, False, want_chunk_states=True)
    cs_plan.run()
    go = torch.randn(batch, dim, length, generator=gen, device="cuda", dtype=torch.float32).to(dtype)
    bus = _time_us(lambda i: _scan_backward(go, None, g["u"], g["delta"], g["A"], Bm, Cm, g["D"], g["z"], g["dt_bias"], True,
                                            chunk_states=cs_plan.chunk_states), iters=20, warmup=30)
    elt = 2 if dtype != torch.float32 else 4
    fbytes, bbytes = 4 * elt * batch * dim * length, 7 * elt * batch * dim * length
    return {"fwd_us": round(us, 1), "fwd_frac_hbm": round(fbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
            "bwd_us": round(bus, 1), "bwd_frac_hbm": round(bbytes / bus / 1e3 / HBM_PEAK_GBPS, 4),
            "shape": "B=8 D=1536 L=2048 N=16 bf16 activations, B and C (1536, 16) float32"}


def bench_stream():
    """What plain element-wise kernels of the framework reach on this GPU, as the yardstick for the streaming
    kernels: ``dst = 2 * src`` and ``dst.copy_(src)`` on float32 buffers of 64 MiB (source and destination fit the
    256 MB memory-side cache together) and of 1 GiB (they do not)."""
    out = {}
    for mib in (64, 1024):
        n = mib * 1024 * 1024 // 4
        src = torch.empty(n, device="cuda", dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        moved = 2.0 * n * 4
        us = _time_us(lambda i: torch.mul(src, 2.0, out=dst), iters=30, warmup=10)
        out[f"scale_{mib}MiB_GBps"] = round(moved / us / 1e3, 1)
        us = _time_us(lambda i: dst.copy_(src), iters=30, warmup=10)
        out[f"copy_{mib}MiB_GBps"] = round(moved / us / 1e3, 1)
        del src, dst
    out["frac_hbm_peak_scale_1GiB"] = round(out["scale_1024MiB_GBps"] / HBM_PEAK_GBPS, 4)
    return out


def cpu_baseline_scan(dtype=torch.bfloat16, dim=1536, length=2048, nstate=16, budget_s=15.0):
    """Time the CPU restatement of the reference's Python loop on a batch slice
    of the headline workload; returns GB/s of the same algorithmic bytes."""
    from oracle import ops_oracle
    from ssm_amd import configs

    elt = 2 if dtype != torch.float32 else 4
    batch = 1
    inp = configs.scan_inputs(batch, dim, length, nstate, dtype=dtype, seed=0)

    def once():
        t0 = time.perf_counter()
        ops_oracle.selective_scan(inp["u"], inp["delta"], inp["A"], inp["B"], inp["C"], D=inp["D"],
                                  z=inp["z"], dt_bias=inp["dt_bias"], softplus=True,
                                  return_last_state=True)
        return time.perf_counter() - t0

    first = once()
    reps = max(1, min(5, int(budget_s / max(first, 1e-3)) - 1))
    times = [first] + [once() for _ in range(reps)]
    best = sorted(times)[len(times) // 2]
    nbytes = configs.scan_fwd_bytes(batch, dim, length, nstate, elt)
    # configuration 0 at full size (B=1, D=512, L=2048, N=16, float32): the one case the reference publishes
    # a time for (1012.9 ms on its authors' CPU, README.md:53 of the reference)
    c0 = configs.scan_inputs(1, 512, 2048, 16, dtype=torch.float32, seed=0)
    t0s = []
    for _ in range(3):
        t0 = time.perf_counter()
        ops_oracle.selective_scan(c0["u"], c0["delta"], c0["A"], c0["B"], c0["C"], D=c0["D"], z=c0["z"],
                                  dt_bias=c0["dt_bias"], softplus=True, return_last_state=True)
        t0s.append(time.perf_counter() - t0)
    return dict(value=nbytes / best / 1e9, unit="GB/s", cores=torch.get_num_threads(), kind="port",
                config0_ms=round(sorted(t0s)[1] * 1e3, 1), config0_reference_published_ms=1012.9,
                config2_decode=cpu_baseline_decode(), config3_ssd=cpu_baseline_ssd(),
                sample=f"selective_scan fwd, batch slice B={batch} of the headline workload "
                       f"(D={dim}, L={length}, N={nstate}, {str(dtype).split('.')[-1]}), "
                       f"median of {len(times)} runs, {best * 1e3:.0f} ms each; "
                       f"host has {os.cpu_count()} logical cpus",
                seconds_per_call=best)


def cpu_baseline_decode(batch=64, dim=5120, nstate=16, width=4, steps=32):
    """Config 2 on the host: the tensor operations of the reference's ``Mamba1.step`` (window roll, tap sum,
    SiLU: src/ssm/modules/mamba1.py:345-381) followed by the oracle's state step, at full width, for a bounded
    number of the 512 steps (every step costs the same)."""
    from oracle import ops_oracle
    from ssm_amd import configs

    g = torch.Generator().manual_seed(2)
    state = torch.randn(batch, dim, nstate, generator=g)
    window = torch.randn(batch, dim, width, generator=g).to(torch.bfloat16)
    A = -torch.arange(1, nstate + 1, dtype=torch.float32).repeat(dim, 1)
    D, bias = torch.ones(dim), configs.inverse_softplus_dt(dim, g)
    w, cb = torch.rand(dim, width, generator=g) - 0.5, torch.randn(dim, generator=g) * 0.02
    x, z, dt = (torch.randn(batch, dim, generator=g).to(torch.bfloat16) for _ in range(3))
    Bm, Cm = (torch.randn(batch, 1, nstate, generator=g).to(torch.bfloat16) for _ in range(2))

    def step():
        nonlocal window
        window = torch.roll(window, -1, dims=-1)
        window[..., -1] = x
        xc = torch.nn.functional.silu((window.float() * w).sum(-1) + cb).to(torch.bfloat16)
        ops_oracle.selective_state_step(state, xc, dt, A, Bm, Cm, D=D, z=z, dt_bias=bias, softplus=True)

    step()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    per = (time.perf_counter() - t0) / steps
    return {"us_per_step": round(per * 1e6, 1), "steps_timed": steps, "of_steps": 512,
            "shape": f"B={batch}, D={dim}, N={nstate}, K={width}, bf16 activations, fp32 state"}


def cpu_baseline_ssd(length=4096, heads=2, hdim=64, nstate=128):
    """Config 3 on the host: the token-by-token recurrence that fixes the SSD's semantics (float32, two of the
    320 (batch, head) pairs over the whole sequence; pairs are independent, so the whole call costs 160 times
    this with the same threads)."""
    from oracle import ssd_oracle

    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, length, heads, hdim, generator=g)
    dt = torch.rand(1, length, heads, generator=g) * 0.1
    A = -(torch.rand(heads, generator=g) * 15 + 1)
    Bm, Cm = torch.randn(1, length, 1, nstate, generator=g), torch.randn(1, length, 1, nstate, generator=g)
    z = torch.randn(1, length, heads, hdim, generator=g)
    t0 = time.perf_counter()
    ssd_oracle.ssd_sequential(x, dt, A, Bm, Cm, D=torch.ones(heads), z=z, acc=torch.float32)
    sec = time.perf_counter() - t0
    pairs = 4 * 80
    return {"ms_for_sample": round(sec * 1e3, 1), "sample": f"{heads} of {pairs} (batch, head) pairs, L={length}, P={hdim}, N={nstate}",
            "ms_whole_call_extrapolated": round(sec * 1e3 * pairs / heads, 1)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="only the headline kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB elementwise copy (dst = src + 0) three times: "
                         "the reference for hardware byte counters")
    ap.add_argument("--only", default=None,
                    choices=["scan_bwd", "mixer", "conv", "norm", "decode", "ssd", "ssd_train", "dscan", "model", "model1",
                             "scan_facade", "scan_per_channel_bc", "scan_const_bc", "stream"],
                    help="run one of the secondary workloads alone and print its figures "
                         "(for profiling that kernel; not the benchmark line)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: every operator on this path is independent per "
              "(batch, channel) row and no multi-GPU figure is defined; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm device", file=sys.stderr)
        sys.exit(1)

    if args.copy_calibration:
        src = torch.full((64 * 1024 * 1024,), 1.0, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.add(src, 0.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    from ssm_amd import configs

    if args.only:
        fn = {"scan_bwd": bench_scan_bwd, "conv": bench_conv, "norm": bench_norm, "decode": bench_decode,
              "mixer": bench_mixer_config1, "ssd": bench_ssd, "ssd_train": bench_ssd_train, "dscan": bench_dscan, "model": bench_model,
              "model1": bench_model1, "scan_facade": bench_scan_facade,
              "scan_per_channel_bc": bench_scan_per_channel_bc, "scan_const_bc": bench_scan_const_bc,
              "stream": bench_stream}[args.only]
        bench_scan_fwd(1, 0)            # the untimed spin-up of the default run, so that figures compare
        print(json.dumps({args.only: fn()}))
        return

    r = bench_scan_fwd(args.steps, args.warmup)
    value = r["bytes"] / r["wall_s"] / 1e9
    achieved = r["bytes"] / (r["kernel_ms"] * 1e-3) / 1e9
    counters = headline_counters()
    valu = None
    if counters["valu_insts"]:
        # vector-ALU instructions of one launch at the nominal 4 clocks each on 1024 SIMDs, against the kernel's time
        busy_s = counters["valu_insts"] * 4.0 / (SIMDS * CLOCK_GHZ * 1e9)
        valu = {"insts_per_launch": int(counters["valu_insts"]), "clocks_per_inst": 4, "clock_ghz": CLOCK_GHZ,
                "simds": SIMDS, "frac": round(busy_s / (r["kernel_ms"] * 1e-3), 4),
                "insts_per_state_step": round(counters["valu_insts"] * 64.0 / (8 * 1536 * 2048 * 16), 2),
                "source": "profiles/scan_fwd_bf16_headline_pmc_SQ.txt"}
    line = {
        "metric": "selective_scan GB/s (%HBM peak)",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(r["wall_s"] * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "selective_scan forward, B=8 D=1536 L=2048 N=16, bf16 activations, "
                               "fp32 state, G=1 time-varying B/C, D skip, z gate, dt_bias, softplus",
                   "io_dtype": "bf16", "arithmetic": "fp32", "untimed_spin_up_launches": SPIN_UP_LAUNCHES,
                   "tokens_per_step": r["tokens"],
                   "tokens_per_s": round(r["tokens"] / r["wall_s"], 1),
                   "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": counters["traffic"], "traffic_source": counters["source"],
                     "kernel": "scan_fwd_fast_kernel<bf16, bf16, 32 lanes per row, 2 rows in turn, 12 waves>",
                     "kernel_us": round(r["kernel_ms"] * 1e3, 2),
                     "algorithmic_bytes": r["bytes"], "valu": valu},
    }
    if not args.no_extra:
        extra = {}
        r32 = bench_scan_fwd(max(10, args.steps // 2), 3, dtype=torch.float32)
        a32 = r32["bytes"] / (r32["kernel_ms"] * 1e-3) / 1e9
        extra["selective_scan_fwd_fp32_io"] = {
            "kernel_us": round(r32["kernel_ms"] * 1e3, 2), "GBps": round(a32, 1),
            "frac_hbm": round(a32 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": r32["bytes"]}
        extra["selective_scan_fwd_through_ops_entry"] = bench_scan_facade()
        extra["selective_scan_fwd_per_channel_bc"] = bench_scan_per_channel_bc()
        extra["selective_scan_constant_bc"] = bench_scan_const_bc()
        extra["selective_scan_bwd_bf16"] = bench_scan_bwd()
        extra["mamba1_mixer_config1_fwd_bwd"] = bench_mixer_config1()
        extra["dw_causal_conv_bf16"] = bench_conv()
        extra["fused_add_rmsnorm"] = bench_norm()
        extra["decode_step_config2"] = bench_decode()
        extra["ssd_chunk_scan_diagonal"] = bench_dscan()
        extra["ssd_combined_config3"] = bench_ssd()
        extra["ssd_config3_backward_and_packed"] = bench_ssd_train()
        extra["mamba2_130m_style_model_config4"] = bench_model()
        extra["mamba1_130m_style_model_config1_shape"] = bench_model1()
        extra["elementwise_streaming_yardstick"] = bench_stream()
        line["extra"] = extra
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_scan()
    print(json.dumps(line))


if __name__ == "__main__":
    main()

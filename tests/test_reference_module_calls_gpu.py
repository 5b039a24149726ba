"""The operator calls of the reference's own modules, argument for argument.

``Mamba1.forward`` (/root/reference/src/ssm/modules/mamba1.py:201-246) convolves a permuted view of the input
projection, promotes to its compute type (float32 for 16-bit activations) and calls ``selective_scan`` by keyword
with ``B`` and ``C`` expanded per channel and step, ``(B, D, N, L)``, ``delta`` and the gate as permuted views;
``Mamba1.step`` (:327-381) calls ``selective_state_step`` on a batch slice of its cache with per-row ``(B, D, N)``
projections; ``Mamba2.forward`` (mamba2.py:157-199) convolves the same way and calls ``ssd_chunk_scan`` with ``A``,
``B``, ``C``, ``D`` as slices of ``(H, P)`` parameters and ``seq_lens`` as a Python list.  The tensors below are
built the way those lines build them (same shapes, types, views and keywords, random values); the results are the
oracle's on the same tensors."""

import pytest
import torch

from oracle import ops_oracle as O
from tests.closeness import fp32_close, half_close

pytestmark = pytest.mark.gpu


def _ops():
    from ssm_amd import ops
    return ops


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_mamba1_forward_calls(dtype):
    batch, seqlen, inner, nstate, width = 2, 96, 24, 8, 4
    g = torch.Generator().manual_seed(31)
    compute = torch.float32                                      # _compute_dtype: 16-bit activations compute in float32
    in_proj = torch.randn(batch, seqlen, 2 * inner, generator=g).to(dtype)
    conv_weight, conv_bias = torch.randn(inner, width, generator=g) * 0.3, torch.randn(inner, generator=g) * 0.1
    Bp, Cp = torch.randn(inner, nstate, generator=g), torch.randn(inner, nstate, generator=g)
    A_log, Dp, dt_bias = torch.rand(inner, nstate, generator=g), torch.ones(inner), torch.randn(inner, generator=g)
    delta_lin = torch.randn(batch, seqlen, inner, generator=g)
    B_proj, C_proj = torch.randn(batch, seqlen, inner, generator=g) * 0.5, torch.randn(batch, seqlen, inner, generator=g) * 0.5

    def forward(ops, dev):
        to = lambda t: t.to(dev)
        projected, gate = to(in_proj).chunk(2, dim=-1)
        conv_input = projected.permute(0, 2, 1)
        conv_out = ops.dw_causal_conv(conv_input, to(conv_weight), bias=to(conv_bias), activation="silu").to(compute)
        delta = to(delta_lin).permute(0, 2, 1)
        u = conv_out
        z = gate.permute(0, 2, 1).to(compute)
        B_gates, C_gates = to(B_proj).permute(0, 2, 1).to(compute), to(C_proj).permute(0, 2, 1).to(compute)
        B = to(Bp).to(compute).view(1, inner, nstate, 1) * (1 + B_gates.unsqueeze(2))
        C = to(Cp).to(compute).view(1, inner, nstate, 1) * (1 + C_gates.unsqueeze(2))
        A = -torch.exp(to(A_log).to(compute))
        out = ops.selective_scan(u=u, delta=delta, A=A, B=B, C=C, D=to(Dp), z=z, dt_bias=to(dt_bias), softplus=True)
        return conv_out, out

    conv_gpu, out_gpu = forward(_ops(), "cuda")
    conv_cpu, out_cpu = forward(O, "cpu")
    assert conv_gpu.shape == (batch, inner, seqlen) and out_gpu.shape == (batch, inner, seqlen)
    assert out_gpu.dtype == compute
    if dtype == torch.float32:
        fp32_close(conv_gpu.cpu(), conv_cpu.double(), conv_cpu, what="conv")
        fp32_close(out_gpu.cpu(), out_cpu.double(), out_cpu, what="scan", rtol=1e-4, atol_rms=1e-4)
    else:
        half_close(conv_gpu.cpu(), conv_cpu, what="conv")
        # the scan reads the GPU's own conv output (rounded to bfloat16 before the promotion, as the module rounds it)
        _, out_ref = (lambda c: (c, O.selective_scan(
            u=c, delta=delta_lin.permute(0, 2, 1), A=-torch.exp(A_log),
            B=Bp.view(1, inner, nstate, 1) * (1 + B_proj.permute(0, 2, 1).unsqueeze(2)),
            C=Cp.view(1, inner, nstate, 1) * (1 + C_proj.permute(0, 2, 1).unsqueeze(2)),
            D=Dp, z=in_proj.chunk(2, dim=-1)[1].permute(0, 2, 1).to(compute), dt_bias=dt_bias, softplus=True)))(conv_gpu.cpu())
        fp32_close(out_gpu.cpu(), out_ref.double(), out_ref, what="scan", rtol=1e-4, atol_rms=1e-4)


def test_mamba1_step_call_on_a_slice_of_the_cache():
    batch, inner, nstate = 3, 24, 8
    g = torch.Generator().manual_seed(32)
    ssm_cache = torch.randn(batch + 2, inner, nstate, generator=g)
    conv_out, delta, z = (torch.randn(batch, inner, generator=g) for _ in range(3))
    A = -torch.exp(torch.rand(inner, nstate, generator=g))
    Bp, Cp = torch.randn(inner, nstate, generator=g), torch.randn(inner, nstate, generator=g)
    B_proj, C_proj = torch.randn(batch, inner, generator=g) * 0.5, torch.randn(batch, inner, generator=g) * 0.5
    Dp, dt_bias = torch.ones(inner), torch.randn(inner, generator=g)

    def step(ops, dev):
        to = lambda t: t.to(dev)
        cache = to(ssm_cache).clone()
        ssm_state = cache[1:1 + batch]                                   # ssm_cache[batch_start:batch_end]
        B = to(Bp).unsqueeze(0) * (1 + to(B_proj).unsqueeze(-1))          # (B, D, N)
        C = to(Cp).unsqueeze(0) * (1 + to(C_proj).unsqueeze(-1))
        out = ops.selective_state_step(ssm_state, to(conv_out), to(delta), to(A), B, C, to(Dp), z=to(z),
                                       dt_bias=to(dt_bias), softplus=True)
        return out, cache

    out_gpu, cache_gpu = step(_ops(), "cuda")
    out_cpu, cache_cpu = step(O, "cpu")
    fp32_close(out_gpu.cpu(), out_cpu.double(), out_cpu, what="y")
    fp32_close(cache_gpu.cpu(), cache_cpu.double(), cache_cpu, what="cache")
    assert torch.equal(cache_gpu[0].cpu(), ssm_cache[0]) and torch.equal(cache_gpu[-1].cpu(), ssm_cache[-1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_mamba2_forward_calls(dtype):
    batch, seqlen, heads, headdim, width = 2, 80, 3, 8, 4
    extra = 5                                                        # channels of the projection beyond the SSM's
    ssm_dim = heads * headdim
    g = torch.Generator().manual_seed(33)
    compute = torch.float32
    projected = torch.randn(batch, seqlen, ssm_dim + extra, generator=g).to(dtype)
    conv_weight, conv_bias = torch.randn(ssm_dim + extra, width, generator=g) * 0.3, torch.randn(ssm_dim + extra, generator=g) * 0.1
    dt_w, dt_b = torch.randn(heads + 1, headdim, generator=g) * 0.3, torch.randn(heads + 1, generator=g)
    A_log, Bp, Cp = (torch.randn(heads + 1, headdim, generator=g) * 0.5 for _ in range(3))
    Dp = torch.ones(heads + 1, headdim)
    seq_lens = [seqlen, 37]

    def forward(ops, dev):
        to = lambda t: t.to(dev)
        conv_out_cf = ops.dw_causal_conv(to(projected).permute(0, 2, 1), to(conv_weight), bias=to(conv_bias),
                                         activation="silu").to(compute)
        ssm_heads = conv_out_cf[:, :ssm_dim].contiguous().view(batch, heads, headdim, seqlen)
        X = ssm_heads.permute(0, 3, 1, 2).contiguous()
        dt = torch.einsum("bhpl,hp->bhl", ssm_heads.to(compute), to(dt_w)[:heads].to(compute))
        dt = torch.nn.functional.softplus((dt + to(dt_b)[:heads].view(1, heads, 1)).transpose(1, 2))
        return ops.ssd_chunk_scan(X=X, dt=dt, A=-torch.exp(to(A_log)[:heads].to(compute)), B=to(Bp)[:heads],
                                  C=to(Cp)[:heads], chunk_size=16, D=to(Dp)[:heads], z=None,
                                  seq_meta={"seq_lens": seq_lens})

    got, want = forward(_ops(), "cuda").cpu(), forward(O, "cpu")
    assert got.shape == (batch, seqlen, heads, headdim) and got.dtype == compute
    assert bool((got[1, 37:] == 0).all())
    if dtype == torch.float32:
        fp32_close(got, want.double(), want, what="Y", rtol=1e-4, atol_rms=1e-4)
    else:
        half_close(got, want, what="Y")            # the two chains round the conv output to bfloat16 separately


def test_mamba1_projections_factor_into_a_scan_with_constant_projections():
    """``Mamba1.forward`` (src/ssm/modules/mamba1.py:229-247) materialises ``B = base_B (1 + B_gates)`` and ``C`` likewise
    as ``(B, D, N, L)`` tensors, 16 times the activations.  The time-varying factor does not depend on the state
    index, so it moves out of the recurrence: the same output is the scan with the constant ``(D, N)`` projections
    on ``u (1 + B_gates)``, its result scaled by ``(1 + C_gates)``, plus the skip term and the gate outside.  Checked
    here for values and every gradient through the operators of this package (float32, 1e-4)."""
    ops = _ops()
    batch, seqlen, inner, nstate = 2, 300, 48, 8
    g = torch.Generator().manual_seed(41)
    leaves = dict(
        u=torch.randn(batch, inner, seqlen, generator=g), delta=torch.randn(batch, inner, seqlen, generator=g),
        A=-torch.exp(torch.rand(inner, nstate, generator=g)), base_B=torch.randn(inner, nstate, generator=g),
        base_C=torch.randn(inner, nstate, generator=g), gB=torch.randn(batch, inner, seqlen, generator=g) * 0.5,
        gC=torch.randn(batch, inner, seqlen, generator=g) * 0.5, D=torch.randn(inner, generator=g),
        z=torch.randn(batch, inner, seqlen, generator=g), dt_bias=torch.randn(inner, generator=g))
    go = torch.randn(batch, inner, seqlen, generator=g).cuda()

    def run(factored):
        t = {k: v.clone().cuda().requires_grad_() for k, v in leaves.items()}
        if factored:
            core = ops.selective_scan(t["u"] * (1 + t["gB"]), t["delta"], t["A"], t["base_B"], t["base_C"],
                                      dt_bias=t["dt_bias"], softplus=True)
            y = (core * (1 + t["gC"]) + t["D"].view(1, -1, 1) * t["u"]) * torch.nn.functional.silu(t["z"])
        else:
            Bm = t["base_B"].view(1, inner, nstate, 1) * (1 + t["gB"].unsqueeze(2))
            Cm = t["base_C"].view(1, inner, nstate, 1) * (1 + t["gC"].unsqueeze(2))
            y = ops.selective_scan(t["u"], t["delta"], t["A"], Bm, Cm, D=t["D"], z=t["z"], dt_bias=t["dt_bias"], softplus=True)
        y.backward(go)
        return y.detach(), {k: v.grad for k, v in t.items()}

    y_m, g_m = run(False)
    y_f, g_f = run(True)
    scale = lambda t: float(t.double().pow(2).mean().sqrt()) + 1e-30
    assert float((y_m - y_f).abs().max()) <= 1e-4 * scale(y_m)
    for k in leaves:
        assert float((g_m[k] - g_f[k]).abs().max()) <= 1e-4 * scale(g_m[k]) + 1e-6, k

"""GPU parity of the state-space-duality (Mamba-2) operators: component vectors
shipped by the reference, the float64 sequential recurrence, and the bf16 MFMA
kernels against the shape-generic kernels at the benchmark shape."""

import pytest
import torch

from oracle import ssd_oracle as S
from tests import fixtures as fx

pytestmark = pytest.mark.gpu
TF32 = dict(rtol=2e-2, atol=2e-2)          # the shipped vectors were produced with TF32 dots
FP32_TOL = dict(rtol=1e-4, atol=1e-4)


def ssd():
    from ssm_amd.ops import ssd as m
    return m


# gradients of 16-bit calls: sums of many rounded products
GRAD_ATOL_RMS, GRAD_MEAN_RMS = 6e-2, 2e-2
# dA, per head, against the sum over batch and time of the magnitudes of its terms dt_t q_t (seen over some two hundred
# random cases: 1.4e-2 at worst with 16-bit operands, median 5e-4; 1.1e-4 and 3e-6 in float32)
DA_TERM_BAR_HALF, DA_TERM_BAR_F32 = 2e-2, 5e-4


def half_close(got, want, what="", atol_rms=4e-2, mean_rms=3e-3, rtol=2e-2):
    """16-bit operands against a float64 (or float32) result: every element within ``rtol`` of itself or
    ``atol_rms`` of the result's root mean square (not of its maximum: the largest element says nothing about
    what an ordinary one may be off by), and the mean error an order of magnitude below that."""
    got, want = got.detach().float().cpu().double(), want.detach().cpu().double()
    rms = float(want.pow(2).mean().sqrt()) + 1e-30
    err = (got - want).abs()
    torch.testing.assert_close(got, want, rtol=rtol, atol=atol_rms * rms,
                               msg=lambda m: f"{what}: {m} (max err / rms {float(err.max()) / rms:.3e}, "
                                             f"mean err / rms {float(err.mean()) / rms:.3e})")
    assert float(err.mean()) < mean_rms * rms, f"{what}: mean err / rms {float(err.mean()) / rms:.3e}"


def cu(t):
    return None if t is None else t.cuda()


def kernels_taken(fn):
    """Run ``fn()`` once more on the test-hooks build of the library (the same sources compiled with
    ``-DSSM_TEST_HOOKS``, include/ssm_amd_testing.h) and return which matrix-core kernels its calls launched:
    bit 0 bmm_chunk, bit 1 chunk_state, bit 2 chunk_scan, bit 3 the one-pass forward.  The shipped library
    picks its kernels by the same code but keeps no record."""
    from ssm_amd import _lib
    with _lib.test_hooks_build() as lib:
        lib.ssm_ssd_mfma_launches()
        fn()
        return lib.ssm_ssd_mfma_launches()


def test_chunk_cumsum_vectors():
    rec = fx.upstream("ssd_components", "chunk_cumsum"); i = rec["inputs"]
    dA, dt_c = ssd().chunk_cumsum(cu(i["dt"]), cu(i["A"]), 3, dt_bias=cu(i["dt_bias"]), dt_softplus=True)
    torch.testing.assert_close(dA.cpu(), rec["outputs"]["dA_cumsum"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dt_c.cpu(), rec["outputs"]["dt_out"], rtol=1e-5, atol=1e-6)
    rec = fx.upstream("ssd_components", "chunk_cumsum_clamped"); i = rec["inputs"]
    dA, dt_c = ssd().chunk_cumsum(cu(i["dt"]), cu(i["A"]), 3, dt_limit=(0.01, 1.0))
    torch.testing.assert_close(dA.cpu(), rec["outputs"]["dA_cumsum"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dt_c.cpu(), rec["outputs"]["dt_out"], rtol=1e-5, atol=1e-6)


def test_bmm_vectors():
    rec = fx.upstream("ssd_bmm", "basic"); i = rec["inputs"]
    torch.testing.assert_close(ssd().bmm_chunk(cu(i["a"]), cu(i["b"]), 3).cpu(), rec["outputs"]["out"], **TF32)
    rec = fx.upstream("ssd_bmm", "grouped"); i = rec["inputs"]
    torch.testing.assert_close(ssd().bmm_chunk(cu(i["a"]), cu(i["b"]), 3).cpu(), rec["outputs"]["out"], **TF32)
    rec = fx.upstream("ssd_bmm", "causal_seq"); i = rec["inputs"]
    got = ssd().bmm_chunk(cu(i["a"]), cu(i["b"]), 3, seq_idx=cu(i["seq_idx"]), causal=True).cpu()
    tri = torch.tril(torch.ones(3, 3, dtype=torch.bool))
    torch.testing.assert_close(got[..., tri], rec["outputs"]["out"][..., tri], **TF32)


def test_chunk_state_vector():
    rec = fx.upstream("ssd_components", "chunk_state"); i = rec["inputs"]
    st = ssd().chunk_state(cu(i["B"]), cu(i["x"]), cu(i["dt"]), cu(i["dA_cumsum"]))
    torch.testing.assert_close(st.cpu(), rec["outputs"]["states"], **TF32)


def test_state_passing_vector():
    rec = fx.upstream("ssd_components", "state_passing"); i = rec["inputs"]
    entering, final = ssd().state_passing(cu(i["states"]), cu(i["dA_last"]))
    torch.testing.assert_close(entering.cpu(), rec["outputs"]["states_passed"], rtol=1e-5, atol=1e-6)
    b, nc, h, p, n = i["states"].shape
    torch.testing.assert_close(final.cpu().reshape(b, h, p * n), rec["outputs"]["final_states"], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("case", ["chunk_scan_matrix_D_z", "chunk_scan_vector_D"])
def test_chunk_scan_vectors(case):
    rec = fx.upstream("ssd_components", case); i = rec["inputs"]
    y = ssd().chunk_scan(cu(i["B"]), cu(i["C"]), cu(i["x"]), cu(i["dt"]), cu(i["dA_cumsum"]), cu(i["states"]),
                         D=cu(i["D"]), z=cu(i.get("z")))
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], **TF32)


def test_combined_vector():
    rec = fx.upstream("ssd_combined", "combined_full"); i = rec["inputs"]
    y, fin = ssd().ssd_combined(cu(i["X"]), cu(i["dt"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), int(i["chunk_size"]),
                                D=cu(i["D"]), z=cu(i["z"]), dt_bias=cu(i["dt_bias"]),
                                initial_states=cu(i["initial_states"]), dt_softplus=True, return_final_states=True)
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], **TF32)
    torch.testing.assert_close(fin.cpu(), rec["outputs"]["final_states"], **TF32)


def make(seed, b, l, h, p, g, n, dtype=torch.float32, d_mat=False, use_z=True, use_init=True):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(b, l, h, p, generator=gen).to(dtype)
    dt = torch.nn.functional.softplus(torch.randn(b, l, h, generator=gen) - 3.0)
    A = -(torch.rand(h, generator=gen) * 15 + 1)
    Bm = torch.randn(b, l, g, n, generator=gen).to(dtype)
    Cm = torch.randn(b, l, g, n, generator=gen).to(dtype)
    D = torch.randn(h, p, generator=gen) if d_mat else torch.ones(h)
    z = torch.randn(b, l, h, p, generator=gen).to(dtype) if use_z else None
    init = torch.randn(b, h, p, n, generator=gen) if use_init else None
    return dict(x=x, dt=dt, A=A, B=Bm, C=Cm, D=D, z=z, init=init)


def _leaves(inp, names, dtype=None):
    out = {}
    for k in names:
        v = inp.get(k)
        out[k] = None if v is None else v.clone().requires_grad_(True)
    return out


@pytest.mark.parametrize("shape,Q,dtype,d_mat,use_z,use_init,softplus", [
    ((2, 19, 4, 5, 2, 6), 8, torch.float32, False, True, True, True),
    ((1, 12, 2, 3, 1, 4), 4, torch.float32, True, False, False, False),
    ((2, 64, 4, 16, 4, 32), 16, torch.float32, False, True, True, True),
    ((2, 256, 4, 64, 1, 64), 64, torch.bfloat16, False, True, True, True),
    ((1, 512, 2, 64, 2, 128), 256, torch.bfloat16, True, True, False, True),
    ((1, 256, 2, 128, 1, 64), 64, torch.bfloat16, False, True, True, True),
], ids=lambda v: str(v).replace(" ", ""))
def test_combined_gradients_match_float64_autograd(shape, Q, dtype, d_mat, use_z, use_init, softplus):
    """All nine gradients of (y, final_states) against float64 autograd through the token-by-token
    recurrence, for random upstream gradients of both outputs."""
    b, l, h, p, g, n = shape
    gen = torch.Generator().manual_seed(23 + l)
    x = torch.randn(b, l, h, p, generator=gen).to(dtype)
    dt = torch.randn(b, l, h, generator=gen) * 0.5 if softplus else torch.rand(b, l, h, generator=gen) * 0.3
    A = -(torch.rand(h, generator=gen) + 0.2)
    Bm = (torch.randn(b, l, g, n, generator=gen) * 0.5).to(dtype)
    Cm = (torch.randn(b, l, g, n, generator=gen) * 0.5).to(dtype)
    D = torch.randn(h, p, generator=gen) if d_mat else torch.randn(h, generator=gen)
    z = torch.randn(b, l, h, p, generator=gen).to(dtype) if use_z else None
    bias = torch.randn(h, generator=gen) * 0.3 if softplus else None
    init = torch.randn(b, h, p, n, generator=gen) if use_init else None
    dout = torch.randn(b, l, h, p, generator=gen)
    dfin = torch.randn(b, h, p, n, generator=gen)
    names = ["x", "dt", "A", "B", "C", "D", "z", "dt_bias", "init"]
    vals = dict(x=x, dt=dt, A=A, B=Bm, C=Cm, D=D, z=z, dt_bias=bias, init=init)
    # float64 reference
    w = {k: (None if v is None else v.double().clone().requires_grad_(True)) for k, v in vals.items()}
    # A given per step (the same value at every step): its gradient holds the terms dt_t q_t whose sum is dA
    A_steps = A.double()[None, None, :].expand(b, l, h).clone().requires_grad_(True)
    y64, f64 = S.ssd_sequential(w["x"], w["dt"], A_steps, w["B"], w["C"], D=w["D"], z=w["z"], dt_bias=w["dt_bias"],
                                dt_softplus=softplus, initial_states=w["init"])
    ((y64 * dout.double()).sum() + (f64 * dfin.double()).sum()).backward()
    w["A"].grad = A_steps.grad.sum(dim=(0, 1))
    dA_terms = A_steps.grad.abs().sum(dim=(0, 1))
    # device
    d = {k: (None if v is None else v.cuda().clone().requires_grad_(True)) for k, v in vals.items()}
    y, fin = ssd().ssd_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, D=d["D"], z=d["z"], dt_bias=d["dt_bias"],
                                initial_states=d["init"], dt_softplus=softplus, return_final_states=True)
    ((y.float() * dout.cuda()).sum() + (fin * dfin.cuda()).sum()).backward()
    for k in names:
        if vals[k] is None:
            continue
        want = w[k].grad
        got = d[k].grad.float().cpu().double()
        assert got.shape == want.shape and d[k].grad.dtype == vals[k].dtype
        if k == "A":
            # a sum over the sequence whose terms cancel: every head against the sum of the magnitudes of its own
            # terms (a head's own value, or the largest head's, says little about what the sum may be off by)
            bar = DA_TERM_BAR_F32 if dtype == torch.float32 else DA_TERM_BAR_HALF
            ratio = (got - want).abs() / (dA_terms + 1e-30)
            assert bool((ratio <= bar).all()), f"gradient of A: error / sum |dt_t q_t| per head {ratio.tolist()}"
        elif dtype == torch.float32:
            scale = float(want.abs().max())
            torch.testing.assert_close(got, want, rtol=2e-3, atol=2e-4 * scale, msg=lambda m: f"{k}: {m}")
        else:
            half_close(got, want, f"gradient of {k}", atol_rms=GRAD_ATOL_RMS, mean_rms=GRAD_MEAN_RMS, rtol=3e-2)


def test_combined_gradient_vector_on_the_decaying_head():
    """Gradients shipped by the reference for loss = y.sum() (dt_softplus, D matrix, z, initial
    state).  Head 1 of that case has A > 0, where the upstream kernels clamp the decay inside
    chunks; the comparison is made on head 0 (A < 0), for the inputs that belong to one head."""
    rec = fx.upstream("ssd_combined", "combined_full"); i = rec["inputs"]; gr = rec["gradients"]
    d = {k: cu(i[k]).clone().requires_grad_(True) for k in ("X", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states")}
    y = ssd().ssd_combined(d["X"], d["dt"], d["A"], d["B"], d["C"], int(i["chunk_size"]), D=d["D"], z=d["z"],
                           dt_bias=d["dt_bias"], initial_states=d["initial_states"], dt_softplus=True)
    y.sum().backward()
    pick = {"X": lambda t: t[:, :, 0], "dt": lambda t: t[:, :, 0], "A": lambda t: t[0], "D": lambda t: t[0],
            "z": lambda t: t[:, :, 0], "dt_bias": lambda t: t[0], "initial_states": lambda t: t[:, 0]}
    for k, f in pick.items():
        torch.testing.assert_close(f(d[k].grad.cpu()), f(gr[k]), rtol=5e-2, atol=5e-2, msg=lambda m: f"{k}: {m}")


@pytest.mark.parametrize("dtype,lens,Q,P,N,softplus", [(torch.float32, [40, 24, 64], 32, 16, 8, True),
                                                     (torch.float32, [5, 70, 1, 20], 16, 8, 4, False),
                                                     (torch.bfloat16, [100, 28, 128], 64, 64, 64, True),
                                                     (torch.bfloat16, [100, 30, 70], 64, 128, 32, False)])
def test_gradients_through_per_sequence_end_states_match_the_oracle(dtype, lens, Q, P, N, softplus):
    """A loss on y, the final state and the per-sequence end states together: every gradient against float64
    autograd through the oracle (the end states add their own terms to x, dt, A, B, the bias and the initial
    state).  Some raw steps fall outside the clamp, where the gradient of the step is zero."""
    g = torch.Generator().manual_seed(77)
    H, G = 4, 2
    L = sum(lens)
    mk = lambda *shape: torch.randn(*shape, generator=g)
    base = dict(x=mk(1, L, H, P).to(dtype), dt=torch.rand(1, L, H, generator=g) * 0.6 - (0.3 if softplus else 0.0),
                A=-torch.rand(H, generator=g) * 1.5 - 0.1, B=(mk(1, L, G, N) * 0.5).to(dtype),
                C=(mk(1, L, G, N) * 0.5).to(dtype), D=mk(H), z=mk(1, L, H, P).to(dtype), bias=mk(H) * 0.2,
                init=mk(1, H, P, N))
    limit = (0.3, 0.9) if softplus else (0.05, 0.5)
    cu_l = [0]
    for n in lens:
        cu_l.append(cu_l[-1] + n)
    seq_idx = torch.cat([torch.full((n,), k, dtype=torch.int32) for k, n in enumerate(lens)])[None]
    wy, wf, wv = mk(1, L, H, P), mk(1, H, P, N), mk(len(lens), H, P, N)

    d = {k: cu(v).clone().requires_grad_(True) for k, v in base.items()}
    y, fin, vs = ssd().ssd_combined(d["x"], d["dt"], d["A"], d["B"], d["C"], Q, D=d["D"], z=d["z"], dt_bias=d["bias"],
                                    initial_states=d["init"], dt_softplus=softplus, dt_limit=limit,
                                    return_final_states=True, seq_idx=cu(seq_idx),
                                    cu_seqlens=torch.tensor(cu_l, dtype=torch.int32).cuda(),
                                    return_varlen_states=True, states_dtype=torch.float32)
    ((y.float() * cu(wy)).sum() + (fin * cu(wf)).sum() + (vs * cu(wv)).sum()).backward()

    r = {k: v.detach().double().requires_grad_(True) for k, v in base.items()}
    oy, of, ov = S.ssd_combined(r["x"], r["dt"], r["A"], r["B"], r["C"], Q, D=r["D"], z=r["z"], dt_bias=r["bias"],
                                initial_states=r["init"], dt_softplus=softplus, dt_limit=limit, seq_idx=seq_idx,
                                cu_seqlens=cu_l)
    torch.testing.assert_close(vs.cpu().double(), ov.detach(), rtol=2e-2 if dtype != torch.float32 else 1e-4,
                               atol=(2e-2 if dtype != torch.float32 else 1e-5) * float(ov.detach().abs().max()))
    ((oy * wy).sum() + (of * wf).sum() + (ov * wv).sum()).backward()
    for k in base:
        got, want = d[k].grad.cpu().double(), r[k].grad
        assert got.shape == want.shape and d[k].grad.dtype == base[k].dtype, k
        scale = float(want.pow(2).mean().sqrt())
        if dtype == torch.float32:
            torch.testing.assert_close(got, want, rtol=1e-3, atol=2e-4 * scale, msg=lambda m: f"{k}: {m}")
        else:
            err = (got - want).abs()
            assert float(err.max()) <= 0.08 * scale + 0.05 * float(want.abs().max()), (k, float(err.max()), scale)
            assert float(err.mean()) <= 0.02 * scale, (k, float(err.mean()), scale)

    # the end states alone: only their own node of the graph runs
    d2 = {k: cu(v).clone().requires_grad_(True) for k, v in base.items()}
    vs2 = ssd().ssd_combined(d2["x"], d2["dt"], d2["A"], d2["B"], d2["C"], Q, D=d2["D"], z=d2["z"], dt_bias=d2["bias"],
                             initial_states=d2["init"], dt_softplus=softplus, dt_limit=limit, seq_idx=cu(seq_idx),
                             cu_seqlens=torch.tensor(cu_l, dtype=torch.int32).cuda(), return_varlen_states=True,
                             states_dtype=torch.float32)[1]
    (vs2 * cu(wv)).sum().backward()
    r2 = {k: v.detach().double().requires_grad_(True) for k, v in base.items()}
    ov2 = S.ssd_combined(r2["x"], r2["dt"], r2["A"], r2["B"], r2["C"], Q, D=r2["D"], z=r2["z"], dt_bias=r2["bias"],
                         initial_states=r2["init"], dt_softplus=softplus, dt_limit=limit, seq_idx=seq_idx,
                         cu_seqlens=cu_l)[2]
    (ov2 * wv).sum().backward()
    for k in ("x", "dt", "A", "B", "bias", "init"):
        got, want = d2[k].grad.cpu().double(), r2[k].grad
        scale = float(want.pow(2).mean().sqrt())
        tol = dict(rtol=1e-3, atol=2e-4 * scale) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2 * scale)
        torch.testing.assert_close(got, want, msg=lambda m: f"end states alone, {k}: {m}", **tol)
    assert d2["C"].grad is None or float(d2["C"].grad.abs().max()) == 0.0


def test_gradients_through_end_states_need_matching_boundaries():
    x = torch.zeros(1, 8, 2, 4).cuda().requires_grad_(True)
    dt = torch.zeros(1, 8, 2).cuda()
    A = -torch.ones(2).cuda()
    Bm = torch.zeros(1, 8, 1, 4).cuda()
    seq_idx = torch.tensor([[0, 0, 0, 1, 1, 1, 1, 1]], dtype=torch.int32).cuda()
    with pytest.raises(ValueError):
        ssd().ssd_combined(x, dt, A, Bm, Bm, 4, seq_idx=seq_idx,
                           cu_seqlens=torch.tensor([0, 4, 8], dtype=torch.int32).cuda(), return_varlen_states=True)


@pytest.mark.parametrize("dtype,lens,Q,P,N", [(torch.float32, [40, 24, 64], 32, 16, 8),
                                            (torch.float32, [64, 64], 64, 8, 4),
                                            (torch.bfloat16, [100, 28, 128], 64, 64, 64)])
def test_gradients_of_packed_sequences_equal_those_of_the_sequences_alone(dtype, lens, Q, P, N):
    """A packed row with seq_idx gives every input the gradient it gets when each sequence runs alone (the
    first one with the initial state): per-step gradients side by side, parameter gradients added up."""
    g = torch.Generator().manual_seed(41)
    H, G = 4, 2
    L = sum(lens)
    mk = lambda *shape: torch.randn(*shape, generator=g)
    base = dict(x=mk(1, L, H, P).to(dtype), dt=torch.rand(1, L, H, generator=g) * 0.5 + 0.05,
                A=-torch.rand(H, generator=g) * 2 - 0.1, B=mk(1, L, G, N).to(dtype), C=mk(1, L, G, N).to(dtype),
                D=mk(H), z=mk(1, L, H, P).to(dtype), init=mk(1, H, P, N))
    wy = mk(1, L, H, P)
    cu_l = [0]
    for n in lens:
        cu_l.append(cu_l[-1] + n)
    seq_idx = torch.cat([torch.full((n,), k, dtype=torch.int32) for k, n in enumerate(lens)])[None].cuda()

    def leaves(sl=None, with_init=True):
        out = {}
        for k, v in base.items():
            t = v if (sl is None or k in ("A", "D", "init")) else v[:, sl]
            out[k] = t.clone().cuda().requires_grad_(True)
        if not with_init:
            out["init"] = None
        return out

    p = leaves()
    y = ssd().ssd_combined(p["x"], p["dt"], p["A"], p["B"], p["C"], Q, D=p["D"], z=p["z"], initial_states=p["init"],
                           seq_idx=seq_idx)
    (y.float() * wy.cuda()).sum().backward()
    acc = {k: torch.zeros_like(v, dtype=torch.float32) for k, v in base.items()}
    for k_seq in range(len(lens)):
        sl = slice(cu_l[k_seq], cu_l[k_seq + 1])
        q = leaves(sl, with_init=(k_seq == 0))
        yk = ssd().ssd_combined(q["x"], q["dt"], q["A"], q["B"], q["C"], Q, D=q["D"], z=q["z"],
                                initial_states=q["init"])
        (yk.float() * wy[:, sl].cuda()).sum().backward()
        for k in base:
            if q[k] is None or q[k].grad is None:
                continue
            gk = q[k].grad.float().cpu()
            if k in ("A", "D", "init"):
                acc[k] += gk
            else:
                acc[k][:, sl] = gk
    for k in base:
        got, want = p[k].grad.float().cpu(), acc[k]
        if dtype == torch.float32:
            scale = float(want.abs().max()) + 1e-6
            torch.testing.assert_close(got, want, rtol=1e-3, atol=1e-4 * scale, msg=lambda m, k=k: f"gradient of {k}: {m}")
        else:
            half_close(got, want, f"gradient of {k}", atol_rms=GRAD_ATOL_RMS, mean_rms=GRAD_MEAN_RMS, rtol=5e-2)


def test_combined_varlen_vector():
    """Packed row of two sequences (cu_seqlens 0, 3, 6; chunk 3), no seq_idx: y of the plain
    scan, per-sequence end states that do not mix.  Negative raw steps are clamped to 0."""
    rec = fx.upstream("ssd_combined", "combined_varlen"); i = rec["inputs"]
    cu_seqlens = torch.tensor([0, 3, 6], dtype=torch.int32).cuda()
    y, vs = ssd().ssd_combined(cu(i["X"]), cu(i["dt"]), cu(i["A"]), cu(i["B"]), cu(i["C"]), int(i["chunk_size"]),
                               cu_seqlens=cu_seqlens, return_varlen_states=True)
    torch.testing.assert_close(y.cpu(), rec["outputs"]["y"], **TF32)
    torch.testing.assert_close(vs.cpu(), rec["outputs"]["varlen_states"], **TF32)


@pytest.mark.parametrize("Q,lens,dtype,P", [(4, [5, 9, 1, 6], torch.float32, 16), (8, [3, 3, 10], torch.float32, 16),
                                            (64, [100, 28, 200, 56], torch.float32, 16),
                                            (64, [100, 28, 200, 56], torch.bfloat16, 16),
                                            (64, [100, 28, 200, 56], torch.bfloat16, 64),
                                            (128, [300, 1, 83, 128], torch.bfloat16, 32)])
def test_packed_sequences_match_the_oracle_and_separate_runs(Q, lens, dtype, P):
    """seq_idx + cu_seqlens: against the float64 oracle, and sequence by sequence against
    separate calls of the same kernels (the first sequence takes the initial state).  The cases
    with 32 or 64 channels per head run the matrix-core kernels."""
    g = torch.Generator().manual_seed(13)
    H, G, N = 4, 2, 32
    L = sum(lens)
    x = torch.randn(1, L, H, P, generator=g).to(dtype)
    dt = torch.rand(1, L, H, generator=g) * 0.5
    A = -torch.rand(H, generator=g) * 2
    Bm = torch.randn(1, L, G, N, generator=g).to(dtype)
    Cm = torch.randn(1, L, G, N, generator=g).to(dtype)
    D = torch.randn(H, generator=g)
    z = torch.randn(1, L, H, P, generator=g).to(dtype)
    init = torch.randn(1, H, P, N, generator=g)
    cu_l = [0]
    for n in lens:
        cu_l.append(cu_l[-1] + n)
    seq_idx = torch.cat([torch.full((n,), k, dtype=torch.int32) for k, n in enumerate(lens)])[None]
    call = lambda: ssd().ssd_combined(cu(x), cu(dt), cu(A), cu(Bm), cu(Cm), Q, D=cu(D), z=cu(z), initial_states=cu(init),
                                      return_final_states=True, seq_idx=cu(seq_idx),
                                      cu_seqlens=torch.tensor(cu_l, dtype=torch.int32).cuda(),
                                      return_varlen_states=True, states_dtype=torch.float32)
    y, fin, vs = call()
    used = kernels_taken(call)
    assert (used & 6) == (6 if (dtype == torch.bfloat16 and P in (32, 64)) else 0)
    wy, wf, wv = S.ssd_combined(x, dt, A, Bm, Cm, Q, D=D, z=z, initial_states=init, clamp_decay=False,
                                seq_idx=seq_idx, cu_seqlens=cu_l)
    if dtype == torch.float32:
        torch.testing.assert_close(y.float().cpu(), wy.float(), **FP32_TOL)
        torch.testing.assert_close(vs.cpu(), wv.float(), **FP32_TOL)
        torch.testing.assert_close(fin.cpu(), wf.float(), **FP32_TOL)
    else:
        half_close(y, wy, "y")
        half_close(vs, wv, "per-sequence end states")
        half_close(fin, wf, "final states")
    for k in range(len(lens)):
        sl = slice(cu_l[k], cu_l[k + 1])
        yk, fk = ssd().ssd_combined(cu(x[:, sl]), cu(dt[:, sl]), cu(A), cu(Bm[:, sl]), cu(Cm[:, sl]), Q, D=cu(D),
                                    z=cu(z[:, sl]), initial_states=cu(init) if k == 0 else None,
                                    return_final_states=True, states_dtype=torch.float32, fused=False)
        if dtype == torch.float32:
            torch.testing.assert_close(y[:, sl].float().cpu(), yk.float().cpu(), **FP32_TOL)
            torch.testing.assert_close(vs[k].cpu(), fk[0].cpu(), **FP32_TOL)
        else:
            half_close(y[:, sl], yk.float(), f"y of sequence {k} run alone")
            half_close(vs[k], fk[0], f"end state of sequence {k} run alone")


@pytest.mark.parametrize("Q,lens,N", [(64, [100, 28, 64, 64], 64), (128, [300, 1, 83, 128], 128), (64, [64, 64, 64, 64], 64),
                                      (64, [1] * 64 + [3] * 21 + [1, 64], 64), (256, [1] * 256 + [200, 56], 128)])
def test_packed_sequences_on_the_one_pass_kernel(Q, lens, N):
    """seq_idx alone (no per-sequence end states asked for) stays on the one-pass kernel, which separates the
    sequences by an extra decay of 2^-64 at every first step: against the float64 oracle, and against the
    five-kernel path with its explicit masks."""
    g = torch.Generator().manual_seed(29)
    H, G, P = 4, 2, 64
    L = sum(lens)
    bf = torch.bfloat16
    x = torch.randn(2, L, H, P, generator=g).to(bf)
    dt = torch.rand(2, L, H, generator=g) * 0.5
    A = -torch.rand(H, generator=g) * 2
    Bm = torch.randn(2, L, G, N, generator=g).to(bf)
    Cm = torch.randn(2, L, G, N, generator=g).to(bf)
    D = torch.randn(H, generator=g)
    z = torch.randn(2, L, H, P, generator=g).to(bf)
    init = torch.randn(2, H, P, N, generator=g)
    row = torch.cat([torch.full((n,), k, dtype=torch.int32) for k, n in enumerate(lens)])
    seq_idx = torch.stack([row, torch.zeros_like(row)])          # second batch row: one sequence
    call = lambda: ssd().ssd_combined(cu(x), cu(dt), cu(A), cu(Bm), cu(Cm), Q, D=cu(D), z=cu(z), initial_states=cu(init),
                                      return_final_states=True, seq_idx=cu(seq_idx))
    y, fin = call()
    assert kernels_taken(call) & 8
    y5, fin5 = ssd().ssd_combined(cu(x), cu(dt), cu(A), cu(Bm), cu(Cm), Q, D=cu(D), z=cu(z), initial_states=cu(init),
                                  return_final_states=True, seq_idx=cu(seq_idx), fused=False, states_dtype=torch.float32)
    wy, wf = S.ssd_combined(x, dt, A, Bm, Cm, Q, D=D, z=z, initial_states=init, clamp_decay=False, seq_idx=seq_idx)[:2]
    half_close(y, wy, "y, one pass")
    half_close(fin, wf, "final states, one pass")
    half_close(y, y5.float(), "y, one pass against five kernels")
    half_close(fin, fin5, "final states, one pass against five kernels")


def test_packed_arguments_are_checked():
    x = torch.zeros(2, 8, 2, 4).cuda()
    dt = torch.zeros(2, 8, 2).cuda()
    A = -torch.ones(2).cuda()
    Bm = torch.zeros(2, 8, 1, 4).cuda()
    with pytest.raises(ValueError):
        ssd().ssd_combined(x, dt, A, Bm, Bm, 4, return_varlen_states=True)                       # no cu_seqlens
    with pytest.raises(ValueError):
        ssd().ssd_combined(x, dt, A, Bm, Bm, 4, cu_seqlens=torch.tensor([0, 8]).cuda(), return_varlen_states=True)
    with pytest.raises(ValueError):
        ssd().ssd_combined(x, dt, A, Bm, Bm, 4, seq_idx=torch.zeros(2, 7, dtype=torch.int32).cuda())


@pytest.mark.parametrize("shape,Q", [((1, 1, 1, 1, 1, 1), 1), ((2, 19, 4, 5, 2, 6), 8), ((2, 64, 4, 16, 1, 32), 16),
                                     ((1, 300, 2, 64, 2, 128), 64), ((2, 130, 3, 7, 3, 9), 256),
                                     ((1, 250, 2, 100, 1, 70), 96), ((1, 200, 1, 130, 1, 33), 200)],
                         ids=lambda v: str(v).replace(" ", ""))
def test_fp32_combined_matches_float64_recurrence(shape, Q):
    b, l, h, p, g, n = shape
    inp = make(sum(shape), b, l, h, p, g, n, d_mat=(l % 2 == 1))
    y64, f64 = S.ssd_sequential(inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                                initial_states=inp["init"])
    y, fin = ssd().ssd_combined(cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q,
                                D=cu(inp["D"]), z=cu(inp["z"]), initial_states=cu(inp["init"]),
                                return_final_states=True)
    torch.testing.assert_close(y.cpu().double(), y64, **FP32_TOL)
    torch.testing.assert_close(fin.cpu().double(), f64, **FP32_TOL)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_tiled_kernels_match_the_one_thread_per_output_kernels(dtype):
    """Float32 / float16 calls run 64x64 tiles on the float32 matrix cores; ``force_generic`` keeps the
    plain kernels (one thread per output element) as a second opinion: tiles with remainders in every
    dimension, a ragged last chunk and packed sequences."""
    b, l, h, p, g, n, Q = 2, 333, 4, 72, 2, 80, 160
    inp = make(17, b, l, h, p, g, n, d_mat=True)
    seq_idx = torch.zeros(b, l, dtype=torch.int32)
    seq_idx[:, 120:] = 1
    seq_idx[:, 170:] = 2
    args = [cu(inp[k]).to(dtype) if k in ("x", "B", "C") else cu(inp[k]) for k in ("x", "dt", "A", "B", "C")]
    kw = dict(D=cu(inp["D"]), z=cu(inp["z"]).to(dtype), seq_idx=seq_idx.cuda(), return_final_states=True)
    y, fin = ssd().ssd_combined(*args, Q, **kw)
    yg, fing = ssd().ssd_combined(*args, Q, force_generic=True, **kw)
    tol = FP32_TOL if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(y.float(), yg.float(), **tol)
    torch.testing.assert_close(fin, fing, **tol)


def test_components_match_oracle_fp32():
    inp = make(3, 2, 96, 4, 8, 2, 16)
    Q = 32
    dA, dtc = ssd().chunk_cumsum(cu(inp["dt"]), cu(inp["A"]), Q)
    dA_o, dtc_o = S.chunk_cumsum(inp["dt"], inp["A"], Q)
    torch.testing.assert_close(dA.cpu().double(), dA_o, rtol=1e-5, atol=1e-5)
    st = ssd().chunk_state(cu(inp["B"]), cu(inp["x"]), dtc, dA)
    st_o = S.chunk_state(inp["B"], inp["x"], dtc_o, dA_o)
    torch.testing.assert_close(st.cpu().double(), st_o, **FP32_TOL)
    ent, fin = ssd().state_passing(st, dA[..., -1].contiguous(), initial_states=cu(inp["init"]))
    ent_o, fin_o = S.state_passing(st_o, dA_o[..., -1], inp["init"])
    torch.testing.assert_close(ent.cpu().double(), ent_o, **FP32_TOL)
    torch.testing.assert_close(fin.cpu().double(), fin_o, **FP32_TOL)
    CB = ssd().bmm_chunk(cu(inp["C"]), cu(inp["B"]), Q)
    torch.testing.assert_close(CB.cpu().double(), S.bmm_chunk(inp["C"], inp["B"], Q), **FP32_TOL)
    y = ssd().chunk_scan(cu(inp["B"]), cu(inp["C"]), cu(inp["x"]), dtc, dA, ent, D=cu(inp["D"]), z=cu(inp["z"]))
    y_o = S.chunk_scan(inp["B"], inp["C"], inp["x"], dtc_o, dA_o, ent_o, D=inp["D"], z=inp["z"])
    torch.testing.assert_close(y.cpu().double(), y_o, **FP32_TOL)


@pytest.mark.parametrize("shape,Q", [((2, 512, 4, 64, 1, 128), 256), ((1, 256, 2, 64, 2, 64), 64),
                                     ((2, 384, 8, 32, 1, 128), 128), ((1, 700, 2, 64, 1, 128), 256)],
                         ids=lambda v: str(v).replace(" ", ""))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=lambda v: str(v).replace("torch.", ""))
def test_bf16_mfma_matches_generic_and_oracle(shape, Q, dtype):
    """The five matrix-core kernels, for both 16-bit element types (v_mfma_f32_32x32x16_bf16 / _f16)."""
    b, l, h, p, g, n = shape
    inp = make(11, b, l, h, p, g, n, dtype=dtype)
    args = (cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q)
    kw = dict(D=cu(inp["D"]), z=cu(inp["z"]), initial_states=cu(inp["init"]), return_final_states=True)
    y, fin = ssd().ssd_combined(*args, fused=False, **kw)
    used = kernels_taken(lambda: ssd().ssd_combined(*args, fused=False, **kw))
    assert used == 7, f"MFMA kernels used: {used:03b}"      # a ragged end is filled up to whole chunks
    generic = lambda: ssd().ssd_combined(*args, force_generic=True, states_dtype=torch.float32, **kw)
    yg, fing = generic()                                    # the selector routes this call to the test-hooks build
    assert kernels_taken(generic) == 0
    y64, f64 = S.ssd_sequential(inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                                initial_states=inp["init"])
    half_close(yg, y64, "y, plain kernels")
    # states between these kernels are kept in bf16 by default: one more rounding of every carried state
    half_close(y, y64, "y, matrix-core kernels", atol_rms=8e-2)
    half_close(fin, f64, "final states")


FUSED_CASES = [
    # (B, L, H, P, G, N), Q, d_mat, use_z, use_init
    ((2, 512, 4, 64, 1, 128), 256, False, True, True),
    ((1, 1024, 3, 64, 1, 128), 256, True, True, False),
    ((2, 384, 4, 64, 2, 64), 128, False, False, True),
    ((1, 256, 2, 64, 2, 64), 64, True, True, True),
    ((3, 192, 2, 64, 1, 64), 64, False, True, False),
    ((1, 256, 1, 64, 1, 128), 256, False, False, False),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bfloat16", "float16"])
@pytest.mark.parametrize("shape,Q,d_mat,use_z,use_init", FUSED_CASES, ids=lambda v: str(v).replace(" ", ""))
def test_one_pass_matches_oracle_and_five_kernel_path(shape, Q, d_mat, use_z, use_init, dtype):
    """The one-pass kernel in both 16-bit element types (it is compiled per type: v_mfma_f32_32x32x16_bf16 / _f16)."""
    b, l, h, p, g, n = shape
    inp = make(17 + l + Q, b, l, h, p, g, n, dtype=dtype, d_mat=d_mat, use_z=use_z, use_init=use_init)
    args = (cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q)
    kw = dict(D=cu(inp["D"]), z=cu(inp["z"]), initial_states=cu(inp["init"]), return_final_states=True)
    y, fin = ssd().ssd_combined(*args, fused=True, **kw)
    assert kernels_taken(lambda: ssd().ssd_combined(*args, fused=True, **kw)) == 8
    y5, fin5 = ssd().ssd_combined(*args, fused=False, **kw)
    y64, f64 = S.ssd_sequential(inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                                initial_states=inp["init"])
    half_close(y, y64, "y, one pass")
    half_close(fin, f64, "final states, one pass")
    assert y.dtype == dtype
    # the two GPU paths round at different places; they agree to the resolution of the element type
    half_close(y, y5.float(), "y, one pass against five kernels")
    half_close(fin, fin5, "final states, one pass against five kernels")


@pytest.mark.parametrize("d_mat", [False, True], ids=["per-head", "per-channel"])
def test_one_pass_takes_parameters_that_are_views_into_larger_buffers(d_mat):
    """``A``, ``D`` and the bias of a few heads cut out of a model's parameter vectors start at any 4-byte offset."""
    b, l, h, p, g, n, Q = 1, 256, 3, 64, 1, 64, 128
    inp = make(41, b, l, h, p, g, n, dtype=torch.bfloat16, d_mat=d_mat, use_z=True, use_init=False)

    def view(t):                      # the same values one float32 into a larger buffer: not 16-byte aligned
        buf = torch.zeros(t.numel() + 1, device="cuda")
        buf[1:] = cu(t).reshape(-1)
        v = buf[1:].view(t.shape)
        assert v.data_ptr() % 16 == 4
        return v

    args = (cu(inp["x"]), cu(inp["dt"]), view(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q)
    y = ssd().ssd_combined(*args, D=view(inp["D"]), z=cu(inp["z"]), fused=True)
    want = ssd().ssd_combined(cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q, D=cu(inp["D"]),
                              z=cu(inp["z"]), fused=True)
    assert torch.equal(y, want)


def test_one_pass_dt_bias_softplus_and_clamp():
    b, l, h, p, g, n, Q = 2, 256, 4, 64, 1, 64, 128
    inp = make(5, b, l, h, p, g, n, dtype=torch.bfloat16, use_init=False)
    gen = torch.Generator().manual_seed(1)
    raw = torch.randn(b, l, h, generator=gen)
    bias = torch.randn(h, generator=gen) - 2.0
    kw = dict(D=cu(inp["D"]), z=cu(inp["z"]), dt_bias=cu(bias), dt_softplus=True, dt_limit=(0.01, 0.5),
              return_final_states=True)
    y, fin = ssd().ssd_combined(cu(inp["x"]), cu(raw), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q, fused=True, **kw)
    dt_eff = torch.nn.functional.softplus(raw + bias).clamp(0.01, 0.5)
    y64, f64 = S.ssd_sequential(inp["x"], dt_eff, inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"])
    half_close(y, y64, "y")
    half_close(fin, f64, "final states")


@pytest.mark.parametrize("shape,Q,d_mat", [((2, 512, 3, 128, 1, 128), 256, False), ((1, 256, 2, 192, 2, 64), 64, True)],
                         ids=lambda v: str(v).replace(" ", ""))
def test_wide_heads_run_as_heads_of_64_channels(shape, Q, d_mat):
    """headdim 128 / 192 in bf16: the same result as the float64 recurrence, through the one-pass
    kernel (a head of 64k channels is k heads of 64); packed sequences through the five kernels."""
    b, l, h, p, g, n = shape
    inp = make(5 + p, b, l, h, p, g, n, dtype=torch.bfloat16, d_mat=d_mat, use_z=True, use_init=True)
    call = lambda: ssd().ssd_combined(cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q,
                                      D=cu(inp["D"]), z=cu(inp["z"]), initial_states=cu(inp["init"]),
                                      return_final_states=True)
    y, fin = call()
    assert kernels_taken(call) == 8
    y64, f64 = S.ssd_sequential(inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                                initial_states=inp["init"])
    assert tuple(y.shape) == (b, l, h, p) and tuple(fin.shape) == (b, h, p, n)
    half_close(y, y64, "y")
    half_close(fin, f64, "final states")
    seq_idx = torch.zeros(b, l, dtype=torch.int32)
    seq_idx[:, l // 3:] = 1
    yp = ssd().ssd_combined(cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q, D=cu(inp["D"]),
                            z=cu(inp["z"]), initial_states=cu(inp["init"]), seq_idx=cu(seq_idx))
    wy = S.ssd_combined(inp["x"], inp["dt"], inp["A"], inp["B"], inp["C"], Q, D=inp["D"], z=inp["z"],
                        initial_states=inp["init"], clamp_decay=False, seq_idx=seq_idx)
    wy = wy[0] if isinstance(wy, tuple) else wy
    half_close(yp, wy, "y, packed")


@pytest.mark.parametrize("shape,Q,softplus", [((2, 1000, 4, 64, 1, 128), 256, False), ((1, 777, 3, 64, 1, 64), 128, True)],
                         ids=lambda v: str(v).replace(" ", ""))
def test_ragged_length_is_filled_up_with_steps_of_size_zero(shape, Q, softplus):
    """bf16 and a length that is not a whole number of chunks: the call pads with steps of size zero and
    still runs the matrix-core kernels; y, the final state and the gradients match the float64 recurrence."""
    b, l, h, p, g, n = shape
    inp = make(3, b, l, h, p, g, n, dtype=torch.bfloat16, use_init=True)
    gen = torch.Generator().manual_seed(l)
    dt = torch.randn(b, l, h, generator=gen) if softplus else inp["dt"]
    bias = torch.randn(h, generator=gen) * 0.3 if softplus else None
    xg = cu(inp["x"]).requires_grad_(True)
    call = lambda: ssd().ssd_combined(xg, cu(dt), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), Q, D=cu(inp["D"]),
                                      z=cu(inp["z"]), initial_states=cu(inp["init"]),
                                      dt_bias=None if bias is None else cu(bias), dt_softplus=softplus,
                                      return_final_states=True)
    y, fin = call()
    assert kernels_taken(call) != 0 and tuple(y.shape) == (b, l, h, p)
    x64 = inp["x"].double().requires_grad_(True)
    y64, f64 = S.ssd_sequential(x64, dt, inp["A"], inp["B"], inp["C"], D=inp["D"], z=inp["z"],
                                initial_states=inp["init"], dt_bias=bias, dt_softplus=softplus)
    half_close(y, y64, "y")
    half_close(fin, f64, "final states")
    go = torch.randn(b, l, h, p, generator=gen)
    (y.float() * go.cuda()).sum().backward()
    (y64 * go.double()).sum().backward()
    half_close(xg.grad, x64.grad, "gradient of x", atol_rms=GRAD_ATOL_RMS, mean_rms=GRAD_MEAN_RMS, rtol=3e-2)


def test_one_pass_rejects_uncovered_calls():
    inp = make(1, 1, 64, 2, 32, 1, 64, dtype=torch.bfloat16, use_init=False)
    with pytest.raises(ValueError):
        ssd().ssd_combined(cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), 32, fused=True)


def test_config3_shape_bf16():
    """BASELINE config 3: B=4, L=4096, H=80, P=64, N=128, G=1, Q=256, bf16.  Full size on the
    GPU; two heads of one batch row are replayed by the float64 sequential recurrence."""
    inp = make(3, 4, 4096, 80, 64, 1, 128, dtype=torch.bfloat16, use_init=False)
    g3 = {k: cu(v) for k, v in inp.items()}
    call = lambda: ssd().ssd_combined(g3["x"], g3["dt"], g3["A"], g3["B"], g3["C"], 256, D=g3["D"], z=g3["z"],
                                      return_final_states=True)
    y, fin = call()
    assert kernels_taken(call) == 8
    assert y.dtype == torch.bfloat16 and fin.dtype == torch.float32 and tuple(fin.shape) == (4, 80, 64, 128)
    hs = [5, 71]
    y64, f64 = S.ssd_sequential(inp["x"][1:2, :, hs], inp["dt"][1:2, :, hs], inp["A"][hs], inp["B"][1:2],
                                inp["C"][1:2], D=inp["D"][hs], z=inp["z"][1:2, :, hs])
    half_close(y[1:2, :, hs], y64, "y against the float64 recurrence")
    half_close(fin[1:2, hs], f64, "final states against the float64 recurrence")
    # every (batch, head) pair, under the load of the whole grid: the one-pass kernel against the five
    # matrix-core kernels, which share no code with it beyond the operand packing
    y5, fin5 = ssd().ssd_combined(cu(inp["x"]), cu(inp["dt"]), cu(inp["A"]), cu(inp["B"]), cu(inp["C"]), 256,
                                  D=cu(inp["D"]), z=cu(inp["z"]), return_final_states=True, fused=False)
    y5f = y5.float()
    diff = (y.float() - y5f).abs()
    rms = float(y5f.pow(2).mean().sqrt())
    excess = (diff - 2e-2 * y5f.abs()).amax(dim=(1, 3)) / rms    # (B, H): worst element of each pair beyond 2 % of itself
    assert float(excess.max()) < 8e-2, f"worst (batch, head) pair: {excess.max():.3e} of the rms at {excess.argmax()}"
    assert float(diff.mean()) < 3e-3 * rms
    half_close(fin, fin5, "final states, one pass against five kernels, all heads")


def test_ragged_length_with_16_bit_steps_and_a_bias_keeps_the_final_state():
    """bf16 raw steps, a bias, no softplus, a ragged length: the padded steps must have size exactly zero, or the
    final state decays over the padding (A is large here so that even a step of 1e-3 would show)."""
    b, l, h, p, g, n, Q = 1, 300, 2, 64, 1, 64, 256
    inp = make(21, b, l, h, p, g, n, dtype=torch.bfloat16, use_init=True)
    gen = torch.Generator().manual_seed(2)
    bias = torch.rand(h, generator=gen) * 0.5 + 0.1234567
    raw = (inp["dt"].float() * 0.2).to(torch.bfloat16)
    A = -torch.full((h,), 40.0)
    y, fin = ssd().ssd_combined(cu(inp["x"]), cu(raw), cu(A), cu(inp["B"]), cu(inp["C"]), Q, dt_bias=cu(bias),
                                initial_states=cu(inp["init"]), dt_softplus=False, return_final_states=True)
    y64, f64 = S.ssd_sequential(inp["x"], raw, A, inp["B"], inp["C"], dt_bias=bias, dt_softplus=False,
                                initial_states=inp["init"])
    half_close(y, y64, "y")
    half_close(fin, f64, "final states")


def test_growing_states_on_the_one_pass_kernel():
    """Positive A on some heads: the one-pass kernel looks at the sign of a head's A itself and follows the
    upstream kernels there (decays inside a chunk clamped to 1, the carried state growing freely), packed or
    not, so the default path picks it whatever the values of A are and agrees with the five kernels and with
    the oracle's restatement of the clamps."""
    b, l, h, p, g, n, Q = 2, 512, 4, 64, 1, 64, 128
    inp = make(31, b, l, h, p, g, n, dtype=torch.bfloat16, use_init=True)
    A = torch.tensor([0.25, -0.5, 0.04, -3.0])
    dt = torch.rand(b, l, h, generator=torch.Generator().manual_seed(4)) * 0.05 + 0.005
    seq_idx = torch.zeros(b, l, dtype=torch.int32)
    seq_idx[:, 200:] = 1
    seq_idx[:, 333:] = 2
    for sid in (None, seq_idx):
        call = lambda **kw: ssd().ssd_combined(cu(inp["x"]), cu(dt), cu(A), cu(inp["B"]), cu(inp["C"]), Q, D=cu(inp["D"]),
                                               z=cu(inp["z"]), initial_states=cu(inp["init"]), return_final_states=True,
                                               seq_idx=cu(sid), **kw)
        y, fin = call()
        assert kernels_taken(call) == 8
        y5, fin5 = call(fused=False, states_dtype=torch.float32)
        wy, wf = S.ssd_combined(inp["x"], dt, A, inp["B"], inp["C"], Q, D=inp["D"], z=inp["z"], initial_states=inp["init"],
                                clamp_decay=True, seq_idx=sid)[:2]
        for hh in range(h):                # head by head: a growing head is orders of magnitude larger than a decaying one
            half_close(y[:, :, hh], wy[:, :, hh], f"y, head {hh}")
            half_close(fin[:, hh], wf[:, hh], f"final states, head {hh}")
            half_close(y5[:, :, hh], wy[:, :, hh], f"y, five kernels, head {hh}")
            half_close(fin5[:, hh], wf[:, hh], f"final states, five kernels, head {hh}")


def test_one_pass_choice_never_reads_A_on_the_host():
    """``ssd_combined`` under stream capture with ``A`` written anew before every replay, growing on one head:
    the captured call is the eager call (no host read of ``A`` decides anything), and every replay agrees with
    the oracle for the values of ``A`` it was replayed with."""
    b, l, h, p, g, n, Q = 1, 256, 3, 64, 1, 128, 64
    inp = make(77, b, l, h, p, g, n, dtype=torch.bfloat16, use_init=False)
    dev = {k: cu(v) for k, v in inp.items()}
    dt = (torch.rand(b, l, h, generator=torch.Generator().manual_seed(5)) * 0.05 + 0.005)
    dt_g = cu(dt)
    A_log = torch.zeros(h, device="cuda")
    sign = torch.tensor([-1.0, 1.0, -1.0], device="cuda")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run = lambda: ssd().ssd_combined(dev["x"], dt_g, sign * torch.exp(A_log), dev["B"], dev["C"], Q, D=dev["D"],
                                         z=dev["z"], return_final_states=True)
        run()                                              # warm-up outside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            y_g, fin_g = run()
    torch.cuda.current_stream().wait_stream(side)
    for k, values in enumerate(([0.0, -1.5, 1.0], [-2.0, -3.0, 0.5], [1.0, -0.7, -4.0])):
        A_log.copy_(torch.tensor(values))
        graph.replay()
        torch.cuda.synchronize()
        A = (sign * torch.exp(A_log)).cpu()
        y_e, fin_e = ssd().ssd_combined(dev["x"], dt_g, cu(A), dev["B"], dev["C"], Q, D=dev["D"], z=dev["z"],
                                        return_final_states=True)
        assert torch.equal(y_g, y_e) and torch.equal(fin_g, fin_e), f"replay {k} differs from the eager call"
        wy, wf = S.ssd_combined(inp["x"], dt, A, inp["B"], inp["C"], Q, D=inp["D"], z=inp["z"], clamp_decay=True)[:2]
        for hh in range(h):
            half_close(y_g[:, :, hh], wy[:, :, hh], f"y, replay {k}, head {hh}")
            half_close(fin_g[:, hh], wf[:, hh], f"final states, replay {k}, head {hh}")


# ------------------------------------------------------------------ backward: the head-summed matrix of a chunk

@pytest.mark.parametrize("b,l,h,p,g,Q", [(2, 256, 4, 64, 1, 64), (1, 512, 6, 32, 2, 256), (1, 96, 3, 64, 3, 32)],
                         ids=lambda v: str(v))
def test_bwd_dcb_kernel_matches_the_sum_over_heads_in_float64(b, l, h, p, g, Q):
    """``ssm_ssd_bwd_dcb`` against ``sum_h dt_s exp(cs_l - cs_s) <dy_l, x_s>`` (lower triangle) formed in float64
    from the same bf16 operands."""
    from ssm_amd.ops import ssd as ops_ssd
    gen = torch.Generator().manual_seed(5 + l)
    dy = torch.randn(b, l, h, p, generator=gen).to(torch.bfloat16)
    x = torch.randn(b, l, h, p, generator=gen).to(torch.bfloat16)
    dt = torch.nn.functional.softplus(torch.randn(b, l, h, generator=gen) - 2.0)
    A = -(torch.rand(h, generator=gen) * 4 + 0.5)
    dA_cs, dt_c = ops_ssd.chunk_cumsum(dt.cuda(), A.cuda(), Q)
    got = ops_ssd._bwd_dcb(dy.cuda(), x.cuda(), dt_c, dA_cs, g).cpu().double()
    nc, per = l // Q, h // g
    cs = dA_cs.cpu().double()                                    # (B, H, nc, Q)
    dtc = dt_c.cpu().double()
    dyc = dy.double().view(b, nc, Q, g, per, p)
    xc = x.double().view(b, nc, Q, g, per, p)
    m = torch.einsum("bclgrp,bcsgrp->bcgrls", dyc, xc)           # per head
    csh = cs.view(b, g, per, nc, Q).permute(0, 3, 1, 2, 4)       # (B, nc, G, per, Q)
    dth = dtc.view(b, g, per, nc, Q).permute(0, 3, 1, 2, 4)
    w = torch.exp(csh[..., :, None] - csh[..., None, :]) * dth[..., None, :]
    w = w * torch.tril(torch.ones(Q, Q, dtype=torch.float64))
    want = (m * w).sum(3)
    assert got.shape == want.shape
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-5 * float(want.abs().max()))


def test_bwd_states_kernel_casts_reverses_and_anchors():
    from ssm_amd.ops import ssd as ops_ssd
    gen = torch.Generator().manual_seed(9)
    ent_f = torch.randn(2, 5, 3, 8, 12, generator=gen).cuda()
    ent_r = torch.randn(2, 5, 3, 8, 12, generator=gen).cuda()
    f16, r16, anchor = ops_ssd._bwd_states(ent_f, ent_r)
    assert torch.equal(f16, ent_f.to(torch.bfloat16))
    assert torch.equal(r16, ent_r.flip(1).to(torch.bfloat16))
    want = (ent_r.flip(1)[:, :-1].double() * ent_f[:, 1:].double()).sum(dim=(3, 4))
    torch.testing.assert_close(anchor.double(), want, rtol=1e-5, atol=1e-5)
    f1, r1, a1 = ops_ssd._bwd_states(ent_f[:, :1].contiguous(), ent_r[:, :1].contiguous())      # a single chunk
    assert a1.shape == (2, 0, 3) and torch.equal(r1, ent_r[:, :1].to(torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_scale_rows_kernel_rounds_once(dtype):
    from ssm_amd.ops import ssd as ops_ssd
    gen = torch.Generator().manual_seed(2)
    x = torch.randn(3, 37, 5, 12, generator=gen).to(dtype).cuda()
    w = torch.rand(3, 37, 5, generator=gen).cuda()
    got = ops_ssd._scale_rows(x, w, torch.bfloat16)
    assert torch.equal(got, (w[..., None] * x.float()).to(torch.bfloat16))
    assert torch.equal(ops_ssd._scale_rows(x, w, torch.float32), w[..., None] * x.float())


@pytest.mark.parametrize("Q,L,softplus,limit", [(64, 256, True, (0.001, 0.1)), (96, 288, False, (0.0, float("inf"))),
                                                 (256, 256, True, (0.0, float("inf"))), (32, 160, True, (0.01, 1.0))])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bwd_prep_kernel_matches_the_steps_taken_one_by_one(Q, L, softplus, limit, dtype):
    """One launch for what the backward derives from the raw steps: the chunked running sums are those of
    ``chunk_cumsum`` (forward, and over the time-reversed steps that decay by the step after them) to the bit, and the
    two row weights are their exponentials in float64 to a few ulps."""
    import math
    from ssm_amd.ops import ssd as ops_ssd
    gen = torch.Generator().manual_seed(Q + L)
    b, h = 2, 5
    dt = (torch.randn(b, L, h, generator=gen) * (1.0 if softplus else 0.05)).to(dtype).cuda()
    if not softplus:
        dt = dt.abs()
    A = -(torch.rand(h, generator=gen) * 8 + 0.1).cuda()
    bias = torch.randn(h, generator=gen).cuda() * 0.1 if softplus else None
    dA_cs, dt_c, dA_r, dte, w_dy, w_x = ops_ssd._bwd_prep(dt, A, Q, bias, softplus, limit)
    want_cs, want_dt = ops_ssd.chunk_cumsum(dt, A, Q, dt_bias=bias, dt_softplus=softplus, dt_limit=limit)
    assert torch.equal(dA_cs, want_cs) and torch.equal(dt_c, want_dt)
    rows = want_dt.permute(0, 2, 3, 1).reshape(b, L, h)
    assert torch.equal(dte, rows)
    shifted = torch.cat([rows[:, 1:], torch.zeros_like(rows[:, :1])], dim=1).flip(1).contiguous()
    want_r, _ = ops_ssd.chunk_cumsum(shifted, A, Q, dt_limit=(-math.inf, math.inf))
    assert torch.equal(dA_r, want_r)
    by_rows = lambda t: t.permute(0, 2, 3, 1).reshape(b, L, h)
    torch.testing.assert_close(w_dy.double(), torch.exp(by_rows(want_cs).double()), rtol=2e-6, atol=1e-30)
    torch.testing.assert_close(w_x.double(), rows.double() * torch.exp(by_rows(want_r).double()).flip(1), rtol=2e-6, atol=1e-30)


@pytest.mark.parametrize("shape,Q", [((2, 256, 3, 64, 1, 32), 64), ((1, 512, 4, 32, 2, 16), 256), ((2, 192, 2, 128, 1, 64), 96)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v))
def test_operand_scaled_while_staged_equals_the_scaled_tensor(shape, Q, dtype=torch.bfloat16):
    """``x_scale``: the matrix-core ``chunk_state`` and ``chunk_scan`` round ``x * scale`` as they stage ``x`` -- the
    bits of a pass over the tensor ``round(x * scale)`` written beforehand, entering states included."""
    from ssm_amd.ops import ssd as ops_ssd
    b, l, h, p, g, n = shape
    gen = torch.Generator().manual_seed(l + h)
    x = torch.randn(b, l, h, p, generator=gen).to(dtype).cuda()
    Bm = torch.randn(b, l, g, n, generator=gen).to(dtype).cuda()
    Cm = torch.randn(b, l, g, n, generator=gen).to(dtype).cuda()
    dt = (torch.rand(b, l, h, generator=gen) * 0.2).cuda()
    A = -(torch.rand(h, generator=gen) * 4 + 0.1).cuda()
    init = torch.randn(b, h, p, n, generator=gen).cuda()
    dA_cs, dt_c = ops_ssd.chunk_cumsum(dt, A, Q)
    ones = torch.ones_like(dt_c)
    assert ops_ssd._row_scale_ok(x, Bm, Cm, Q)
    scaled = (dt[..., None] * x.float()).to(dtype)
    want = ops_ssd._lin_pass(scaled, ones, dA_cs, Bm, Cm, init, want_entering=True)
    got = ops_ssd._lin_pass(x, ones, dA_cs, Bm, Cm, init, want_entering=True, x_scale=dt_c)
    for a, w, name in zip(got, want, ("y", "final state", "entering states")):
        assert torch.equal(a, w), name
    # a call the matrix-core kernels do not take refuses the scale instead of dropping it
    for other in (torch.float32, torch.float16):
        with pytest.raises(Exception, match="x_row_scale"):
            ops_ssd.chunk_state(Bm.to(other), x.to(other), ones, dA_cs, x_scale=dt_c)
        assert not ops_ssd._row_scale_ok(x.to(other), Bm.to(other), Cm.to(other), Q)


@pytest.mark.parametrize("shape,Q,d_mode,out", [((2, 256, 3, 64, 1, 32), 64, "vec", torch.float32),
                                                 ((1, 512, 4, 32, 2, 16), 256, "mat", torch.bfloat16),
                                                 ((2, 192, 2, 64, 1, 64), 96, "none", torch.bfloat16)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v).replace("torch.", ""))
def test_reversed_pass_finishes_dx_in_its_own_kernel(shape, Q, d_mode, out):
    """``dx_epilogue``: the matrix-core ``chunk_scan`` of the gradient's time-reversed pass writes ``dx`` and the row
    sums ``xu``, ``s1`` instead of its result ``u``; against ``ssm_ssd_bwd_dx`` fed with ``u`` from the same pass
    (equal up to the float32 order of the row sums; the skip term sees ``dy`` after its rounding to bfloat16)."""
    from ssm_amd.ops import ssd as ops_ssd
    b, l, h, p, g, n = shape
    gen = torch.Generator().manual_seed(l + h + p)
    bf = torch.bfloat16
    x = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    dy = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    Bm = torch.randn(b, l, g, n, generator=gen).to(bf).cuda()
    Cm = torch.randn(b, l, g, n, generator=gen).to(bf).cuda()
    dt = (torch.rand(b, l, h, generator=gen) * 0.2).cuda()
    A = -(torch.rand(h, generator=gen) * 4 + 0.1).cuda()
    D = {"none": None, "vec": torch.randn(h, generator=gen).cuda(), "mat": torch.randn(h, p, generator=gen).cuda()}[d_mode]
    dfin = torch.randn(b, h, p, n, generator=gen).cuda()
    dA_cs, dt_c = ops_ssd.chunk_cumsum(dt, A, Q)
    ones = torch.ones_like(dt_c)
    dyr = dy.flip(1).contiguous()
    Cr, Br = Cm.flip(1).contiguous(), Bm.flip(1).contiguous()
    u_r, fin, ent = ops_ssd._lin_pass(dyr, ones, dA_cs, Cr, Br, dfin, want_entering=True)
    want = ops_ssd._bwd_dx(dy, None, x, u_r.contiguous(), dt, D, True, grads_io=(out == bf))
    (dx, xu, s1), fin2, ent2 = ops_ssd._lin_pass(dyr, ones, dA_cs, Cr, Br, dfin, want_entering=True,
                                                  dx_epilogue=(x, dt, D, out, True))
    assert torch.equal(fin, fin2) and torch.equal(ent, ent2)
    assert dx.dtype == out and want[0].dtype == out
    scale = float(want[0].float().abs().max())
    torch.testing.assert_close(dx.float(), want[0].float(), rtol=2.0 ** -7 if out == bf else 1e-6, atol=1e-6 * scale)
    for got, w, name in ((xu, want[1], "xu"), (s1, want[2], "s1")):
        torch.testing.assert_close(got, w, rtol=1e-5, atol=1e-5 * float(w.abs().max()), msg=lambda m_, n_=name: f"{n_}: {m_}")


@pytest.mark.parametrize("shape,Q", [((2, 256, 3, 64, 1, 32), 64), ((1, 512, 4, 32, 2, 16), 256), ((2, 192, 2, 128, 1, 64), 96)],
                         ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v))
def test_reversed_pass_reads_its_operand_in_forward_time(shape, Q):
    """``x_reversed``: a pass over reversed time given ``x`` in forward time equals, to the bit, the pass given the
    reversed copy -- its result, the states, and ``dx`` with its row sums when the kernel finishes those."""
    from ssm_amd.ops import ssd as ops_ssd
    b, l, h, p, g, n = shape
    gen = torch.Generator().manual_seed(l + h + 2)
    bf = torch.bfloat16
    x = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    dy = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    Br = torch.randn(b, l, g, n, generator=gen).to(bf).cuda()
    Cr = torch.randn(b, l, g, n, generator=gen).to(bf).cuda()
    dt = (torch.rand(b, l, h, generator=gen) * 0.2).cuda()
    A = -(torch.rand(h, generator=gen) * 4 + 0.1).cuda()
    D = torch.randn(h, generator=gen).cuda()
    dfin = torch.randn(b, h, p, n, generator=gen).cuda()
    dA_cs, dt_c = ops_ssd.chunk_cumsum(dt, A, Q)
    ones = torch.ones_like(dt_c)
    want = ops_ssd._lin_pass(dy.flip(1).contiguous(), ones, dA_cs, Br, Cr, dfin, want_entering=True)
    got = ops_ssd._lin_pass(dy, ones, dA_cs, Br, Cr, dfin, want_entering=True, x_reversed=True)
    for a, w, name in zip(got, want, ("result", "final state", "entering states")):
        assert torch.equal(a, w), name
    if p <= 64:
        ep = (x, dt, D, bf, True)
        want = ops_ssd._lin_pass(dy.flip(1).contiguous(), ones, dA_cs, Br, Cr, dfin, want_entering=True, dx_epilogue=ep)
        got = ops_ssd._lin_pass(dy, ones, dA_cs, Br, Cr, dfin, want_entering=True, dx_epilogue=ep, x_reversed=True)
        for a, w, name in zip(got[0], want[0], ("dx", "xu", "s1")):
            assert torch.equal(a, w), name
    with pytest.raises(Exception, match="x_time_reversed"):
        ops_ssd.chunk_state(Br.float(), dy.float(), ones, dA_cs, x_reversed=True)


def test_backward_helpers_refuse_calls_they_do_not_cover():
    """The entry points added for the gradient say so when a call is outside what they cover, instead of computing
    something else: whole chunks for the preparation, the matrix-core kernel's own call for a finished ``dx``."""
    from ssm_amd.ops import ssd as ops_ssd
    gen = torch.Generator().manual_seed(0)
    bf = torch.bfloat16
    dt = torch.rand(1, 100, 2, generator=gen).cuda()
    A = -torch.rand(2, generator=gen).cuda()
    with pytest.raises(Exception, match="chunk"):
        ops_ssd._bwd_prep(dt, A, 64, None, False, (0.0, float("inf")))
    b, l, h, p, g, n, Q = 1, 128, 2, 64, 1, 32, 64
    x = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    Bm = torch.randn(b, l, g, n, generator=gen).to(bf).cuda()
    Cm = torch.randn(b, l, g, n, generator=gen).to(bf).cuda()
    dtc = torch.rand(b, l, h, generator=gen).cuda()
    dA_cs, dt_c = ops_ssd.chunk_cumsum(dtc, -torch.rand(h, generator=gen).cuda(), Q)
    ent = torch.zeros(b, l // Q, h, p, n).cuda()
    ep = (x, dtc, None, bf, True)
    # a gate of the call's own, or the shape-generic kernels, cannot finish dx
    with pytest.raises(Exception, match="dx_out"):
        ops_ssd.chunk_scan(Bm, Cm, x, dt_c, dA_cs, ent, z=x, dx_epilogue=ep)
    with pytest.raises(Exception, match="dx_out"):
        ops_ssd.chunk_scan(Bm, Cm, x, dt_c, dA_cs, ent, dx_epilogue=ep, force_generic=True)
    with pytest.raises(Exception, match="x_time_reversed"):
        ops_ssd.chunk_scan(Bm, Cm, x, dt_c, dA_cs, ent, D=torch.ones(h).cuda(), x_reversed=True)
    # and the ordinary call is untouched by all of it
    y = ops_ssd.chunk_scan(Bm, Cm, x, dt_c, dA_cs, ent)
    assert y.shape == x.shape and torch.isfinite(y.float()).all()


def test_one_pass_reads_b_and_c_cut_out_of_wider_rows_in_place():
    """``B`` and ``C`` as the two halves of one projected row (views with a row stride of ``2 G N``) give the bits of
    the call with dense copies, and no copy is made."""
    b, l, h, p, g, n, Q = 2, 512, 4, 64, 2, 64, 128
    gen = torch.Generator().manual_seed(17)
    bf = torch.bfloat16
    x = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    z = torch.randn(b, l, h, p, generator=gen).to(bf).cuda()
    bc = (torch.randn(b, l, 2 * g * n, generator=gen) * 0.5).to(bf).cuda()
    dt = (torch.rand(b, l, h, generator=gen) * 0.2).cuda()
    A = -(torch.rand(h, generator=gen) * 2 + 0.1).cuda()
    D = torch.randn(h, generator=gen).cuda()
    Bv, Cv = (t.reshape(b, l, g, n) for t in torch.split(bc, [g * n, g * n], dim=-1))
    assert not Bv.is_contiguous() and Bv.data_ptr() == bc.data_ptr()
    from ssm_amd.ops import ssd as ops_ssd
    assert ops_ssd._rows_in_place(Cv)[0] is Cv and ops_ssd._rows_in_place(Cv)[1] == 2 * g * n
    y, fin = ssd().ssd_combined(x, dt, A, Bv, Cv, Q, D=D, z=z, return_final_states=True, fused=True)
    y2, fin2 = ssd().ssd_combined(x, dt, A, Bv.contiguous(), Cv.contiguous(), Q, D=D, z=z, return_final_states=True, fused=True)
    assert torch.equal(y, y2) and torch.equal(fin, fin2)

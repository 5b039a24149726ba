"""GPU parity of the reference-semantics ``ssd_chunk_scan`` (diagonal chunk
scan) against the CPU oracle and the reference's two JSON goldens."""

import pytest
import torch

from oracle import ops_oracle as O
from tests import fixtures as fx

pytestmark = pytest.mark.gpu
FP32_TOL = dict(rtol=1e-5, atol=1e-5)
HALF_TOL = dict(rtol=2e-2, atol=2e-3)


def _ops():
    from ssm_amd import ops
    return ops


def dev(t):
    return None if t is None else t.cuda()


@pytest.mark.parametrize("name", ["ssd_chunk_scan_case1", "ssd_chunk_scan_varlen"])
def test_reference_goldens(name):
    i, o, _ = fx.nested_case(name)
    raw = i.get("seq_meta") or {}
    meta = {}
    if raw.get("seq_lens") is not None:
        meta["seq_lens"] = [int(v) for v in raw["seq_lens"]]
    if raw.get("cu_seqlens") is not None:
        meta["cu_seqlens"] = torch.tensor(raw["cu_seqlens"], dtype=torch.long)
    y = _ops().ssd_chunk_scan(dev(i["X"]), dev(i["dt"]), dev(i["A"]), dev(i["B"]), dev(i["C"]),
                              int(i["chunk_size"]), D=dev(i.get("D")), z=dev(i.get("z")), seq_meta=meta or None,
                              initial_states=dev(i.get("initial_states")))
    torch.testing.assert_close(y.cpu(), o["Y"], **FP32_TOL)


def make(seed, b, l, h, p, dtype=torch.float32, bkind=4, ckind=4, a_vec=False, d_mode="vec", z_mode=4, init=True):
    g = torch.Generator().manual_seed(seed)
    X = torch.randn(b, l, h, p, generator=g).to(dtype)
    dt = (torch.rand(b, l, h, generator=g) * 0.2).to(dtype)
    A = -(torch.rand(h, generator=g) * 4 + 0.1) if a_vec else -(torch.rand(h, p, generator=g) * 4 + 0.1)

    def proj(k):
        shape = {2: (h, p), 3: (b, h, p), 4: (b, l, h, p)}[k]
        return torch.randn(*shape, generator=g).to(dtype)

    D = {"none": None, "vec": torch.randn(h, generator=g), "mat": torch.randn(h, p, generator=g)}[d_mode]
    z = {0: None, 3: torch.randn(b, l, h, generator=g).to(dtype), 4: torch.randn(b, l, h, p, generator=g).to(dtype)}[z_mode]
    init_s = torch.randn(b, h, p, generator=g) if init else None
    return dict(X=X, dt=dt, A=A, B=proj(bkind), C=proj(ckind), D=D, z=z, init=init_s)


def both(inp, chunk=64, meta=None):
    yr = O.ssd_chunk_scan(inp["X"], inp["dt"], inp["A"], inp["B"], inp["C"], chunk, D=inp["D"], z=inp["z"],
                          seq_meta=meta, initial_states=inp["init"])
    y = _ops().ssd_chunk_scan(dev(inp["X"]), dev(inp["dt"]), dev(inp["A"]), dev(inp["B"]), dev(inp["C"]), chunk,
                              D=dev(inp["D"]), z=dev(inp["z"]), seq_meta=meta, initial_states=dev(inp["init"]))
    return y.cpu(), yr


@pytest.mark.parametrize("shape", [(1, 1, 1, 1), (2, 6, 2, 3), (2, 37, 3, 5), (1, 384, 4, 64), (2, 1000, 2, 8)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("kinds", [(4, 4), (2, 2), (3, 4), (4, 2)])
def test_fp32_matches_oracle(shape, kinds):
    inp = make(sum(shape), *shape, bkind=kinds[0], ckind=kinds[1])
    y, yr = both(inp)
    torch.testing.assert_close(y, yr, **FP32_TOL)


@pytest.mark.parametrize("a_vec,d_mode,z_mode,init", [(True, "none", 0, False), (True, "mat", 3, True),
                                                      (False, "vec", 4, False), (False, "none", 3, True)])
def test_option_matrix(a_vec, d_mode, z_mode, init):
    inp = make(7, 2, 130, 3, 6, a_vec=a_vec, d_mode=d_mode, z_mode=z_mode, init=init)
    y, yr = both(inp)
    torch.testing.assert_close(y, yr, **FP32_TOL)


def test_ragged_lengths_and_chunk_invariance():
    inp = make(3, 3, 200, 2, 4)
    for meta in ({"seq_lens": [200, 77, 0]}, {"cu_seqlens": torch.tensor([0, 5, 205, 300])}):
        y, yr = both(inp, chunk=16, meta=meta)
        torch.testing.assert_close(y, yr, **FP32_TOL)
    y2, _ = both(inp, chunk=7, meta={"seq_lens": [200, 77, 0]})
    y3, _ = both(inp, chunk=512, meta={"seq_lens": [200, 77, 0]})
    assert torch.equal(y2, y3)
    assert torch.count_nonzero(y2[1, 77:]) == 0 and torch.count_nonzero(y2[2]) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_half(dtype):
    inp = make(5, 2, 384, 4, 64, dtype=dtype)
    y, yr = both(inp)
    assert y.dtype == dtype
    torch.testing.assert_close(y.float(), yr.float(), **HALF_TOL)


def test_config3_outer_shape_bf16_slice():
    """(B, L, H, P) = (4, 4096, 80, 64) in bf16 with A (80,), B, C (80, 64): full size on the
    GPU; two heads are replayed on the oracle (heads are independent)."""
    g = torch.Generator().manual_seed(3)
    X = torch.randn(4, 4096, 80, 64, generator=g).to(torch.bfloat16)
    dt = torch.nn.functional.softplus(torch.randn(4, 4096, 80, generator=g) - 3).to(torch.bfloat16)
    A = -(torch.rand(80, generator=g) * 15 + 1)
    Bm = torch.randn(80, 64, generator=g).to(torch.bfloat16)
    Cm = torch.randn(80, 64, generator=g).to(torch.bfloat16)
    D = torch.ones(80)
    z = torch.randn(4, 4096, 80, 64, generator=g).to(torch.bfloat16)
    y = _ops().ssd_chunk_scan(X.cuda(), dt.cuda(), A.cuda(), Bm.cuda(), Cm.cuda(), 256, D=D.cuda(), z=z.cuda())
    hs = [3, 77]
    yr = O.ssd_chunk_scan(X[:, :, hs], dt[:, :, hs], A[hs], Bm[hs], Cm[hs], 256, D=D[hs], z=z[:, :, hs])
    torch.testing.assert_close(y[:, :, hs].float().cpu(), yr.float(), **HALF_TOL)


def _full_size_heads_oracle(inp, hs, gy, chunk):
    """Forward in float32 and all gradients in float64 of the heads ``hs`` alone (heads are independent)."""
    def cut(k, v):
        if v is None:
            return None
        if k in ("X", "z", "dt") or v.ndim == 4:
            return v[:, :, hs]
        return v[hs]
    sub = {k: cut(k, v) for k, v in inp.items()}
    y32 = O.ssd_chunk_scan(sub["X"], sub["dt"], sub["A"], sub["B"], sub["C"], chunk, D=sub["D"], z=sub["z"])
    leaves = {k: (v.double().clone().requires_grad_(True) if v is not None else None) for k, v in sub.items()}
    y = O.ssd_chunk_scan(leaves["X"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], chunk, D=leaves["D"],
                         z=leaves["z"], acc=torch.float64)
    (y.double() * gy[:, :, hs].double()).sum().backward()
    return y32, {k: (v.grad if v is not None else None) for k, v in leaves.items()}, cut


def test_config3_outer_shape_one_pass_per_token_projections():
    """(B, L, H, P) = (4, 4096, 80, 64), bf16 X, z and per-token B, C of X's shape, **float32 dt**, per-head A and
    D: the call whose forward and backward ``bench.py`` times, which runs the one-pass kernels on a grid of
    320 workgroups.  Forward and, through autograd (which hands the forward's table of round states over), all
    seven gradients of two heads against the oracle on those heads alone (float64 autograd for the gradients)."""
    from tests.closeness import half_close
    g = torch.Generator().manual_seed(43)
    b, l, h, p = 4, 4096, 80, 64
    inp = dict(X=torch.randn(b, l, h, p, generator=g).to(torch.bfloat16),
               dt=torch.rand(b, l, h, generator=g) * 0.1,
               A=-(torch.rand(h, generator=g) * 15 + 1),
               B=torch.randn(b, l, h, p, generator=g).to(torch.bfloat16),
               C=torch.randn(b, l, h, p, generator=g).to(torch.bfloat16),
               D=torch.ones(h), z=torch.randn(b, l, h, p, generator=g).to(torch.bfloat16))
    gy = torch.randn(b, l, h, p, generator=g).to(torch.bfloat16)
    hs = [0, 41, 79]
    as_f32 = {k: v.float() for k, v in inp.items()}
    yr, want, cut = _full_size_heads_oracle(as_f32, hs, gy.float(), 256)
    leaves = {k: dev(v).requires_grad_(True) for k, v in inp.items()}
    y = _ops().ssd_chunk_scan(leaves["X"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 256, D=leaves["D"],
                              z=leaves["z"])
    assert y.dtype == torch.bfloat16
    torch.testing.assert_close(y[:, :, hs].float().cpu(), yr.float(), **HALF_TOL)
    (y * dev(gy)).sum().backward()
    for k, v in leaves.items():
        assert v.grad.dtype == inp[k].dtype and v.grad.shape == inp[k].shape, k
        half_close(cut(k, v.grad), want[k], what=f"grad {k}", atol_rms=4e-2, mean_rms=5e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_config3_outer_shape_one_pass_module_call(dtype):
    """The call of the reference's Mamba2 module at (4, 4096, 80, 64): B, C, A, D as (H, P) float32 parameters, no
    gate, float32 dt (``/root/reference/src/ssm/modules/mamba2.py:189-199``), activations in float32 as the module
    promotes them and in bf16.  Forward and, through autograd, all gradients of three heads against the oracle
    (float64 autograd for the gradients; the float32 oracle arbitrates float32 values)."""
    from tests.closeness import fp32_close, half_close
    g = torch.Generator().manual_seed(44)
    b, l, h, p = 4, 4096, 80, 64
    inp = dict(X=torch.randn(b, l, h, p, generator=g).to(dtype),
               dt=torch.rand(b, l, h, generator=g) * 0.1,
               A=-(torch.rand(h, p, generator=g) * 15 + 1),
               B=torch.randn(h, p, generator=g), C=torch.randn(h, p, generator=g),
               D=torch.ones(h, p), z=None)
    gy = torch.randn(b, l, h, p, generator=g).to(dtype)
    hs = [1, 40, 78]
    as_f32 = {k: (v.float() if v is not None else None) for k, v in inp.items()}
    yr, want, cut = _full_size_heads_oracle(as_f32, hs, gy.float(), 256)
    leaves = {k: (dev(v).requires_grad_(True) if v is not None else None) for k, v in inp.items()}
    y = _ops().ssd_chunk_scan(leaves["X"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 256, D=leaves["D"])
    assert y.dtype == dtype
    half = dtype != torch.float32
    torch.testing.assert_close(y[:, :, hs].float().cpu(), yr.float(), **(HALF_TOL if half else FP32_TOL))
    (y * dev(gy)).sum().backward()
    # float32 autograd through the oracle: what float32 sums over 16384 steps are worth
    l32 = {k: (cut(k, v).clone().requires_grad_(True) if v is not None else None) for k, v in as_f32.items()}
    y32 = O.ssd_chunk_scan(l32["X"], l32["dt"], l32["A"], l32["B"], l32["C"], 256, D=l32["D"])
    (y32 * gy[:, :, hs].float()).sum().backward()
    for k, v in leaves.items():
        if v is None:
            continue
        assert v.grad.dtype == inp[k].dtype and v.grad.shape == inp[k].shape, k
        if half:
            half_close(cut(k, v.grad), want[k], what=f"grad {k}", atol_rms=4e-2, mean_rms=5e-3)
        else:
            fp32_close(cut(k, v.grad), want[k], oracle32=l32[k].grad, what=f"grad {k}", rtol=1e-4, atol_rms=1e-5)


# ---------------------------------------------------------------------------
# backward: all eight gradients against float64 autograd through the CPU restatement
# ---------------------------------------------------------------------------

GRAD_NAMES = ["X", "dt", "A", "B", "C", "D", "z", "init"]


def _grads_oracle(inp, meta, gy):
    leaves = {k: (inp[k].double().clone().requires_grad_(True) if inp.get(k) is not None else None) for k in GRAD_NAMES}
    y = O.ssd_chunk_scan(leaves["X"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 16, D=leaves["D"],
                         z=leaves["z"], seq_meta=meta, initial_states=leaves["init"], acc=torch.float64)
    (y.double() * gy.double()).sum().backward()
    return {k: (v.grad if v is not None else None) for k, v in leaves.items()}


def _grads_gpu(inp, meta, gy):
    leaves = {k: (dev(inp[k]).clone().requires_grad_(True) if inp.get(k) is not None else None) for k in GRAD_NAMES}
    y = _ops().ssd_chunk_scan(leaves["X"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"], 16, D=leaves["D"],
                              z=leaves["z"], seq_meta=meta, initial_states=leaves["init"])
    (y * dev(gy)).sum().backward()
    return {k: (v.grad if v is not None else None) for k, v in leaves.items()}


@pytest.mark.parametrize("kinds", [(4, 4), (2, 3), (3, 2), (4, 2)])
@pytest.mark.parametrize("a_vec,d_mode,z_mode,init", [(False, "vec", 4, True), (True, "mat", 3, True),
                                                      (True, "none", 0, False), (False, "vec", 3, False)])
def test_backward_matches_float64_autograd(kinds, a_vec, d_mode, z_mode, init):
    b, l, h, p = 2, 21, 3, 5
    inp = make(41 + kinds[0] + 3 * kinds[1], b, l, h, p, bkind=kinds[0], ckind=kinds[1], a_vec=a_vec, d_mode=d_mode,
               z_mode=z_mode, init=init)
    gy = torch.randn(b, l, h, p, generator=torch.Generator().manual_seed(8))
    want = _grads_oracle(inp, None, gy)
    got = _grads_gpu(inp, None, gy)
    for k in GRAD_NAMES:
        if want[k] is None:
            assert got[k] is None
            continue
        torch.testing.assert_close(got[k].cpu().double(), want[k], rtol=2e-4, atol=2e-5,
                                   msg=lambda m, n=k: f"grad {n}: {m}")


def test_backward_with_ragged_lengths():
    b, l, h, p = 3, 17, 2, 4
    inp = make(77, b, l, h, p, bkind=4, ckind=4)
    meta = {"seq_lens": [17, 5, 0]}
    gy = torch.randn(b, l, h, p, generator=torch.Generator().manual_seed(9))
    want = _grads_oracle(inp, meta, gy)
    got = _grads_gpu(inp, meta, gy)
    for k in GRAD_NAMES:
        torch.testing.assert_close(got[k].cpu().double(), want[k], rtol=2e-4, atol=2e-5,
                                   msg=lambda m, n=k: f"grad {n}: {m}")
    assert float(got["X"][2].abs().max()) == 0.0        # a row of length 0 receives no gradient


def test_backward_bf16_activations():
    b, l, h, p = 2, 64, 2, 8
    inp = make(78, b, l, h, p, dtype=torch.bfloat16, bkind=4, ckind=4)
    gy = torch.randn(b, l, h, p, generator=torch.Generator().manual_seed(10)).to(torch.bfloat16)
    want = _grads_oracle({k: (v.float() if v is not None else None) for k, v in inp.items()}, None, gy.float())
    got = _grads_gpu(inp, None, gy)
    for k in GRAD_NAMES:
        scale = float(want[k].abs().max()) + 1e-6
        torch.testing.assert_close(got[k].float().cpu().double(), want[k], rtol=3e-2, atol=3e-2 * scale,
                                   msg=lambda m, n=k: f"grad {n}: {m}")


# ------------------------------------------------------------------ the one-pass kernel's call shape

@pytest.mark.parametrize("dtype,hp", [(torch.bfloat16, (4, 64)), (torch.float16, (2, 64)), (torch.float32, (3, 64)),
                                      (torch.bfloat16, (8, 32))], ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("length,z_mode,d_mode,init,ragged", [(333, 4, "vec", True, False), (128, 0, "none", False, False),
                                                               (1000, 4, "vec", False, True), (7, 4, "none", True, True)])
def test_one_pass_call_shape(dtype, hp, length, z_mode, d_mode, init, ragged):
    """Per-token B and C of X's type, float32 dt, per-head A and D, a gate of X's shape or none, channels in whole
    waves: the kernel that reads every input once (rounds of 128 steps over 16 waves), over lengths that are not a
    multiple of a round, with an entering state and with rows that end early."""
    h, p = hp
    b = 3
    inp = make(length + h, b, length, h, p, dtype=dtype, a_vec=True, d_mode=d_mode, z_mode=z_mode, init=init)
    inp["dt"] = inp["dt"].float()
    meta = {"seq_lens": [length, max(length // 3, 0), 0]} if ragged else None
    y, yr = both(inp, meta=meta)
    assert y.dtype == dtype
    torch.testing.assert_close(y.float(), yr.float(), **(FP32_TOL if dtype == torch.float32 else HALF_TOL))
    if ragged:
        assert torch.count_nonzero(y[2]) == 0 and torch.count_nonzero(y[1, length // 3:]) == 0


@pytest.mark.parametrize("dtype,hp", [(torch.bfloat16, (4, 64)), (torch.float16, (2, 128)), (torch.float32, (3, 64)),
                                      (torch.bfloat16, (8, 32)), (torch.float32, (8, 16))],
                         ids=lambda v: str(v).replace("torch.", ""))
@pytest.mark.parametrize("length,z_mode,d_mode,init,ragged", [(333, 4, "vec", True, False), (128, 0, "none", False, False),
                                                               (200, 4, "vec", False, True), (7, 4, "none", True, True)])
def test_one_pass_backward_call_shape(dtype, hp, length, z_mode, d_mode, init, ragged):
    """The same call shape backwards (a table of the states entering every 64 steps, then one walk from the end that
    reads every input once): all eight gradients against float64 autograd through the oracle and against the general
    two-kernel path, with float32 gradients and with dB, dC, dz written in the tensors' own types."""
    ops = _ops()
    h, p = hp
    b = 3
    inp = make(2 * length + h, b, length, h, p, dtype=dtype, a_vec=True, d_mode=d_mode, z_mode=z_mode, init=init)
    inp["dt"] = inp["dt"].float()
    lens = [length, max(length // 3, 0), 0] if ragged else None
    meta = {"seq_lens": lens} if ragged else None
    gy = torch.randn(b, length, h, p, generator=torch.Generator().manual_seed(length)).to(dtype)
    want = _grads_oracle({k: (v.float() if v is not None else None) for k, v in inp.items()}, meta, gy.float())
    d = {k: dev(v) for k, v in inp.items()}
    lengths = torch.tensor(lens, dtype=torch.int32).cuda() if ragged else None
    run = lambda **kw: ops._dscan_backward(dev(gy), d["X"], d["dt"], d["A"], d["B"], d["C"], 64, d["D"], d["z"], lengths,
                                           d["init"], **kw)
    one = run()
    two = run(two_kernels=True)
    own = run(grads_in_input_dtype=True)
    names = ["X", "dt", "A", "B", "C", "D", "z", "init"]
    half = dtype != torch.float32
    for k, g1, g2, g3 in zip(names, one, two, own):
        if want[k] is None:
            assert g1 is None and g3 is None
            continue
        w = want[k]
        scale = float(w.abs().max()) + 1e-6
        tol = dict(rtol=3e-2, atol=3e-2 * scale) if half else dict(rtol=2e-4, atol=2e-5 * max(scale, 1.0))
        assert g1.dtype == (dtype if k == "X" else torch.float32) and g1.shape == w.shape, k
        torch.testing.assert_close(g1.float().cpu().double(), w, msg=lambda m, n=k: f"grad {n} against the oracle: {m}", **tol)
        # the two paths sum in different orders; both are float32 sums of the same terms
        torch.testing.assert_close(g1.float(), g2.float(), rtol=1e-2 if half else 1e-4,
                                   atol=(1e-2 if half else 1e-5) * max(scale, 1.0),
                                   msg=lambda m, n=k: f"grad {n} against the two-kernel path: {m}")
        # the same arithmetic compiled a second time (fused differently here and there): one rounding of the type apart
        ulp = {torch.float32: 2.0 ** -20, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}
        if k in ("B", "C", "z"):
            assert g3.dtype == dtype, k
            torch.testing.assert_close(g3.float(), g1.float(), rtol=ulp[dtype], atol=ulp[dtype] * 1e-2 * max(scale, 1.0),
                                       msg=lambda m, n=k: f"grad {n} in its own type: {m}")
        else:
            assert g3.dtype == g1.dtype, k
            torch.testing.assert_close(g3.float(), g1.float(), rtol=ulp[dtype] if k == "X" else 1e-5,
                                       atol=1e-5 * max(scale, 1.0), msg=lambda m, n=k: f"grad {n}: {m}")
    if ragged:
        assert float(one[0][2].abs().max()) == 0.0 and float(one[3][1, length // 3:].abs().max()) == 0.0
    # the forward can leave the table of round states for the backward: the same gradients without the extra sweep
    y, table = ops._dscan_forward(d["X"], d["dt"], d["A"], d["B"], d["C"], 64, d["D"], d["z"], lengths, d["init"],
                                  want_round_states=True)
    assert table is not None and tuple(table.shape) == (b, (length + 63) // 64, h * p)
    for k, g1, g4 in zip(names, one, run(round_states=table)):
        if g1 is not None:
            torch.testing.assert_close(g4, g1, rtol=1e-6, atol=0, msg=lambda m, n=k: f"grad {n} with the forward's table: {m}")
    # and through autograd, which does exactly that and returns every gradient in its tensor's type
    auto = _grads_gpu(inp, meta, gy)
    for k, g3 in zip(names, own):
        if g3 is None:
            continue
        key = "init" if k == "init" else k
        assert auto[key].dtype == inp[key].dtype and auto[key].shape == inp[key].shape, k
        torch.testing.assert_close(auto[key].float(), g3.to(inp[key].dtype).float().reshape(inp[key].shape), rtol=1e-6, atol=0,
                                   msg=lambda m, n=k: f"grad {n} through autograd: {m}")


# ------------------------------------------------------------------ B and C as parameters: the reference module's call

@pytest.mark.parametrize("dtype,hp,kinds", [(torch.float32, (3, 64), (2, 2)), (torch.bfloat16, (4, 64), (2, 3)),
                                            (torch.float16, (2, 128), (3, 2)), (torch.float32, (8, 16), (3, 3)),
                                            (torch.bfloat16, (8, 32), (2, 2))],
                         ids=lambda v: str(v).replace("torch.", "").replace(" ", ""))
@pytest.mark.parametrize("length,a_vec,z_mode,d_mode,init,ragged",
                         [(333, False, 0, "mat", False, False), (128, True, 4, "vec", True, False),
                          (200, False, 0, "mat", False, True), (7, False, 4, "none", True, True),
                          (130, True, 0, "none", False, False)])
def test_one_pass_with_parameter_projections(dtype, hp, kinds, length, a_vec, z_mode, d_mode, init, ragged):
    """``B`` and ``C`` of shape ``(H, P)`` or ``(B, H, P)`` -- float32 parameters beside activations of any type -- with
    ``A`` and ``D`` per channel or per head, no gate (or one of X's shape) and ``seq_lens``: what the reference's Mamba2
    module passes (src/ssm/modules/mamba2.py:189-199).  The one-pass kernels keep the two projections in registers and
    sum their gradients over time.  Forward against the oracle; every gradient against float64 autograd through the
    oracle and against the general two-kernel path; the forward's table of round states in place of the sweep."""
    ops = _ops()
    h, p = hp
    b = 3
    inp = make(3 * length + h, b, length, h, p, dtype=dtype, bkind=kinds[0], ckind=kinds[1], a_vec=a_vec, d_mode=d_mode,
               z_mode=z_mode, init=init)
    inp["dt"] = inp["dt"].float()
    inp["B"], inp["C"] = inp["B"].float(), inp["C"].float()
    lens = [length, max(length // 3, 0), 0] if ragged else None
    meta = {"seq_lens": lens} if ragged else None
    half = dtype != torch.float32
    y, yr = both(inp, meta=meta)
    assert y.dtype == dtype
    torch.testing.assert_close(y.float(), yr.float(), **(HALF_TOL if half else FP32_TOL))
    if ragged:
        assert torch.count_nonzero(y[2]) == 0 and torch.count_nonzero(y[1, length // 3:]) == 0

    gy = torch.randn(b, length, h, p, generator=torch.Generator().manual_seed(length)).to(dtype)
    want = _grads_oracle({k: (v.float() if v is not None else None) for k, v in inp.items()}, meta, gy.float())
    d = {k: dev(v) for k, v in inp.items()}
    lengths = torch.tensor(lens, dtype=torch.int32).cuda() if ragged else None
    run = lambda **kw: ops._dscan_backward(dev(gy), d["X"], d["dt"], d["A"], d["B"], d["C"], 64, d["D"], d["z"], lengths,
                                           d["init"], **kw)
    one = run()
    two = run(two_kernels=True)
    for k, g1, g2 in zip(GRAD_NAMES, one, two):
        if want[k] is None:
            assert g1 is None
            continue
        w = want[k]
        scale = float(w.abs().max()) + 1e-6
        tol = dict(rtol=3e-2, atol=3e-2 * scale) if half else dict(rtol=2e-4, atol=2e-5 * max(scale, 1.0))
        assert g1.dtype == (dtype if k == "X" else torch.float32) and g1.shape == w.shape, k
        torch.testing.assert_close(g1.float().cpu().double(), w, msg=lambda m, n=k: f"grad {n} against the oracle: {m}", **tol)
        torch.testing.assert_close(g1.float(), g2.float(), rtol=1e-2 if half else 1e-4,
                                   atol=(1e-2 if half else 1e-5) * max(scale, 1.0),
                                   msg=lambda m, n=k: f"grad {n} against the two-kernel path: {m}")
    if ragged:
        assert float(one[0][2].abs().max()) == 0.0 and float(one[1][1, length // 3:].abs().max()) == 0.0
    y2, table = ops._dscan_forward(d["X"], d["dt"], d["A"], d["B"], d["C"], 64, d["D"], d["z"], lengths, d["init"],
                                   want_round_states=True)
    assert table is not None and tuple(table.shape) == (b, (length + 63) // 64, h * p)
    for k, g1, g4 in zip(GRAD_NAMES, one, run(round_states=table)):
        if g1 is not None:
            torch.testing.assert_close(g4, g1, rtol=1e-6, atol=0, msg=lambda m, n=k: f"grad {n} with the forward's table: {m}")
    auto = _grads_gpu(inp, meta, gy)
    for k, g1 in zip(GRAD_NAMES, run(grads_in_input_dtype=True)):
        if g1 is None:
            continue
        assert auto[k].dtype == inp[k].dtype and auto[k].shape == inp[k].shape, k
        torch.testing.assert_close(auto[k].float(), g1.to(inp[k].dtype).float().reshape(inp[k].shape), rtol=1e-6, atol=0,
                                   msg=lambda m, n=k: f"grad {n} through autograd: {m}")

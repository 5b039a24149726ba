"""Pins the CPU oracle against every vector the reference holds for the path,
library special cases and closed forms.  CPU only."""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ops_oracle as O
from oracle import ssd_oracle as S
from tests import fixtures as fx

torch.manual_seed(0)


# ------------------------------------------------------------- selective scan

@pytest.mark.parametrize("name", ["selective_scan_case1", "selective_scan_grouped"])
def test_scan_reference_nested_goldens(name):
    i, o, _ = fx.nested_case(name)
    y, h = O.selective_scan(i["u"], i["delta"], i["A"], i["B"], i["C"], D=i["D"], z=i["z"],
                            dt_bias=i["dt_bias"], softplus=bool(i["softplus"]),
                            return_last_state=True)
    torch.testing.assert_close(y, o["out"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(h, o["last_state"], rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("case", fx.flat_cases(), ids=lambda c: c[0])
def test_scan_reference_flat_goldens(case):
    _, i, o = case
    y, h = O.selective_scan(i["u"], i["delta"], i["A"], i["B"], i["C"], D=i["D"], z=i["z"],
                            dt_bias=i["dt_bias"], softplus=True, return_last_state=True)
    torch.testing.assert_close(y, o["y"], rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(h, o["state"], rtol=1e-6, atol=1e-6)


def _upstream_scan_args(case):
    rec = fx.upstream("selective_scan", case)
    i = rec["inputs"]
    B, C = i["B"], i["C"]
    if case == "time_varying_3d":          # upstream (batch, N, L) == one group
        B, C = B[:, None], C[:, None]
    if case == "grouped_time_varying":
        # The vector was recorded with D=3 channels and G=2 groups, which the
        # reference rejects (G must divide D); upstream then reads channel 2's
        # projections out of bounds.  Channels 0-1 (one per group) are well
        # defined, and so are the B/C gradients of batch row 0.
        i = dict(i)
        for k in ("u", "delta"):
            i[k] = i[k][:, :2]
        i["A"] = i["A"][:2]
        i["delta_bias"] = i["delta_bias"][:2]
    flags = {
        "full": dict(softplus=True),
        "minimal": dict(softplus=False),
        "minimal_fp16": dict(softplus=False),
        "minimal_bf16": dict(softplus=False),
        "grouped_time_varying": dict(softplus=True),
        "time_varying_3d": dict(softplus=True),
    }[case]
    return rec, i, B, C, flags


@pytest.mark.parametrize("case", ["full", "minimal", "minimal_fp16", "minimal_bf16",
                                  "grouped_time_varying", "time_varying_3d"])
def test_scan_upstream_forward_and_grads(case):
    rec, i, B, C, flags = _upstream_scan_args(case)
    leaves = {}

    def leaf(t):
        return None if t is None else t.clone().requires_grad_(True)

    leaves["u"], leaves["delta"], leaves["A"] = leaf(i["u"]), leaf(i["delta"]), leaf(i["A"])
    leaves["B"], leaves["C"] = leaf(B), leaf(C)
    leaves["D"], leaves["z"] = leaf(i.get("D")), leaf(i.get("z"))
    leaves["delta_bias"] = leaf(i.get("delta_bias"))
    y = O.selective_scan(leaves["u"], leaves["delta"], leaves["A"], leaves["B"], leaves["C"],
                         D=leaves["D"], z=leaves["z"], dt_bias=leaves["delta_bias"], **flags)
    half = i["u"].dtype != torch.float32
    tol = dict(rtol=2e-2, atol=2e-2) if half else dict(rtol=1e-4, atol=1e-5)
    want = rec["outputs"]["y"]
    if case == "grouped_time_varying":
        want = want[:, :2]
    torch.testing.assert_close(y, want, **tol)
    y.float().sum().backward()
    for name, g in rec["gradients"].items():
        if g is None:
            continue
        got = leaves[name].grad
        if case == "time_varying_3d" and name in ("B", "C"):
            got = got[:, 0]
        if case == "grouped_time_varying":
            if name in ("B", "C"):
                got, g = got[0], g[0]
            elif name in ("A", "delta_bias"):
                g = g[:2]
            else:
                g = g[:, :2]
        gtol = dict(rtol=3e-2, atol=3e-2) if half else dict(rtol=2e-4, atol=2e-5)
        ok = torch.isfinite(g)        # upstream's backward overflowed on rows with A > 0
        if not ok.any():
            continue
        torch.testing.assert_close(got.to(g.dtype)[ok], g[ok], **gtol)


def test_scan_geometric_series_closed_form():
    # B = C = 1, constant delta and u: h_t = b (1 - a^t) / (1 - a)
    Bsz, D, L, N = 1, 3, 40, 2
    A = -torch.rand(D, N, dtype=torch.float64) - 0.1
    dt = 0.05
    u = torch.full((Bsz, D, L), 0.7, dtype=torch.float64)
    delta = torch.full((Bsz, D, L), dt, dtype=torch.float64)
    ones = torch.ones(D, N, dtype=torch.float64)
    y, h = O.selective_scan(u, delta, A, ones, ones, return_last_state=True)
    a = torch.exp(dt * A)
    t = torch.arange(1, L + 1, dtype=torch.float64)
    hs = dt * 0.7 * (1 - a[:, :, None] ** t) / (1 - a[:, :, None])      # (D,N,L)
    torch.testing.assert_close(y[0], hs.sum(1), rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(h[0], hs[:, :, -1], rtol=1e-10, atol=1e-12)


def test_scan_equals_repeated_state_step():
    Bsz, D, L, N, G = 2, 4, 9, 3, 2
    u = torch.randn(Bsz, D, L); delta = torch.randn(Bsz, D, L)
    A = -torch.rand(D, N); Bm = torch.randn(Bsz, G, N, L); Cm = torch.randn(Bsz, G, N, L)
    Dk = torch.randn(D); z = torch.randn(Bsz, D, L); bias = torch.randn(D)
    y, h = O.selective_scan(u, delta, A, Bm, Cm, D=Dk, z=z, dt_bias=bias, softplus=True,
                            return_last_state=True)
    st = torch.zeros(Bsz, D, N)
    for t in range(L):
        yt = O.selective_state_step(st, u[:, :, t], delta[:, :, t], A, Bm[..., t], Cm[..., t],
                                    D=Dk, z=z[:, :, t], dt_bias=bias, softplus=True)
        torch.testing.assert_close(yt, y[:, :, t], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(st, h, rtol=1e-5, atol=1e-6)


# ----------------------------------------------------------------- state step

def test_state_step_upstream_baseline():
    rec = fx.upstream("selective_state_update", "baseline_full")
    i = rec["inputs"]
    st = i["state"].clone()
    y = O.selective_state_step(st, i["x"], i["dt"], i["A"], i["B"][:, None], i["C"][:, None],
                               D=i["D"], z=i["z"], dt_bias=i["dt_bias"], softplus=True)
    torch.testing.assert_close(y, rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(st, rec["outputs"]["updated_state"], rtol=1e-4, atol=1e-5)


def test_state_step_upstream_grouped_heads():
    # upstream carries a head axis: (B,H,D,N); fold H*D into channels, groups == H
    rec = fx.upstream("selective_state_update", "grouped")
    i = rec["inputs"]
    b, h, d, n = i["state"].shape
    st = i["state"].reshape(b, h * d, n).clone()
    y = O.selective_state_step(st, i["x"].reshape(b, h * d), i["dt"].reshape(b, h * d),
                               i["A"].reshape(h * d, n), i["B"], i["C"],
                               dt_bias=i["dt_bias"].reshape(h * d), softplus=False)
    torch.testing.assert_close(y.reshape(b, h, d), rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(st.reshape(b, h, d, n), rec["outputs"]["updated_state"],
                               rtol=1e-4, atol=1e-5)


# ------------------------------------------- reference-semantics ssd_chunk_scan

@pytest.mark.parametrize("name", ["ssd_chunk_scan_case1", "ssd_chunk_scan_varlen"])
def test_dscan_reference_goldens(name):
    i, o, _ = fx.nested_case(name)
    meta = {}
    raw = i.get("seq_meta") or {}
    if raw.get("seq_lens") is not None:
        meta["seq_lens"] = [int(v) for v in raw["seq_lens"]]
    if raw.get("cu_seqlens") is not None:
        meta["cu_seqlens"] = torch.tensor(raw["cu_seqlens"], dtype=torch.long)
    y = O.ssd_chunk_scan(i["X"], i["dt"], i["A"], i["B"], i["C"], int(i["chunk_size"]),
                         D=i.get("D"), z=i.get("z"), seq_meta=meta or None,
                         initial_states=i.get("initial_states"))
    torch.testing.assert_close(y, o["Y"], rtol=1e-5, atol=1e-6)


def test_dscan_chunk_invariance_and_tail():
    X = torch.randn(2, 11, 3, 4); dt = torch.rand(2, 11, 3)
    A = -torch.rand(3, 4); Bm = torch.randn(3, 4); Cm = torch.randn(2, 3, 4)
    ys = [O.ssd_chunk_scan(X, dt, A, Bm, Cm, q, seq_meta={"seq_lens": [11, 6]}) for q in (1, 4, 64)]
    torch.testing.assert_close(ys[0], ys[1]); torch.testing.assert_close(ys[0], ys[2])
    assert torch.count_nonzero(ys[0][1, 6:]) == 0


def test_dscan_is_scan_with_one_state_per_channel():
    Bsz, L, H, P = 2, 7, 2, 3
    X = torch.randn(Bsz, L, H, P); dt = torch.rand(Bsz, L, H)
    A = -torch.rand(H, P); Bm = torch.randn(Bsz, L, H, P); Cm = torch.randn(Bsz, L, H, P)
    y = O.ssd_chunk_scan(X, dt, A, Bm, Cm, 4)
    u = X.reshape(Bsz, L, H * P).permute(0, 2, 1)
    dl = dt[..., None].expand(Bsz, L, H, P).reshape(Bsz, L, H * P).permute(0, 2, 1)
    B4 = Bm.reshape(Bsz, L, H * P).permute(0, 2, 1)[:, :, None, :]
    C4 = Cm.reshape(Bsz, L, H * P).permute(0, 2, 1)[:, :, None, :]
    ys = O.selective_scan(u, dl, A.reshape(H * P, 1), B4, C4)
    torch.testing.assert_close(ys.permute(0, 2, 1).reshape(Bsz, L, H, P), y, rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------------ conv

def test_conv_upstream_channels_first_silu():
    rec = fx.upstream("dw_causal_conv", "channels_first_silu")
    i = rec["inputs"]
    x = i["x"].clone().requires_grad_(True); w = i["weight"].clone().requires_grad_(True)
    b = i["bias"].clone().requires_grad_(True)
    y = O.dw_causal_conv(x, w, b, activation="silu")
    torch.testing.assert_close(y, rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    y.sum().backward()
    for name, t in (("x", x), ("weight", w), ("bias", b)):
        torch.testing.assert_close(t.grad, rec["gradients"][name], rtol=1e-4, atol=1e-5)


def test_conv_upstream_channels_last_identity():
    rec = fx.upstream("dw_causal_conv", "channels_last_identity")
    i = rec["inputs"]
    x = i["x"].clone().requires_grad_(True); w = i["weight"].clone().requires_grad_(True)
    y = O.dw_causal_conv(x, w, None, activation="identity")
    torch.testing.assert_close(y, rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    y.sum().backward()
    torch.testing.assert_close(x.grad, rec["gradients"]["x"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(w.grad, rec["gradients"]["weight"], rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("K", [1, 2, 3, 4, 5])
def test_conv_equals_library_conv1d(K):
    x = torch.randn(2, 6, 13, dtype=torch.float64); w = torch.randn(6, K, dtype=torch.float64)
    b = torch.randn(6, dtype=torch.float64)
    want = F.silu(F.conv1d(F.pad(x, (K - 1, 0)), w[:, None], bias=b, groups=6))
    torch.testing.assert_close(O.dw_causal_conv(x, w, b, "silu"), want)
    got_last = O.dw_causal_conv(x.permute(0, 2, 1).contiguous(), w[:, None, :], b, "swish")
    torch.testing.assert_close(got_last, want.permute(0, 2, 1))


# ------------------------------------------------------------------ layer norm

def test_norm_upstream_layer_norm_prenorm():
    rec = fx.upstream("layer_norms", "layer_norm_prenorm")
    i = rec["inputs"]
    x = i["x"].clone().requires_grad_(True); w = i["w"].clone().requires_grad_(True)
    b = i["b"].clone().requires_grad_(True); r = i["residual"].clone().requires_grad_(True)
    y, res_out = O.fused_layer_norm_with_residual(x, w, b, residual=r, is_rms=False, eps=1e-6,
                                                  prenorm=True, residual_in_fp32=True)
    torch.testing.assert_close(y, rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(res_out, rec["outputs"]["residual_out"], rtol=1e-5, atol=1e-6)
    y.sum().backward()
    for name, t in (("x", x), ("w", w), ("b", b), ("residual", r)):
        torch.testing.assert_close(t.grad, rec["gradients"][name], rtol=1e-3, atol=2e-5)


def test_norm_upstream_rms():
    rec = fx.upstream("layer_norms", "rms_norm")
    i = rec["inputs"]
    x = i["x"].clone().requires_grad_(True); w = i["w"].clone().requires_grad_(True)
    y = O.fused_layer_norm(x, w, None, is_rms=True, eps=1e-6, prenorm=False, residual_in_fp32=False)
    torch.testing.assert_close(y, rec["outputs"]["y"], rtol=1e-4, atol=1e-5)
    y.sum().backward()
    torch.testing.assert_close(x.grad, rec["gradients"]["x"], rtol=1e-3, atol=2e-5)
    torch.testing.assert_close(w.grad, rec["gradients"]["w"], rtol=1e-3, atol=2e-5)


@pytest.mark.parametrize("prenorm", [True, False])
@pytest.mark.parametrize("rms", [True, False])
def test_norm_equals_library(prenorm, rms):
    x = torch.randn(2, 5, 16); r = torch.randn(2, 5, 16); w = torch.randn(16); b = torch.randn(16)
    y = O.fused_layer_norm(x, w, b, residual=r, is_rms=rms, eps=1e-5, prenorm=prenorm)
    v = x + r if prenorm else x
    if rms:
        want = F.rms_norm(v, (16,), weight=w, eps=1e-5) + b
    else:
        want = F.layer_norm(v, (16,), weight=w, bias=b, eps=1e-5)
    if not prenorm:
        want = want + r
    torch.testing.assert_close(y, want, rtol=1e-5, atol=1e-5)


# -------------------------------------------------------------------- true SSD

def test_ssd_cumsum_fixtures():
    rec = fx.upstream("ssd_components", "chunk_cumsum"); i = rec["inputs"]
    dA, dt_c = S.chunk_cumsum(i["dt"], i["A"], 3, dt_bias=i["dt_bias"], dt_softplus=True)
    torch.testing.assert_close(dA.float(), rec["outputs"]["dA_cumsum"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dt_c.float(), rec["outputs"]["dt_out"], rtol=1e-5, atol=1e-6)
    rec = fx.upstream("ssd_components", "chunk_cumsum_clamped"); i = rec["inputs"]
    dA, dt_c = S.chunk_cumsum(i["dt"], i["A"], 3, dt_limit=(0.01, 1.0))
    torch.testing.assert_close(dA.float(), rec["outputs"]["dA_cumsum"], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(dt_c.float(), rec["outputs"]["dt_out"], rtol=1e-5, atol=1e-6)


TF32 = dict(rtol=2e-2, atol=2e-2)     # the vectors were produced with TF32 dot products


def test_ssd_chunk_state_fixture():
    rec = fx.upstream("ssd_components", "chunk_state"); i = rec["inputs"]
    st = S.chunk_state(i["B"], i["x"], i["dt"], i["dA_cumsum"], clamp_decay=True)
    torch.testing.assert_close(st.float(), rec["outputs"]["states"], **TF32)


def test_ssd_state_passing_fixture():
    rec = fx.upstream("ssd_components", "state_passing"); i = rec["inputs"]
    entering, final = S.state_passing(i["states"], i["dA_last"])
    torch.testing.assert_close(entering.float(), rec["outputs"]["states_passed"], rtol=1e-5, atol=1e-6)
    b, nc, h, p, n = i["states"].shape
    torch.testing.assert_close(final.float().reshape(b, h, p * n), rec["outputs"]["final_states"],
                               rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("case", ["chunk_scan_matrix_D_z", "chunk_scan_vector_D"])
def test_ssd_chunk_scan_fixtures(case):
    rec = fx.upstream("ssd_components", case); i = rec["inputs"]
    y = S.chunk_scan(i["B"], i["C"], i["x"], i["dt"], i["dA_cumsum"], i["states"],
                     D=i["D"], z=i.get("z"), clamp_decay=True)
    torch.testing.assert_close(y.float(), rec["outputs"]["y"], **TF32)


def test_ssd_bmm_fixtures():
    rec = fx.upstream("ssd_bmm", "basic"); i = rec["inputs"]
    torch.testing.assert_close(S.bmm_chunk(i["a"], i["b"], 3).float(), rec["outputs"]["out"], **TF32)
    rec = fx.upstream("ssd_bmm", "grouped"); i = rec["inputs"]
    torch.testing.assert_close(S.bmm_chunk(i["a"], i["b"], 3).float(), rec["outputs"]["out"], **TF32)
    rec = fx.upstream("ssd_bmm", "causal_seq"); i = rec["inputs"]
    got = S.bmm_chunk(i["a"], i["b"], 3, seq_idx=i["seq_idx"], causal=True).float()
    tri = torch.tril(torch.ones(3, 3, dtype=torch.bool))
    torch.testing.assert_close(got[..., tri], rec["outputs"]["out"][..., tri], **TF32)


def test_ssd_combined_fixture_and_grads():
    rec = fx.upstream("ssd_combined", "combined_full"); i = rec["inputs"]
    names = ["X", "dt", "A", "B", "C", "D", "z", "dt_bias", "initial_states"]
    leaves = {k: i[k].double().clone().requires_grad_(True) for k in names}
    y, fin = S.ssd_combined(leaves["X"], leaves["dt"], leaves["A"], leaves["B"], leaves["C"],
                            int(i["chunk_size"]), D=leaves["D"], z=leaves["z"],
                            dt_bias=leaves["dt_bias"], initial_states=leaves["initial_states"],
                            dt_softplus=True, clamp_decay=True)
    torch.testing.assert_close(y.float(), rec["outputs"]["y"], **TF32)
    torch.testing.assert_close(fin.float(), rec["outputs"]["final_states"], **TF32)
    y.sum().backward()
    for k, g in rec["gradients"].items():
        if g is None:
            continue
        torch.testing.assert_close(leaves[k].grad.float(), g, rtol=5e-2, atol=5e-2)


def test_ssd_combined_varlen_fixture():
    """Packed row of two sequences (cu_seqlens 0, 3, 6; chunk 3): y is the plain result (the
    upstream call passes no seq_idx), the per-sequence end states do not mix."""
    rec = fx.upstream("ssd_combined", "combined_varlen"); i = rec["inputs"]
    A = fx.upstream("ssd_combined", "combined_full")["inputs"]["A"]
    y, _, vs = S.ssd_combined(i["X"], i["dt"], i["A"] if "A" in i else A, i["B"], i["C"], int(i["chunk_size"]),
                              clamp_decay=True, cu_seqlens=[0, 3, 6])
    torch.testing.assert_close(y.float(), rec["outputs"]["y"], **TF32)
    torch.testing.assert_close(vs.float(), rec["outputs"]["varlen_states"], **TF32)


@pytest.mark.parametrize("Q,lens", [(4, [5, 9, 1, 6]), (8, [3, 3, 10]), (3, [3, 3]), (16, [7, 2, 11])])
def test_ssd_packed_with_seq_idx_equals_separate_sequences(Q, lens):
    """A packed row with seq_idx (and cu_seqlens for the end states) gives, sequence by
    sequence, what the token-by-token recurrence gives on each sequence alone; the initial
    state goes to the first sequence (id 0) only."""
    g = torch.Generator().manual_seed(11)
    H, P, G, N = 4, 3, 2, 5
    L = sum(lens)
    x = torch.randn(1, L, H, P, generator=g, dtype=torch.float64)
    dt = torch.rand(1, L, H, generator=g, dtype=torch.float64)
    A = -torch.rand(H, generator=g, dtype=torch.float64) * 2
    Bm = torch.randn(1, L, G, N, generator=g, dtype=torch.float64)
    Cm = torch.randn(1, L, G, N, generator=g, dtype=torch.float64)
    D = torch.randn(H, P, generator=g, dtype=torch.float64)
    z = torch.randn(1, L, H, P, generator=g, dtype=torch.float64)
    init = torch.randn(1, H, P, N, generator=g, dtype=torch.float64)
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    seq_idx = torch.cat([torch.full((n,), k, dtype=torch.int32) for k, n in enumerate(lens)])[None]
    y, fin, vs = S.ssd_combined(x, dt, A, Bm, Cm, Q, D=D, z=z, initial_states=init, clamp_decay=False,
                                seq_idx=seq_idx, cu_seqlens=cu)
    for k in range(len(lens)):
        sl = slice(cu[k], cu[k + 1])
        yk, fk = S.ssd_sequential(x[:, sl], dt[:, sl], A, Bm[:, sl], Cm[:, sl], D=D, z=z[:, sl],
                                  initial_states=init if k == 0 else None)
        torch.testing.assert_close(y[:, sl], yk, rtol=1e-10, atol=1e-10)
        torch.testing.assert_close(vs[k], fk[0], rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(fin[0], vs[-1], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("Q", [1, 4, 8, 32])
def test_ssd_chunked_equals_sequential(Q):
    g = torch.Generator().manual_seed(5)
    Bsz, L, H, P, G, N = 2, 19, 4, 5, 2, 6
    x = torch.randn(Bsz, L, H, P, generator=g, dtype=torch.float64)
    dt = torch.rand(Bsz, L, H, generator=g, dtype=torch.float64)
    A = -torch.rand(H, generator=g, dtype=torch.float64) * 3
    Bm = torch.randn(Bsz, L, G, N, generator=g, dtype=torch.float64)
    Cm = torch.randn(Bsz, L, G, N, generator=g, dtype=torch.float64)
    D = torch.randn(H, generator=g, dtype=torch.float64)
    z = torch.randn(Bsz, L, H, P, generator=g, dtype=torch.float64)
    init = torch.randn(Bsz, H, P, N, generator=g, dtype=torch.float64)
    y0, f0 = S.ssd_sequential(x, dt, A, Bm, Cm, D=D, z=z, initial_states=init)
    y1, f1 = S.ssd_combined(x, dt, A, Bm, Cm, Q, D=D, z=z, initial_states=init, clamp_decay=False)
    torch.testing.assert_close(y1, y0, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(f1, f0, rtol=1e-10, atol=1e-10)


def test_ssd_reduces_to_diagonal_scan_when_N_is_1():
    g = torch.Generator().manual_seed(6)
    Bsz, L, H, P = 2, 9, 3, 4
    x = torch.randn(Bsz, L, H, P, generator=g, dtype=torch.float64)
    dt = torch.rand(Bsz, L, H, generator=g, dtype=torch.float64)
    A = -torch.rand(H, generator=g, dtype=torch.float64)
    Bm = torch.randn(Bsz, L, H, 1, generator=g, dtype=torch.float64)
    Cm = torch.randn(Bsz, L, H, 1, generator=g, dtype=torch.float64)
    y0, _ = S.ssd_sequential(x, dt, A, Bm, Cm)
    y1 = O.ssd_chunk_scan(x, dt, A, Bm.expand(Bsz, L, H, P), Cm.expand(Bsz, L, H, P), 4)
    torch.testing.assert_close(y1, y0, rtol=1e-10, atol=1e-12)

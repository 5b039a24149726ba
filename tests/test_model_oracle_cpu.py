"""The CPU oracle stacks (oracle/model_oracle.py), checked without a GPU: built on the pinned operator oracles,
their wiring is pinned by what the reference's module tests hold for its stacks -- the dense forward equals
token-by-token stepping on a cache (tests/modules/test_mamba1.py:44-60, test_mamba2.py:70-86 of the
reference) -- with the stepping side written from the single-step operator oracles and a rolling window,
by causality, and by a one-layer block against library routines (``F.conv1d``, ``F.rms_norm``)."""

import math

import torch
import torch.nn.functional as F

from oracle import model_oracle as M
from oracle import ops_oracle as O


def _mamba1_weights(seed, d=32, layers=2, N=8, K=4, vocab=50):
    g = torch.Generator().manual_seed(seed)
    di, R = 2 * d, 2
    rnd = lambda *s, std=0.2: torch.randn(*s, generator=g) * std
    ls = []
    for _ in range(layers):
        dt = torch.exp(torch.rand(di, generator=g) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
        ls.append(dict(norm_w=1 + rnd(d, std=0.1), in_proj_x=rnd(di, d), in_proj_z=rnd(di, d),
                       conv_w=torch.rand(di, K, generator=g) - 0.5, conv_b=rnd(di, std=0.02),
                       x_proj=rnd(R + 2 * N, di), dt_proj=rnd(di, R, std=R ** -0.5),
                       dt_bias=dt + torch.log(-torch.expm1(-dt)),
                       A=-torch.arange(1, N + 1, dtype=torch.float32).repeat(di, 1) * (1 + 0.1 * torch.rand(di, N, generator=g)),
                       D=1 + rnd(di, std=0.1), out_proj=rnd(d, di)))
    return dict(embedding=rnd(vocab, d, std=1.0), final_norm_w=1 + rnd(d, std=0.1), layers=ls), dict(d_state=N, dt_rank=R, eps=1e-5)


def _mamba2_weights(seed, d=32, layers=2, N=8, G=2, P=8, K=4, vocab=50):
    g = torch.Generator().manual_seed(seed)
    di = 2 * d
    H = di // P
    conv_dim = di + 2 * G * N
    rnd = lambda *s, std=0.2: torch.randn(*s, generator=g) * std
    ls = []
    for _ in range(layers):
        dt = torch.exp(torch.rand(H, generator=g) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
        ls.append(dict(norm_w=1 + rnd(d, std=0.1), in_proj=rnd(di + conv_dim + H, d),
                       conv_w=torch.rand(conv_dim, K, generator=g) - 0.5, conv_b=rnd(conv_dim, std=0.02),
                       dt_bias=dt + torch.log(-torch.expm1(-dt)), A=-(torch.rand(H, generator=g) * 15 + 1),
                       D=1 + rnd(H, std=0.1), gate_norm_w=1 + rnd(di, std=0.1), out_proj=rnd(d, di)))
    return (dict(embedding=rnd(vocab, d, std=1.0), final_norm_w=1 + rnd(d, std=0.1), layers=ls),
            dict(d_inner=di, nheads=H, headdim=P, d_state=N, ngroups=G, eps=1e-5))


def test_oracle_stacks_are_causal():
    for make, fwd in ((_mamba1_weights, M.mamba1_forward), (_mamba2_weights, M.mamba2_forward)):
        w, kw = make(0)
        tok = torch.randint(0, 50, (2, 12), generator=torch.Generator().manual_seed(1))
        full = fwd(w, tok, acc=torch.float64, **kw)
        tok2 = tok.clone()
        tok2[:, 7:] = (tok2[:, 7:] + 3) % 50
        other = fwd(w, tok2, acc=torch.float64, **kw)
        torch.testing.assert_close(full[:, :7], other[:, :7], rtol=0, atol=0)
        assert (full[:, 7:] - other[:, 7:]).abs().max() > 1e-3
        torch.testing.assert_close(fwd(w, tok[:, :5], acc=torch.float64, **kw), full[:, :5], rtol=1e-12, atol=1e-12)


def test_mamba1_oracle_stack_equals_stepping_on_a_cache():
    """Dense forward == one token at a time with a rolling conv window and ``selective_state_step``."""
    w, kw = _mamba1_weights(2)
    N, R, eps = kw["d_state"], kw["dt_rank"], kw["eps"]
    tok = torch.randint(0, 50, (2, 9), generator=torch.Generator().manual_seed(3))
    dense = M.mamba1_forward(w, tok, acc=torch.float64, **kw)
    f64 = lambda t: t.double()
    Bsz, K = 2, 4
    di = w["layers"][0]["in_proj_x"].shape[0]
    windows = [torch.zeros(Bsz, di, K, dtype=torch.float64) for _ in w["layers"]]
    states = [torch.zeros(Bsz, di, N, dtype=torch.float64) for _ in w["layers"]]
    for t in range(tok.shape[1]):
        hidden, residual = f64(w["embedding"])[tok[:, t]], None
        for lw, win, st in zip(w["layers"], windows, states):
            residual = hidden if residual is None else hidden + residual
            h = F.rms_norm(residual, (residual.shape[-1],), f64(lw["norm_w"]), eps)
            x, z = h @ f64(lw["in_proj_x"]).t(), h @ f64(lw["in_proj_z"]).t()
            win.copy_(torch.cat([win[:, :, 1:], x[:, :, None]], dim=2))
            u = F.silu((win * f64(lw["conv_w"])[None]).sum(-1) + f64(lw["conv_b"]))
            low = u @ f64(lw["x_proj"]).t()
            dt = low[:, :R] @ f64(lw["dt_proj"]).t()
            y = O.selective_state_step(st, u, dt, f64(lw["A"]), low[:, R:R + N].unsqueeze(1), low[:, R + N:].unsqueeze(1),
                                       D=f64(lw["D"]), z=z, dt_bias=f64(lw["dt_bias"]), softplus=True)
            hidden = y @ f64(lw["out_proj"]).t()
        residual = hidden + residual
        logits = F.rms_norm(residual, (residual.shape[-1],), f64(w["final_norm_w"]), eps) @ f64(w["embedding"]).t()
        torch.testing.assert_close(logits, dense[:, t], rtol=1e-9, atol=1e-9)


def test_mamba2_oracle_stack_equals_stepping_on_a_cache():
    """Dense forward == one token at a time: rolling window over x|B|C, per-head state h (P x N) updated as
    h <- exp(dt A) h + dt x (outer) B, y = h C + D x, gate, gated norm."""
    w, kw = _mamba2_weights(4)
    di, H, P, N, G, eps = kw["d_inner"], kw["nheads"], kw["headdim"], kw["d_state"], kw["ngroups"], kw["eps"]
    conv_dim = di + 2 * G * N
    tok = torch.randint(0, 50, (2, 10), generator=torch.Generator().manual_seed(5))
    dense = M.mamba2_forward(w, tok, acc=torch.float64, **kw)
    f64 = lambda t: t.double()
    windows = [torch.zeros(2, conv_dim, 4, dtype=torch.float64) for _ in w["layers"]]
    states = [torch.zeros(2, H, P, N, dtype=torch.float64) for _ in w["layers"]]
    for t in range(tok.shape[1]):
        hidden, residual = f64(w["embedding"])[tok[:, t]], None
        for li, lw in enumerate(w["layers"]):
            residual = hidden if residual is None else hidden + residual
            h = F.rms_norm(residual, (residual.shape[-1],), f64(lw["norm_w"]), eps)
            z, xBC, dt = torch.split(h @ f64(lw["in_proj"]).t(), [di, conv_dim, H], dim=-1)
            windows[li] = torch.cat([windows[li][:, :, 1:], xBC[:, :, None]], dim=2)
            xBC = F.silu((windows[li] * f64(lw["conv_w"])[None]).sum(-1) + f64(lw["conv_b"]))
            x, Bm, Cm = torch.split(xBC, [di, G * N, G * N], dim=-1)
            x = x.reshape(2, H, P)
            Bh = Bm.reshape(2, G, N).repeat_interleave(H // G, dim=1)
            Ch = Cm.reshape(2, G, N).repeat_interleave(H // G, dim=1)
            step = F.softplus(dt + f64(lw["dt_bias"]))
            decay = torch.exp(step * f64(lw["A"]))
            states[li] = decay[:, :, None, None] * states[li] + (step[:, :, None] * x)[..., None] * Bh[:, :, None, :]
            y = (states[li] * Ch[:, :, None, :]).sum(-1) + f64(lw["D"])[None, :, None] * x
            y = (y * F.silu(z.reshape(2, H, P))).reshape(2, di)
            hidden = F.rms_norm(y, (di,), f64(lw["gate_norm_w"]), eps) @ f64(lw["out_proj"]).t()
        residual = hidden + residual
        logits = F.rms_norm(residual, (residual.shape[-1],), f64(w["final_norm_w"]), eps) @ f64(w["embedding"]).t()
        torch.testing.assert_close(logits, dense[:, t], rtol=1e-9, atol=1e-9)


def test_one_layer_mamba1_block_against_library_routines():
    """One layer, one sequence: conv through ``F.conv1d`` on a padded input, norms through ``F.rms_norm``, the scan as
    an explicit loop over time in float64."""
    w, kw = _mamba1_weights(6, layers=1)
    N, R, eps = kw["d_state"], kw["dt_rank"], kw["eps"]
    tok = torch.randint(0, 50, (1, 11), generator=torch.Generator().manual_seed(7))
    dense = M.mamba1_forward(w, tok, acc=torch.float64, **kw)
    lw = {k: v.double() for k, v in w["layers"][0].items()}
    emb = w["embedding"].double()
    res = emb[tok]
    h = F.rms_norm(res, (res.shape[-1],), lw["norm_w"], eps)
    x = (h @ lw["in_proj_x"].t()).transpose(1, 2)
    z = (h @ lw["in_proj_z"].t()).transpose(1, 2)
    u = F.silu(F.conv1d(F.pad(x, (3, 0)), lw["conv_w"][:, None], lw["conv_b"], groups=x.shape[1]))
    low = torch.einsum("rd,bdl->brl", lw["x_proj"], u)
    delta = F.softplus(torch.einsum("dr,brl->bdl", lw["dt_proj"], low[:, :R]) + lw["dt_bias"][None, :, None])
    state = torch.zeros(1, x.shape[1], N, dtype=torch.float64)
    ys = []
    for t in range(tok.shape[1]):
        state = torch.exp(delta[:, :, t, None] * lw["A"][None]) * state \
            + (delta[:, :, t] * u[:, :, t])[..., None] * low[:, None, R:R + N, t]
        ys.append((state * low[:, None, R + N:, t]).sum(-1) + lw["D"] * u[:, :, t])
    y = torch.stack(ys, dim=-1) * F.silu(z)
    out = y.transpose(1, 2) @ lw["out_proj"].t() + res
    logits = F.rms_norm(out, (out.shape[-1],), w["final_norm_w"].double(), eps) @ emb.t()
    torch.testing.assert_close(logits, dense, rtol=1e-9, atol=1e-9)

"""CPU oracle for the two language-model stacks of ``ssm_amd.harness``.

TEST INFRASTRUCTURE ONLY: nothing under ``ssm_amd/`` may import this module.

The stacks are rebuilt here from the operator oracles (``ops_oracle``, ``ssd_oracle``) and plain
``torch`` matrix products on the CPU, in one accumulation dtype throughout (float32 by default, no
rounding to 16 bits between operators), from *explicit weight tensors*: the caller hands over the
very tensors the GPU stack holds, so the comparison does not depend on reproducing a random
initialisation.  What the structure follows:

* stack (embedding, pre-norm residual blocks with the residual stream kept apart from the
  normalised activations, final norm, tied output projection):
  /root/reference/src/ssm/models/lm.py:308-392 and :416-420; block order add -> norm -> mixer:
  /root/reference/src/ssm/modules/block.py:109-131;
* Mamba-1 mixer (in_proj -> causal conv + SiLU -> x_proj -> dt_proj -> selective scan with gate ->
  out_proj): /root/reference/src/ssm/modules/mamba1.py:176-260;
* Mamba-2 mixer in its published form (one projection to z | xBC | dt, conv over x|B|C, per-head
  scalar decay, gated RMSNorm before the output projection): the reference's module
  (/root/reference/src/ssm/modules/mamba2.py:20-140) is a simplified block around its diagonal scan;
  the configuration under test (d_state = 128, one B/C group) is the state-space-duality block whose
  operator semantics ``ssd_oracle`` restates from the shipped vectors.

The property the reference's own module tests hold for its stacks -- a cached single-token step
reproduces the dense forward (/root/reference/tests/modules/test_mamba1.py:44-60,
tests/modules/test_mamba2.py:70-86) -- is what these functions serve as the dense side of: the
logits of position t of one forward over the whole sequence are what prefill + cached steps must give.
"""

from __future__ import annotations

from typing import Dict, List

import torch

from . import ops_oracle as O
from . import ssd_oracle as S


def _rms(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return v * torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps) * w.to(v.dtype)


def mamba2_forward(weights: Dict, tokens: torch.Tensor, *, d_inner: int, nheads: int, headdim: int, d_state: int,
                   ngroups: int, eps: float, acc=torch.float32) -> torch.Tensor:
    """``tokens (B, L)`` -> logits ``(B, L, vocab)`` in ``acc``.

    ``weights``: ``embedding (V, d)``, ``final_norm_w (d,)`` and ``layers``: a list of dicts with
    ``norm_w (d,)``, ``in_proj (d_inner + conv_dim + H, d)``, ``conv_w (conv_dim, K)``, ``conv_b (conv_dim,)``,
    ``dt_bias (H,)``, ``A (H,)``, ``D (H,)``, ``gate_norm_w (d_inner,)``, ``out_proj (d, d_inner)``."""
    emb = weights["embedding"].to(acc)
    hidden = emb[tokens]
    residual = None
    Bsz, L = tokens.shape
    G, N, H, P = ngroups, d_state, nheads, headdim
    conv_dim = d_inner + 2 * G * N
    for lw in weights["layers"]:
        residual = hidden if residual is None else hidden + residual
        h = _rms(residual, lw["norm_w"], eps)
        zxbcdt = h @ lw["in_proj"].to(acc).t()
        z, xBC, dt = torch.split(zxbcdt, [d_inner, conv_dim, H], dim=-1)
        xBC = O.dw_causal_conv(xBC.contiguous(), lw["conv_w"].to(acc), lw["conv_b"].to(acc), activation="silu", acc=acc)
        x, Bm, Cm = torch.split(xBC, [d_inner, G * N, G * N], dim=-1)
        y, _ = S.ssd_sequential(x.reshape(Bsz, L, H, P), dt, lw["A"], Bm.reshape(Bsz, L, G, N),
                                Cm.reshape(Bsz, L, G, N), D=lw["D"], z=z.reshape(Bsz, L, H, P),
                                dt_bias=lw["dt_bias"], dt_softplus=True, acc=acc)
        y = _rms(y.reshape(Bsz, L, d_inner), lw["gate_norm_w"], eps)
        hidden = y @ lw["out_proj"].to(acc).t()
    residual = hidden + residual
    return _rms(residual, weights["final_norm_w"], eps) @ emb.t()


def mamba1_forward(weights: Dict, tokens: torch.Tensor, *, d_state: int, dt_rank: int, eps: float,
                   acc=torch.float32) -> torch.Tensor:
    """``tokens (B, L)`` -> logits ``(B, L, vocab)`` in ``acc``.

    ``layers`` entries: ``norm_w (d,)``, ``in_proj_x``, ``in_proj_z (d_inner, d)``, ``conv_w (d_inner, K)``,
    ``conv_b (d_inner,)``, ``x_proj (R + 2N, d_inner)``, ``dt_proj (d_inner, R)``, ``dt_bias (d_inner,)``,
    ``A (d_inner, N)``, ``D (d_inner,)``, ``out_proj (d, d_inner)``."""
    emb = weights["embedding"].to(acc)
    hidden = emb[tokens]
    residual = None
    N, R = d_state, dt_rank
    for lw in weights["layers"]:
        residual = hidden if residual is None else hidden + residual
        h = _rms(residual, lw["norm_w"], eps)
        ht = h.transpose(1, 2)                                               # (B, d, L)
        x = torch.matmul(lw["in_proj_x"].to(acc), ht)                        # (B, d_inner, L)
        z = torch.matmul(lw["in_proj_z"].to(acc), ht)
        u = O.dw_causal_conv(x, lw["conv_w"].to(acc), lw["conv_b"].to(acc), activation="silu", acc=acc)
        low = torch.matmul(lw["x_proj"].to(acc), u)                          # (B, R + 2N, L)
        delta = torch.matmul(lw["dt_proj"].to(acc), low[:, :R])
        Bm = low[:, R:R + N].unsqueeze(1)                                    # (B, 1, N, L)
        Cm = low[:, R + N:].unsqueeze(1)
        y = O.selective_scan(u, delta, lw["A"], Bm, Cm, D=lw["D"], z=z, dt_bias=lw["dt_bias"], softplus=True,
                             acc=acc)
        hidden = torch.matmul(y.to(acc).transpose(1, 2), lw["out_proj"].to(acc).t())
    residual = hidden + residual
    return _rms(residual, weights["final_norm_w"], eps) @ emb.t()


def weights_to_cpu(model, names: List[str]) -> Dict:
    """The tensors a GPU stack of ``ssm_amd.harness`` holds, copied to the CPU as they are (same values,
    same dtypes): ``names`` lists the per-layer attributes."""
    return {
        "embedding": model.embedding.detach().cpu(),
        "final_norm_w": model.final_norm_w.detach().cpu(),
        "layers": [{n: getattr(layer, n).detach().cpu() for n in names} for layer in model.layers],
    }


MAMBA2_LAYER_TENSORS = ["norm_w", "in_proj", "conv_w", "conv_b", "dt_bias", "A", "D", "gate_norm_w", "out_proj"]
MAMBA1_LAYER_TENSORS = ["norm_w", "in_proj_x", "in_proj_z", "conv_w", "conv_b", "x_proj", "dt_proj", "dt_bias", "A",
                        "D", "out_proj"]

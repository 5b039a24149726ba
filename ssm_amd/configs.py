"""Synthetic inputs of the benchmark configurations.

Values are drawn on the CPU from a seeded generator (so a CPU checker and the
GPU see identical bits) with the distributions the benchmark definition
prescribes:

* ``u, delta_raw, z ~ N(0, 1)``
* ``A[d, n] = -(n + 1)``
* ``B, C ~ N(0, 1)``, one group, time-varying ``(B, 1, N, L)``
* ``D = 1``
* ``dt_bias = softplus^-1(dt)`` with ``dt`` log-uniform in ``[1e-3, 0.1]``
"""

from __future__ import annotations

import math

import torch


def inverse_softplus_dt(n: int, gen: torch.Generator, lo: float = 1e-3, hi: float = 0.1) -> torch.Tensor:
    dt = torch.exp(torch.rand(n, generator=gen) * (math.log(hi) - math.log(lo)) + math.log(lo))
    return dt + torch.log(-torch.expm1(-dt))


def scan_inputs(batch: int, dim: int, length: int, nstate: int, dtype=torch.float32, seed: int = 0,
                groups: int = 1) -> dict:
    """Inputs of ``selective_scan`` for configs 0 and 1 (CPU tensors)."""
    g = torch.Generator().manual_seed(seed)
    return dict(
        u=torch.randn(batch, dim, length, generator=g).to(dtype),
        delta=torch.randn(batch, dim, length, generator=g).to(dtype),
        z=torch.randn(batch, dim, length, generator=g).to(dtype),
        A=-torch.arange(1, nstate + 1, dtype=torch.float32).repeat(dim, 1).contiguous(),
        B=torch.randn(batch, groups, nstate, length, generator=g).to(dtype),
        C=torch.randn(batch, groups, nstate, length, generator=g).to(dtype),
        D=torch.ones(dim),
        dt_bias=inverse_softplus_dt(dim, g),
    )


def scan_fwd_bytes(batch: int, dim: int, length: int, nstate: int, elt: int, groups: int = 1) -> int:
    """Compulsory traffic of one forward scan: u, delta, z read and y written
    once, B and C read once, A/D/bias read once, last_state written once."""
    return (4 * elt * batch * dim * length + 2 * elt * batch * groups * nstate * length
            + 4 * dim * (nstate + 2) + elt * batch * dim * nstate)


def to_device(d: dict, device="cuda") -> dict:
    return {k: (v.to(device) if isinstance(v, torch.Tensor) else v) for k, v in d.items()}

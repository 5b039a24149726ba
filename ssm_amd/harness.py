"""Language-model stacks built on the operators of this package (Mamba-2 and Mamba-1 blocks): the
measurement harness for whole-model prefill and greedy decoding.

It is not a port of the reference's modules.  The reference's ``Mamba2`` block
(/root/reference/src/ssm/modules/mamba2.py:20-140) is a simplified block around
its diagonal ``ssd_chunk_scan``; this harness is the state-space-duality block the
benchmark configuration describes (``d_state = 128``, one B/C group, gated
RMSNorm before the output projection), as published with Mamba-2:

    residual, h = add + RMSNorm                        fused_layer_norm_with_residual
    z | xBC | dt = in_proj(h)                          GEMMs (torch), one per part of the row
    xBC = silu(conv1d(xBC))                            dw_causal_conv_channels_last, x and B|C apart
    y = SSD(x, dt, A, B, C, D, gate z)                 ssm_amd.ops.ssd.ssd_combined
    out = out_proj(RMSNorm(y))                         fused_layer_norm, GEMM (torch)

and, per generated token, the same block on cached states:

    conv window roll + taps + silu ;                   mamba2_decode_step (both in place, reads the row of the
    h <- exp(dt A) h + dt x (x) B ;  y = h C + D x     input projection as it is)

``Mamba1LM`` is the same harness around the selective scan (``d_state = 16``, input-dependent
``dt``, ``B``, ``C`` from the convolution's output, as published with Mamba), whose mixer at 130M size has
exactly the shape of the scan benchmark (1536 channels, 16 states, 4 taps):

    x | z = in_proj(h)  (channels first)               GEMM (torch)
    u = silu(conv1d(x))                                dw_causal_conv (channels first)
    dt_low | B | C = x_proj(u);  delta = dt_proj(dt_low)   GEMMs (torch)
    y = scan(u, delta, A, B, C, D, gate z)             selective_scan(return_last_state=True)
    out = out_proj(y)                                  GEMM (torch)

and per generated token ``conv_window_step`` on the cached window, the two small projections and
``selective_state_step`` on the state the prefill's scan handed over (the reference prefills its cache
token by token, /root/reference/src/ssm/modules/mamba1.py:306-322).

Weights are random (N(0, 0.02), tied embeddings) as the benchmark prescribes.
What pins it: every operator has its own parity tests; the stack itself is
checked for self-consistency (prefill + cached decoding reproduces the logits of
one full forward).  Parity with a particular trained checkpoint or with the
reference's simplified block is not claimed.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional, Tuple

import torch

from . import ops
from .ops import ssd as ssd_ops


@dataclass
class Mamba2Config:
    d_model: int = 768
    n_layer: int = 24
    expand: int = 2
    headdim: int = 64
    d_state: int = 128
    ngroups: int = 1
    d_conv: int = 4
    chunk_size: int = 256
    vocab_size: int = 50280
    eps: float = 1e-5
    dtype: torch.dtype = torch.bfloat16

    @property
    def d_inner(self) -> int:
        return self.expand * self.d_model

    @property
    def nheads(self) -> int:
        return self.d_inner // self.headdim

    @property
    def conv_dim(self) -> int:
        return self.d_inner + 2 * self.ngroups * self.d_state


class _Layer:
    def __init__(self, cfg: Mamba2Config, gen: torch.Generator, device):
        d, di, H = cfg.d_model, cfg.d_inner, cfg.nheads
        proj = di + cfg.conv_dim + H

        def rnd(*shape, std=0.02):
            return (torch.randn(*shape, generator=gen) * std).to(cfg.dtype).to(device)

        self.norm_w = torch.ones(d, dtype=torch.float32, device=device)
        self.in_proj = rnd(proj, d)
        self.conv_w = (torch.rand(cfg.conv_dim, cfg.d_conv, generator=gen) - 0.5).to(cfg.dtype).to(device)
        self.conv_b = rnd(cfg.conv_dim)
        dt = torch.exp(torch.rand(H, generator=gen) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
        self.dt_bias = (dt + torch.log(-torch.expm1(-dt))).float().to(device)      # inverse softplus
        self.A = (-(torch.rand(H, generator=gen) * 15.0 + 1.0)).float().to(device)
        self.D = torch.ones(H, dtype=torch.float32, device=device)
        self.gate_norm_w = torch.ones(di, dtype=torch.float32, device=device)
        self.out_proj = rnd(d, di)
        # float32 copies of the convolution parameters for the single-token step
        self.conv_w_f32 = self.conv_w.float().contiguous()
        self.conv_b_f32 = self.conv_b.float().contiguous()
        # The rows of the input projection by what they produce (views, no copies): over a whole sequence each
        # part is projected on its own, so that z, the conv inputs and dt come out as dense tensors the kernels
        # take as they are -- slicing one projected row of 2 d_inner + 2 G N + H columns would cost a strided
        # copy of z, x|B|C and x again per layer (0.67 GB at 16 x 2048 tokens).
        gn2 = cfg.conv_dim - di
        self.in_proj_z, self.in_proj_x, self.in_proj_bc, self.in_proj_dt = torch.split(self.in_proj, [di, di, gn2, H], dim=0)
        # taps and bias as the kernels take them (float32, the same values): cut once, not converted on every call
        self.conv_w_x, self.conv_w_bc = (t.contiguous() for t in torch.split(self.conv_w_f32, [di, gn2], dim=0))
        self.conv_b_x, self.conv_b_bc = (t.contiguous() for t in torch.split(self.conv_b_f32, [di, gn2], dim=0))


@dataclass
class DecodeCache:
    conv: List[torch.Tensor]       # per layer (B, conv_dim, K): the last K inputs of the convolution, oldest first
    ssm: List[torch.Tensor]        # per layer (B, H, P, N) float32
    residual: Optional[torch.Tensor] = None


class _GreedyDecoding:
    """Prefill, then single-token steps on cached states; shared by both stacks, which supply
    ``forward(tokens, return_cache, last_only)`` and ``step(tokens, cache)``."""

    @torch.no_grad()
    def generate(self, tokens: torch.Tensor, new_tokens: int, use_graph: bool = True) -> Tuple[torch.Tensor, dict]:
        """Greedy decoding: prefill on ``tokens (B, L)``, then ``new_tokens`` single-token steps on
        cached states.  With ``use_graph`` the step is captured once as a HIP graph and replayed.
        Returns ``(generated (B, new_tokens), timings in seconds)``."""
        start, mid, end = (torch.cuda.Event(enable_timing=True) for _ in range(3))
        start.record()
        logits, cache = self.forward(tokens, return_cache=True, last_only=True)
        nxt = logits[:, -1].float().argmax(-1)
        mid.record()
        out = [nxt]
        if use_graph and new_tokens > 1:
            static_tok = nxt.clone()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):                              # warm-up outside capture, on a scratch cache
                scratch = DecodeCache([c.clone() for c in cache.conv], [s.clone() for s in cache.ssm])
                self.step(static_tok, scratch)
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_next = self.step(static_tok, cache).float().argmax(-1)
            # the capture run did not execute: the cache is still the prefill's
            for _ in range(new_tokens - 1):
                graph.replay()
                static_tok.copy_(static_next)
                out.append(static_next.clone())
        else:
            for _ in range(new_tokens - 1):
                nxt = self.step(nxt, cache).float().argmax(-1)
                out.append(nxt)
        end.record()
        torch.cuda.synchronize()
        return torch.stack(out, dim=1), {"prefill_s": start.elapsed_time(mid) * 1e-3,
                                          "decode_s": mid.elapsed_time(end) * 1e-3}


class Mamba2LM(_GreedyDecoding):
    """Embedding -> n_layer blocks -> final norm -> tied output projection."""

    def __init__(self, cfg: Mamba2Config, device="cuda", seed: int = 0):
        self.cfg = cfg
        self.device = torch.device(device)
        gen = torch.Generator().manual_seed(seed)
        self.embedding = (torch.randn(cfg.vocab_size, cfg.d_model, generator=gen) * 0.02).to(cfg.dtype).to(self.device)
        self.layers = [_Layer(cfg, gen, self.device) for _ in range(cfg.n_layer)]
        self.final_norm_w = torch.ones(cfg.d_model, dtype=torch.float32, device=self.device)

    # ------------------------------------------------------------------ full sequence
    def _mixer(self, layer: _Layer, h: torch.Tensor, want_state: bool):
        cfg = self.cfg
        Bsz, L, _ = h.shape
        di, H, P, G, N = cfg.d_inner, cfg.nheads, cfg.headdim, cfg.ngroups, cfg.d_state
        z = h @ layer.in_proj_z.t()
        x_in = h @ layer.in_proj_x.t()
        bc_in = h @ layer.in_proj_bc.t()
        dt = h @ layer.in_proj_dt.t()
        # (B, L, C) channels last; the taps are per channel, so x and B|C convolve separately
        x = ops.dw_causal_conv_channels_last(x_in, layer.conv_w_x, layer.conv_b_x, activation="silu")
        bc = ops.dw_causal_conv_channels_last(bc_in, layer.conv_w_bc, layer.conv_b_bc, activation="silu")
        Bm, Cm = torch.split(bc, [G * N, G * N], dim=-1)
        out = ssd_ops.ssd_combined(x.reshape(Bsz, L, H, P), dt, layer.A, Bm.reshape(Bsz, L, G, N),
                                   Cm.reshape(Bsz, L, G, N), cfg.chunk_size, D=layer.D,
                                   z=z.reshape(Bsz, L, H, P), dt_bias=layer.dt_bias, dt_softplus=True,
                                   return_final_states=want_state)
        y, final = out if want_state else (out, None)
        y = ops.fused_layer_norm(y.reshape(Bsz, L, di), layer.gate_norm_w, None, is_rms=True, eps=cfg.eps)
        res = y @ layer.out_proj.t()
        if not want_state:
            return res, None, None
        K = cfg.d_conv
        window = torch.cat([x_in[:, -K:], bc_in[:, -K:]], dim=-1)              # the conv inputs of the last K tokens
        if L < K:
            window = torch.cat([torch.zeros(Bsz, K - L, cfg.conv_dim, dtype=window.dtype, device=h.device), window], dim=1)
        return res, window.transpose(1, 2).contiguous(), final.contiguous()

    def forward(self, tokens: torch.Tensor, return_cache: bool = False, last_only: bool = False):
        """tokens (B, L) -> logits (B, L, vocab) in the model dtype, or (B, 1, vocab) for the last
        position only (and the decoding cache)."""
        cfg = self.cfg
        hidden = self.embedding[tokens]
        residual = None
        conv, ssm = [], []
        for layer in self.layers:
            hidden, residual = ops.fused_layer_norm_with_residual(hidden, layer.norm_w, None, residual=residual,
                                                                  is_rms=True, eps=cfg.eps)
            hidden, cw, st = self._mixer(layer, hidden, return_cache)
            if return_cache:
                conv.append(cw)
                ssm.append(st)
        hidden, residual = ops.fused_layer_norm_with_residual(hidden, self.final_norm_w, None, residual=residual,
                                                              is_rms=True, eps=cfg.eps)
        logits = (hidden[:, -1:] if last_only else hidden) @ self.embedding.t()
        if return_cache:
            return logits, DecodeCache(conv, ssm)
        return logits

    # ------------------------------------------------------------------ one token
    def step(self, tokens: torch.Tensor, cache: DecodeCache) -> torch.Tensor:
        """tokens (B,) -> logits (B, vocab); the cache is updated in place."""
        cfg = self.cfg
        di, H, P, G, N, K = cfg.d_inner, cfg.nheads, cfg.headdim, cfg.ngroups, cfg.d_state, cfg.d_conv
        hidden = self.embedding[tokens][:, None]                      # (B, 1, d)
        Bsz = hidden.shape[0]
        residual = None
        for layer, cw, st in zip(self.layers, cache.conv, cache.ssm):
            hidden, residual = ops.fused_layer_norm_with_residual(hidden, layer.norm_w, None, residual=residual,
                                                                  is_rms=True, eps=cfg.eps)
            zxbcdt = hidden[:, 0] @ layer.in_proj.t()
            y = ops.mamba2_decode_step(zxbcdt, cw, st, layer.conv_w_f32, layer.conv_b_f32, layer.A, D=layer.D,
                                       dt_bias=layer.dt_bias, ngroups=G, softplus=True, gate=True)
            y = ops.fused_layer_norm(y[:, None], layer.gate_norm_w, None, is_rms=True, eps=cfg.eps)
            hidden = y @ layer.out_proj.t()
        hidden, residual = ops.fused_layer_norm_with_residual(hidden, self.final_norm_w, None, residual=residual,
                                                              is_rms=True, eps=cfg.eps)
        return hidden[:, 0] @ self.embedding.t()


# ---------------------------------------------------------------------------------------------
# Mamba-1: the selective scan as the mixer
# ---------------------------------------------------------------------------------------------

@dataclass
class Mamba1Config:
    d_model: int = 768
    n_layer: int = 24
    expand: int = 2
    d_state: int = 16
    d_conv: int = 4
    dt_rank: int = 0              # 0: ceil(d_model / 16)
    vocab_size: int = 50280
    eps: float = 1e-5
    dtype: torch.dtype = torch.bfloat16

    @property
    def d_inner(self) -> int:
        return self.expand * self.d_model

    @property
    def rank(self) -> int:
        return self.dt_rank or -(-self.d_model // 16)


class _Layer1:
    def __init__(self, cfg: Mamba1Config, gen: torch.Generator, device):
        d, di, N, R = cfg.d_model, cfg.d_inner, cfg.d_state, cfg.rank

        def rnd(*shape, std=0.02):
            return (torch.randn(*shape, generator=gen) * std).to(cfg.dtype).to(device)

        self.norm_w = torch.ones(d, dtype=torch.float32, device=device)
        self.in_proj_x, self.in_proj_z = rnd(di, d), rnd(di, d)
        self.in_proj_xz = torch.cat([self.in_proj_x, self.in_proj_z], dim=0)      # one GEMM per token when decoding
        self.conv_w = (torch.rand(di, cfg.d_conv, generator=gen) - 0.5).float().to(device)
        self.conv_b = (torch.randn(di, generator=gen) * 0.02).float().to(device)
        self.x_proj = rnd(R + 2 * N, di)
        self.dt_proj = rnd(di, R, std=R ** -0.5)
        dt = torch.exp(torch.rand(di, generator=gen) * (math.log(0.1) - math.log(1e-3)) + math.log(1e-3))
        self.dt_bias = (dt + torch.log(-torch.expm1(-dt))).float().to(device)      # inverse softplus
        self.A = (-torch.arange(1, N + 1, dtype=torch.float32).repeat(di, 1)).to(device)
        self.D = torch.ones(di, dtype=torch.float32, device=device)
        self.out_proj = rnd(d, di)


class Mamba1LM(_GreedyDecoding):
    """Embedding -> n_layer Mamba-1 blocks -> final norm -> tied output projection."""

    def __init__(self, cfg: Mamba1Config, device="cuda", seed: int = 0):
        self.cfg = cfg
        self.device = torch.device(device)
        gen = torch.Generator().manual_seed(seed)
        self.embedding = (torch.randn(cfg.vocab_size, cfg.d_model, generator=gen) * 0.02).to(cfg.dtype).to(self.device)
        self.layers = [_Layer1(cfg, gen, self.device) for _ in range(cfg.n_layer)]
        self.final_norm_w = torch.ones(cfg.d_model, dtype=torch.float32, device=self.device)

    def _mixer(self, layer: _Layer1, h: torch.Tensor, want_state: bool):
        cfg = self.cfg
        Bsz, L, _ = h.shape
        N, R, K = cfg.d_state, cfg.rank, cfg.d_conv
        ht = h.transpose(1, 2)                                        # (B, d, L) view: the GEMMs write channels first
        x = torch.matmul(layer.in_proj_x, ht)                         # (B, d_inner, L)
        z = torch.matmul(layer.in_proj_z, ht)
        u = ops.dw_causal_conv(x, layer.conv_w, layer.conv_b, activation="silu")
        low = torch.matmul(layer.x_proj, u)                           # (B, R + 2N, L)
        delta = torch.matmul(layer.dt_proj, low[:, :R])               # (B, d_inner, L)
        Bm = low[:, R:R + N].unsqueeze(1).contiguous()                # (B, 1, N, L): one group
        Cm = low[:, R + N:].unsqueeze(1).contiguous()
        out = ops.selective_scan(u, delta, layer.A, Bm, Cm, D=layer.D, z=z, dt_bias=layer.dt_bias, softplus=True,
                                 return_last_state=want_state)
        y, last = out if want_state else (out, None)
        res = torch.matmul(y.transpose(1, 2), layer.out_proj.t())     # (B, L, d)
        if not want_state:
            return res, None, None
        window = x[:, :, -K:] if L >= K else torch.cat(
            [torch.zeros(Bsz, cfg.d_inner, K - L, dtype=x.dtype, device=h.device), x], dim=2)
        return res, window.contiguous(), last.float().contiguous()

    def forward(self, tokens: torch.Tensor, return_cache: bool = False, last_only: bool = False):
        """tokens (B, L) -> logits (B, L, vocab), or (B, 1, vocab) for the last position only (and the
        decoding cache: per layer the convolution window (B, d_inner, K) and the state (B, d_inner, N))."""
        cfg = self.cfg
        hidden = self.embedding[tokens]
        residual = None
        conv, ssm = [], []
        for layer in self.layers:
            hidden, residual = ops.fused_layer_norm_with_residual(hidden, layer.norm_w, None, residual=residual,
                                                                  is_rms=True, eps=cfg.eps)
            hidden, cw, st = self._mixer(layer, hidden, return_cache)
            if return_cache:
                conv.append(cw)
                ssm.append(st)
        hidden, residual = ops.fused_layer_norm_with_residual(hidden, self.final_norm_w, None, residual=residual,
                                                              is_rms=True, eps=cfg.eps)
        logits = (hidden[:, -1:] if last_only else hidden) @ self.embedding.t()
        if return_cache:
            return logits, DecodeCache(conv, ssm)
        return logits

    def step(self, tokens: torch.Tensor, cache: DecodeCache) -> torch.Tensor:
        """tokens (B,) -> logits (B, vocab); the cache is updated in place."""
        cfg = self.cfg
        N, R = cfg.d_state, cfg.rank
        hidden = self.embedding[tokens][:, None]
        residual = None
        for layer, cw, st in zip(self.layers, cache.conv, cache.ssm):
            hidden, residual = ops.fused_layer_norm_with_residual(hidden, layer.norm_w, None, residual=residual,
                                                                  is_rms=True, eps=cfg.eps)
            hrow = hidden[:, 0]
            xz = hrow @ layer.in_proj_xz.t()                          # (B, 2 d_inner): x is read in place, z copied
            x, z = xz[:, :cfg.d_inner], xz[:, cfg.d_inner:]
            u = ops.conv_window_step(cw, x, layer.conv_w, layer.conv_b, activation="silu")
            low = u @ layer.x_proj.t()                                # (B, R + 2N)
            dt = low[:, :R] @ layer.dt_proj.t()
            y = ops.selective_state_step(st, u, dt, layer.A, low[:, R:R + N].unsqueeze(1), low[:, R + N:].unsqueeze(1),
                                         D=layer.D, z=z, dt_bias=layer.dt_bias, softplus=True)
            hidden = (y @ layer.out_proj.t())[:, None]
        hidden, residual = ops.fused_layer_norm_with_residual(hidden, self.final_norm_w, None, residual=residual,
                                                              is_rms=True, eps=cfg.eps)
        return hidden[:, 0] @ self.embedding.t()

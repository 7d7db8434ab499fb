"""Sequence mixers for layer-spec models: windowed attention with pooled blocks, the Mamba-2
state-space mixer, and the block that runs both side by side on one normed input.

Every mixer reads its slice of the layer's fused input projection ``u`` [T, *] (one GEMM per
layer produces the attention's q | k | v | gate, the state-space z | x | B | C | dt and the
feed-forward's up rows), works on a ragged step (``ops.seqmix.RaggedMeta``) and keeps what it
must remember in the engine's paged cache (``engine.paged.RunCache``: key / value pages and
pooled entries for attention, convolution tail and state matrix per slot for the state-space
side).  Scores, softmax, decays, state and norms are fp32 whatever the activation dtype.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from ..ops import seqmix
from .configs import SSDSpec, WindowAttnSpec
from .layers import Linear


_ROPE_TABLES: dict = {}
_ROPE_RETIRED: list = []


class WindowPoolAttention(nn.Module):
    """Grouped-query softmax attention whose query at position i sees the last ``window`` tokens
    and one mean key / value per block of ``pool`` tokens lying wholly before the window
    (b pool + pool - 1 <= i - window), all in one softmax; rotary positions (optionally
    YaRN-blended) on the first ``rot_dims`` coordinates; a per-head sigmoid gate on the output."""

    def __init__(self, spec: WindowAttnSpec, width: int, dtype, device):
        super().__init__()
        self.spec = spec
        self.o = Linear(spec.heads * spec.vdim, width, False, dtype, device)
        self._rope = None

    def rope(self, n: int, device) -> Optional[torch.Tensor]:
        """cos / sin rows for positions [0, n): one table per (rotation constants, device), shared by
        every layer that rotates alike, grown by doubling."""
        s = self.spec
        if not s.rot_dims:
            return None
        if self._rope is None or self._rope.shape[0] < n or self._rope.device != torch.device(device):
            key = (s.rot_dims, s.rot_base, tuple(sorted((s.rot_scaling or {}).items())), str(torch.device(device)))
            tab = _ROPE_TABLES.get(key)
            if tab is None or tab.shape[0] < n:
                from .. import ops
                rows = 2048
                while rows < n:
                    rows *= 2
                if tab is not None:
                    _ROPE_RETIRED.append(tab)           # a captured graph may still read the smaller table
                tab = _ROPE_TABLES[key] = ops.rope_tables(s.rot_dims, rows, s.rot_base, s.rot_scaling, device=device)
            self._rope = tab
        return self._rope

    def forward(self, u: torch.Tensor, c0: int, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        """``u`` columns [c0, ..) hold q | k | v | gate.  Returns the o-projection's output [T, W]."""
        s = self.spec
        nq, nk, nv, ng = s.proj_sizes
        proj = u[:, c0:c0 + nq + nk + nv]
        q = seqmix.rope_paged_write(proj, meta, self.rope(meta.max_keys, u.device), run.k, run.v, s.heads, s.rot_dims)
        if s.window is not None and s.pool:
            seqmix.pool_blocks(run.k, run.v, run.k_pool, run.v_pool, meta, s.pool)
        gate = u[:, c0 + nq + nk + nv:c0 + nq + nk + nv + ng] if ng else None
        a = seqmix.window_pool_attention(q, gate, run.k, run.v, run.k_pool, run.v_pool, meta, s.scale, s.window,
                                         s.pool if s.window is not None else None)
        return self.o(a)


class SSDMixer(nn.Module):
    """Mamba-2: causal depthwise convolution + silu over x | B | C, step sizes softplus(dt + bias),
    per head S <- exp(-exp(A_log) dt) S + dt B x^T and y = S^T C + D x carried token to token in
    fp32, then y * silu(z), an RMS norm in ``norm_groups`` parts and the output projection."""

    def __init__(self, spec: SSDSpec, width: int, eps: float, dtype, device):
        super().__init__()
        self.spec, self.eps = spec, eps
        C = spec.conv_channels
        P = lambda *shape, dt=torch.float32: nn.Parameter(torch.zeros(*shape, dtype=dt, device=device),
                                                          requires_grad=False)
        self.conv_w, self.conv_b = P(C, spec.conv), P(C)          # small recurrence constants stay fp32
        self.dt_bias, self.A_log, self.D = P(spec.heads), P(spec.heads), P(spec.heads)
        self.norm_w = P(spec.inner)
        self.o = Linear(spec.inner, width, False, dtype, device)

    def forward(self, u: torch.Tensor, c0: int, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        """``u`` columns [c0, ..) hold z | x | B | C | dt."""
        s = self.spec
        inner, C = s.inner, s.conv_channels
        xbc = seqmix.conv_silu(u, c0 + inner, C, self.conv_w, self.conv_b, run.conv, meta)
        y = seqmix.ssd_scan(xbc, u, c0 + inner + C, self.dt_bias, self.A_log, self.D, run.ssm, meta, s.heads, s.vdim,
                            s.state, s.groups)
        g = seqmix.gated_group_norm(y, u[:, c0:c0 + inner], self.norm_w, s.norm_groups, self.eps, u.dtype)
        return self.o(g)


class ParallelMixer(nn.Module):
    """Attention and state-space mixer side by side on the same input; the result is half the
    sum of the two outputs, each RMS-normed over the width with its own weight (the sum, the
    residual add and an optional third addend run in one kernel: ``seqmix.combine_residual``)."""

    def __init__(self, attn: WindowAttnSpec, ssd: SSDSpec, width: int, eps: float, dtype, device):
        super().__init__()
        self.eps = eps
        self.left = WindowPoolAttention(attn, width, dtype, device)
        self.right = SSDMixer(ssd, width, eps, dtype, device)
        self.left_out = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device), requires_grad=False)
        self.right_out = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device), requires_grad=False)

    @property
    def in_rows(self) -> int:
        return sum(self.left.spec.proj_sizes) + self.right.spec.in_size

    def forward(self, x: torch.Tensor, u: torch.Tensor, meta, run, extra: Optional[torch.Tensor] = None):
        """x fp32 [T, W] (residual stream, updated in place) += mixer(u) + extra."""
        a = self.left(u, 0, meta, run)
        r = self.right(u, sum(self.left.spec.proj_sizes), meta, run)
        return seqmix.combine_residual(x, a, r, self.left_out, self.right_out, self.eps, extra)

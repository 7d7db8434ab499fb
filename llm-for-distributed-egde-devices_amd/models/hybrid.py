"""Layer-spec language models (arch "nudadra"): every layer is described by its own entry of
``ModelConfig.layer_specs``, a span of layers may run several times in a row, and the residual
stream is fp32.

Per layer (parallel form):  h = norm(x) ;  x <- x + mixer(h) + ff(h), with one norm whose gain is a
single number, a ``ParallelMixer`` (models/mixers.py) and a squared-ReLU feed-forward.  The
layer's input projections (attention q | k | v | gate, state-space z | x | B | C | dt,
feed-forward up) are one fused GEMM over h.

Looped span: before each pass t of layers [start, stop) the stream becomes
W_in [x ; x0] + step[t] (x0 = the scaled embedding); every pass owns its cache and state, so the
cache is indexed by *run* (``ModelConfig.layer_runs``), not by layer.

The model runs ragged steps only (``forward(ids, meta, cache)``): the paged engine
(engine/ragged.py) drives prefill portions and decode tokens of several sequences through it
in one call.
"""
from __future__ import annotations

import zlib
from typing import Dict, Optional

import torch
import torch.nn as nn

from ..ops import seqmix
from .configs import LayerSpec, ModelConfig
from .layers import Linear, ScalarNorm
from .mixers import ParallelMixer


class HybridLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: LayerSpec, idx: int, dtype, device):
        super().__init__()
        assert spec.mixer == "parallel", spec.mixer
        W = cfg.hidden_size
        self.idx, self.spec = idx, spec
        self.norm1 = ScalarNorm(cfg.norm_eps, device)
        self.mix = ParallelMixer(spec.attn, spec.ssd, W, cfg.norm_eps, dtype, device)
        self.ff = spec.ff or 0
        # rows: attention q | k | v | gate, state-space z | x | B | C | dt, feed-forward up
        self.proj_in = Linear(W, self.mix.in_rows + self.ff, False, dtype, device)
        self.down = Linear(self.ff, W, False, dtype, device) if self.ff else None

    def forward(self, x: torch.Tensor, meta: seqmix.RaggedMeta, run) -> torch.Tensor:
        h = self.norm1(x, self.proj_in.weight.dtype)
        u = self.proj_in(h)
        m = self.down(seqmix.relu2(u, self.mix.in_rows, self.ff)) if self.ff else None
        return self.mix(x, u, meta, run, m)


class HybridLM(nn.Module):
    ragged = True          # runs RaggedMeta steps over a paged cache (engine.ragged)

    def __init__(self, cfg: ModelConfig, dtype=torch.bfloat16, device=None):
        super().__init__()
        assert cfg.layer_specs is not None
        self.cfg, self.dtype = cfg, dtype
        W = cfg.hidden_size
        self.first, self.last = 0, cfg.num_layers
        self.has_embed = self.has_head = True
        self.embed = nn.Parameter(torch.empty(cfg.vocab_size, W, dtype=dtype, device=device), requires_grad=False)
        self.layers = nn.ModuleList([HybridLayer(cfg, s, i, dtype, device) for i, s in enumerate(cfg.layer_specs)])
        self.runs = cfg.layer_runs()
        if cfg.loop is not None:
            self.loop_in = Linear(2 * W, W, False, dtype, device)
            self.loop_step = nn.Parameter(torch.zeros(cfg.loop.times, W, dtype=torch.float32, device=device),
                                          requires_grad=False)
        self.final_norm = ScalarNorm(cfg.norm_eps, device)
        self.lm_head = Linear(W, cfg.vocab_size, False, dtype, device)

    @property
    def device(self):
        return self.embed.device

    @torch.no_grad()
    def confidence(self, ids) -> float:
        """mean over the text's tokens of max softmax probability (eval.metrics.confidence_score):
        one ragged prompt pass through a cache of its own."""
        from .. import ops
        from ..engine.ragged import RaggedEngine
        eng = RaggedEngine(self, len(ids), slots=1, use_graphs=False)
        logits = eng.step([("c", list(ids), list(range(len(ids))))])
        return float(ops.max_softmax_prob(logits).mean())

    def run_specs(self):
        """The LayerSpec of every run, in order (sizes the paged cache)."""
        return [self.cfg.layer_specs[i] for i, _ in self.runs]

    def forward(self, ids: torch.Tensor, meta: seqmix.RaggedMeta, cache, rows: Optional[torch.Tensor] = None,
                taps: Optional[list] = None) -> torch.Tensor:
        """ids [T] (flat step) -> fp32 logits of ``rows`` (flat row indices; None: every row).
        ``taps`` (a list) receives the residual stream after every run."""
        cfg = self.cfg
        x0 = seqmix.embedding_scaled(ids, self.embed, cfg.embed_scale)
        x = x0.clone() if cfg.loop is not None else x0
        for r, (i, t) in enumerate(self.runs):
            if t is not None and i == cfg.loop.start:
                x = seqmix.linear_f32(seqmix.cat_cast(x, x0, self.dtype), self.loop_in.weight, self.loop_step[t])
            x = self.layers[i](x, meta, cache.run(r))
            if taps is not None:
                taps.append(x.clone())
        if rows is not None:
            if rows.numel() == 0:                        # nothing asked for: the step only fed the cache
                return torch.empty(0, cfg.vocab_size, dtype=torch.float32, device=x.device)
            x = x.index_select(0, rows)
        h = self.final_norm(x, self.dtype)
        return self.lm_head(h).float()


# --------------------------------------------------------------------------- weights
def _layer_tensors(i: int, spec: LayerSpec, t: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """Checkpoint names (``l<i>.norm1``, ``l<i>.mix.left.q`` ...) -> this package's parameter
    names with the fused input projection."""
    p, o = f"l{i}.", f"layers.{i}."
    L, R = p + "mix.left.", p + "mix.right."
    rows = [t[L + "q"], t[L + "k"], t[L + "v"]] + ([t[L + "g"]] if spec.attn.gate else []) + [t[R + "in"]]
    if spec.ff:
        rows.append(t[p + "mlp.up"])
    out = {o + "norm1.weight": t[p + "norm1"].reshape(1), o + "proj_in.weight": torch.cat(rows, 0),
           o + "mix.left.o.weight": t[L + "o"], o + "mix.left_out": t[L + "out"],
           o + "mix.right.conv_w": t[R + "conv"], o + "mix.right.conv_b": t[R + "conv.b"],
           o + "mix.right.dt_bias": t[R + "dt_bias"], o + "mix.right.A_log": t[R + "A_log"],
           o + "mix.right.D": t[R + "D"], o + "mix.right.norm_w": t[R + "norm"],
           o + "mix.right.o.weight": t[R + "o"], o + "mix.right_out": t[R + "out"]}
    if spec.ff:
        out[o + "down.weight"] = t[p + "mlp.down"]
    return out


def convert_nudadra_tensors(cfg: ModelConfig, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    out = {"embed": tensors["embed"], "final_norm.weight": tensors["final.norm"].reshape(1),
           "lm_head.weight": tensors["head"]}
    if cfg.loop is not None:
        out["loop_in.weight"] = tensors["loop.in"]
        out["loop_step"] = tensors["loop.step"]
    for i, spec in enumerate(cfg.layer_specs):
        out.update(_layer_tensors(i, spec, tensors))
    return out


def export_nudadra_tensors(model: HybridLM) -> Dict[str, torch.Tensor]:
    """Inverse of ``convert_nudadra_tensors`` (checkpoint names, 16-bit storage)."""
    cfg, dt = model.cfg, torch.bfloat16
    p = {k: v.detach() for k, v in model.named_parameters()}
    out = {"embed": p["embed"], "final.norm": p["final_norm.weight"].reshape(()), "head": p["lm_head.weight"]}
    if cfg.loop is not None:
        out["loop.in"], out["loop.step"] = p["loop_in.weight"], p["loop_step"]
    for i, s in enumerate(cfg.layer_specs):
        o, q = f"layers.{i}.", f"l{i}."
        nq, nk, nv, ng = s.attn.proj_sizes
        w = p[o + "proj_in.weight"]
        cuts = [nq, nk, nv] + ([ng] if ng else []) + [s.ssd.in_size] + ([s.ff] if s.ff else [])
        names = ["mix.left.q", "mix.left.k", "mix.left.v"] + (["mix.left.g"] if ng else []) + ["mix.right.in"] + \
            (["mlp.up"] if s.ff else [])
        for nm, part in zip(names, torch.split(w, cuts, 0)):
            out[q + nm] = part
        out[q + "norm1"] = p[o + "norm1.weight"].reshape(())
        for ours, theirs in (("mix.left.o.weight", "mix.left.o"), ("mix.left_out", "mix.left.out"),
                             ("mix.right.conv_w", "mix.right.conv"), ("mix.right.conv_b", "mix.right.conv.b"),
                             ("mix.right.dt_bias", "mix.right.dt_bias"), ("mix.right.A_log", "mix.right.A_log"),
                             ("mix.right.D", "mix.right.D"), ("mix.right.norm_w", "mix.right.norm"),
                             ("mix.right.o.weight", "mix.right.o"), ("mix.right_out", "mix.right.out")):
            out[q + theirs] = p[o + ours]
        if s.ff:
            out[q + "mlp.down"] = p[o + "down.weight"]
    return {k: v.to(dt).contiguous() for k, v in out.items()}


@torch.no_grad()
def load_into_hybrid(model: HybridLM, tensors: Dict[str, torch.Tensor]) -> HybridLM:
    missing = []
    for name, p in model.named_parameters():
        t = tensors.get(name)
        if t is None:
            missing.append(name)
            continue
        assert tuple(t.shape) == tuple(p.shape), f"{name}: {tuple(t.shape)} vs {tuple(p.shape)}"
        p.copy_(t.to(p.dtype))
    if missing:
        raise KeyError(f"checkpoint is missing {missing[:8]}{'...' if len(missing) > 8 else ''}")
    return model


@torch.no_grad()
def init_random_hybrid_(model: HybridLM, seed: int = 0) -> HybridLM:
    """Random weights for benchmarks and tests: projections N(0, 1/sqrt(fan in)) rounded to bf16,
    gains near 1, decay rates and step-size biases in the usual Mamba-2 ranges."""
    for name, p in model.named_parameters():
        g = torch.Generator(device="cpu").manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
        r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float32)
        leaf = name.split(".")[-1]
        if leaf == "weight" and p.dim() == 2:
            v = r(*p.shape) / p.shape[1] ** 0.5
        elif name == "embed":
            v = r(*p.shape)
        elif leaf == "weight" and p.dim() == 1:          # scalar norm gains
            v = 1.0 + 0.1 * r(*p.shape)
        elif leaf == "A_log":
            v = torch.log(1.0 + 7.0 * torch.rand(*p.shape, generator=g))
        elif leaf == "dt_bias":
            v = torch.log(torch.expm1(0.01 + 0.2 * torch.rand(*p.shape, generator=g)))
        elif leaf in ("left_out", "right_out", "norm_w", "D"):
            v = 1.0 + 0.1 * r(*p.shape)
        elif leaf == "conv_w":
            v = r(*p.shape) / p.shape[1] ** 0.5
        else:                                            # conv_b, loop_step
            v = 0.1 * r(*p.shape)
        p.copy_(v.to(torch.bfloat16).to(p.dtype))
    return model


def build_hybrid(cfg: ModelConfig, dtype=torch.bfloat16, device=None, seed: Optional[int] = 0) -> HybridLM:
    m = HybridLM(cfg, dtype=dtype, device=device).eval()
    if seed is not None:
        init_random_hybrid_(m, seed)
    return m

"""A plain, slow implementation of the Nudadra design, one function per mechanism.

Everything is float64 torch on the CPU and written for reading, not for speed: attention builds
each query's visible set one key at a time, the state-space layer steps token by token.  The
tests compare the framework (models / engine / ops) with these functions; nothing here imports
the framework.

Notation: T tokens of one sequence, positions 0..T-1.  A model is a dict ``cfg`` in the layout of
the design's config.json and a dict ``w`` of tensors under the checkpoint's names.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


# --------------------------------------------------------------------------- small pieces
def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its last axis divided by sqrt(mean(x^2) + eps)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number."""
    return rms(x, eps) * g


def group_norm(x, weight, groups: int, eps: float):
    """x [.., C] normalised in ``groups`` equal parts, each by its own root mean square."""
    C = x.shape[-1]
    parts = x.reshape(*x.shape[:-1], groups, C // groups)
    return rms(parts, eps).reshape(x.shape) * weight


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def relu_squared_mlp(h, up, down):
    return (torch.relu(h @ up.T) ** 2) @ down.T


# --------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict):
    """(frequency per pair [dims/2], multiplier of cos and sin) with the YaRN blend when the
    config carries ``scaling``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(t):
        return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(half)], dtype=F64)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, pos: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    """x [T, heads, D]; the first rot.dims coordinates of each head turn by pos * frequency, pair
    (i, i + dims/2); the rest pass."""
    if not rot:
        return x
    dims = int(rot["dims"])
    half = dims // 2
    f, mult = rotary_frequencies(rot)
    ang = pos.to(F64)[:, None] * f[None]                   # [T, half]
    c, s = (ang.cos() * mult)[:, None], (ang.sin() * mult)[:, None]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


# --------------------------------------------------------------------------- windowed attention with pooled blocks
def visible(i: int, window: Optional[int], pool: Optional[int]):
    """(token positions, block numbers) that query position i sees."""
    if window is None:
        return list(range(i + 1)), []
    toks = [j for j in range(i + 1) if 0 <= i - j < window]
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - window:
            blocks.append(b)
            b += 1
    return toks, blocks


def window_pool_attention(q, k, v, scale: float, window: Optional[int], pool: Optional[int]):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] (already rotated) -> [T, H, Dv].  One softmax over
    the window's tokens and the means of the blocks that lie wholly before the window."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=F64)
    for i in range(T):
        toks, blocks = visible(i, window, pool)
        for h in range(H):
            g = h // (H // G)
            keys = [k[j, g] for j in toks] + [k[b * pool:(b + 1) * pool, g].mean(0) for b in blocks]
            vals = [v[j, g] for j in toks] + [v[b * pool:(b + 1) * pool, g].mean(0) for b in blocks]
            K, V = torch.stack(keys), torch.stack(vals)
            p = torch.softmax((K @ q[i, h]) * scale, 0)
            out[i, h] = p @ V
    return out


def attention_branch(h, w: Dict[str, torch.Tensor], pre: str, c: dict, pos):
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    T = h.shape[0]
    q = (h @ w[pre + "q"].T).view(T, H, D)
    k = (h @ w[pre + "k"].T).view(T, G, D)
    v = (h @ w[pre + "v"].T).view(T, G, Dv)
    q, k = rotate(q, pos, c.get("rot")), rotate(k, pos, c.get("rot"))
    mask = c.get("mask") or {}
    o = window_pool_attention(q, k, v, float(c["scale"]), mask.get("size"), mask.get("pool"))
    gate = torch.sigmoid(h @ w[pre + "g"].T)               # [T, H]
    return (o * gate[..., None]).reshape(T, H * Dv) @ w[pre + "o"].T


# --------------------------------------------------------------------------- state-space branch
def causal_conv(x, weight, bias):
    """x [T, C]; weight [C, taps] whose last column meets the current token; zeros before 0."""
    T, C = x.shape
    taps = weight.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], 0)
    out = torch.zeros(T, C, dtype=x.dtype)
    for t in range(T):
        out[t] = (pad[t:t + taps].T * weight).sum(-1) + bias
    return out


def ssd_scan(x, B, C, dt, A_log, D, groups: int):
    """x [T, Hs, P], B / C [T, groups, N], dt [T, Hs] (after softplus).  Per head: S <- exp(-exp(A_log) dt) S
    + dt B x^T, y = S^T C + D x, S [N, P] from zero."""
    T, Hs, P = x.shape
    N = B.shape[-1]
    y = torch.zeros(T, Hs, P, dtype=F64)
    for h in range(Hs):
        g = h // (Hs // groups)
        S = torch.zeros(N, P, dtype=F64)
        a = torch.exp(A_log[h])
        for t in range(T):
            S = torch.exp(-a * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


def ssm_branch(h, w, pre: str, c: dict, eps: float):
    Hs, P, N, G = c["heads"], c["vdim"], c["state"], c["groups"]
    inner = Hs * P
    T = h.shape[0]
    u = h @ w[pre + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    x = xbc[:, :inner].view(T, Hs, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"])
    y = ssd_scan(x, B, C, dt, w[pre + "A_log"], w[pre + "D"], G).reshape(T, inner)
    y = group_norm(y * silu(z), w[pre + "norm"], c["norm_groups"], eps)
    return y @ w[pre + "o"].T


# --------------------------------------------------------------------------- layer and model
def parallel_mixer(h, w, pre: str, c: dict, eps: float, pos):
    left = attention_branch(h, w, pre + "left.", c["left"], pos)
    right = ssm_branch(h, w, pre + "right.", c["right"], eps)
    return 0.5 * (rms(left, eps) * w[pre + "left.out"] + rms(right, eps) * w[pre + "right.out"])


def layer(x, w, i: int, spec: dict, eps: float, pos):
    pre = f"l{i}."
    h = scalar_norm(x, w[pre + "norm1"], eps)
    out = parallel_mixer(h, w, pre + "mix.", spec["mixer"], eps, pos)
    if spec.get("mlp"):
        out = out + relu_squared_mlp(h, w[pre + "mlp.up"], w[pre + "mlp.down"])
    return x + out


def layer_runs(cfg: dict) -> List[tuple]:
    """[(layer index, pass number or None)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens, collect: Optional[list] = None):
    """Logits [T, vocab] of one sequence from position 0 (float64).  ``collect`` receives the
    residual stream after every layer run."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    pos = torch.arange(len(ids))
    x0 = w["embed"][ids] * float(cfg["embedding"]["scale"])
    x = x0
    loop = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t is not None and i == loop["start"]:
            x = torch.cat([x, x0], -1) @ w["loop.in"].T + w["loop.step"][t]
        x = layer(x, w, i, cfg["layers"][i], eps, pos)
        if collect is not None:
            collect.append(x.clone())
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].T

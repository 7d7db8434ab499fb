"""A plain, slow implementation of the Pagonex design, one function per mechanism.

Everything is float64 torch on the CPU and written for reading, not for speed: attention expands
every head's keys and values from the latent and scores one query at a time, the delta-rule layer
steps token by token, the mixture of experts loops over tokens.  The tests compare the framework
(models / engine / ops) with these functions; nothing here imports the framework.

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
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def causal_conv(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x [T, C], weight [C, taps]: y_t = sum_j weight[:, j] x_(t - taps + 1 + j), zeros before t = 0."""
    T, C = x.shape
    taps = weight.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += weight[:, j] * x[s]
    return y


def input_conv(x, weight):
    """What a sublayer reads: its input plus the causal convolution of that input."""
    return x + causal_conv(x, weight)


# --------------------------------------------------------------------------- embedding
def embed(ids: List[int], table, bigram, b: dict):
    """Token row plus the row of the (previous, current) pair's bucket; a sequence's first token takes
    the table's last row."""
    n = int(b["buckets"])
    rows = []
    for t, tok in enumerate(ids):
        r = n if t == 0 else (ids[t - 1] * int(b["mul_prev"]) + tok * int(b["mul_cur"])) % n
        rows.append(table[tok] + bigram[r])
    return torch.stack(rows)


# --------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict):
    """(frequency per pair [dims / 2], multiplier of cos and sin); YaRN blend when ``scaling`` is given."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])
    where = lambda turns: dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(where(float(sc["fast"]))), 0)
    hi = min(math.ceil(where(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(float(f[i]) / factor * ramp + float(f[i]) * (1 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, pos: int, rot: dict) -> torch.Tensor:
    """x [.., n]: coordinates (2i, 2i + 1), i < dims / 2, turn by pos * f_i; the rest passes."""
    f, gain = rotary_frequencies(rot)
    y = x.clone()
    for i in range(int(rot["dims"]) // 2):
        a = pos * float(f[i])
        c, s = math.cos(a) * gain, math.sin(a) * gain
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        y[..., 2 * i] = u * c - v * s
        y[..., 2 * i + 1] = v * c + u * s
    return y


# --------------------------------------------------------------------------- latent attention
def latent_kv(h, w, p: str, m: dict, eps: float):
    """The cached part of a latent-attention layer: (normed latent [T, kv_rank], rotated shared key
    part [T, rot_dim])."""
    r = int(m["kv_rank"])
    d = h @ w[p + "dkv"].T
    c = rms(d[:, :r], eps) * w[p + "dkv.norm"]
    kr = torch.stack([rotate_pairs(d[t, r:], t, m["rot"]) for t in range(h.shape[0])])
    return c, kr


def latent_attention(h, w, p: str, m: dict, eps: float, kv=None):
    """h [T, W] -> [T, W].  ``kv``: (latent, rotated key part) of another layer to use instead of
    this layer's own down projection."""
    T = h.shape[0]
    H, D, R, Dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    cq = rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).reshape(T, H, D + R)
    c, kr = kv if kv is not None else latent_kv(h, w, p, m, eps)
    kn = (c @ w[p + "uk"].T).reshape(T, H, D)
    v = (c @ w[p + "uv"].T).reshape(T, H, Dv)
    size = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, Dv, dtype=F64)
    for i in range(T):
        js = [j for j in range(i + 1) if size is None or i - j < int(size)]
        for hh in range(H):
            qr = rotate_pairs(q[i, hh, D:], i, m["rot"])
            s = torch.stack([(q[i, hh, :D] @ kn[j, hh] + qr @ kr[j]) * float(m["scale"]) for j in js])
            pw = torch.softmax(s, 0)
            out[i, hh] = sum(pw[n] * v[j, hh] for n, j in enumerate(js))
    return out.reshape(T, H * Dv) @ w[p + "o"].T, (c, kr)


# --------------------------------------------------------------------------- gated delta rule
def delta_rule(q, k, v, g, beta):
    """One head.  q, k, g [T, N], v [T, P], beta [T].  S [N, P] starts at zero; per token: rows of S
    decay by g, the write is beta (v - S^T k) along k, the read-out S^T q sees it."""
    T, N = q.shape
    S = torch.zeros(N, v.shape[1], dtype=F64)
    out = []
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def channel_delta(h, w, p: str, m: dict, eps: float):
    T = h.shape[0]
    H, G, N, P = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    short = lambda name: silu(causal_conv(h @ w[p + name].T, w[p + name + ".conv"]))
    unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
    q = unit(short("q").reshape(T, G, N)) * N ** -0.5
    k = unit(short("k").reshape(T, G, N))
    v = short("v").reshape(T, H, P)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    rate = torch.exp(w[p + "A_log"])[None, :, None]
    g = torch.exp(-rate * softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, N))
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, P)
    heads = []
    for hh in range(H):
        kvh = hh // (H // G)
        o = delta_rule(q[:, kvh], k[:, kvh], v[:, hh], g[:, hh], beta[:, hh])
        heads.append(rms(o, eps) * w[p + "norm"] * gate[:, hh])
    return torch.cat(heads, -1) @ w[p + "o"].T


# --------------------------------------------------------------------------- feed-forward
def expert(h, w, p: str, limit: float):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[p + "down"].T


def moe(h, w, p: str, m: dict):
    r = m["router"]
    E, top = int(r["experts"]), int(r["top"])
    s = torch.softmax(h @ w[p + "router"].T, -1)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        pick = sorted(range(E), key=lambda e: -float(s[t, e]))[:top]
        tot = sum(s[t, e] for e in pick) + 1e-20
        for e in pick:
            out[t] += s[t, e] / tot * float(r["scale"]) * expert(h[t:t + 1], w, f"{p}e{e}.", float(m["expert"]["limit"]))[0]
    if m.get("shared"):
        out = out + expert(h, w, p + "shared.", float(m["shared"]["limit"]))
    return out


# --------------------------------------------------------------------------- the model
def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: List[int], taps: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; ``taps`` receives the residual stream after every layer."""
    w = {k: v.to(F64) for k, v in w.items()}
    ids = [int(t) for t in ids]
    eps = float(cfg["norm"]["eps"])
    big = (cfg.get("embedding") or {}).get("bigram")
    x = embed(ids, w["embed"], w["bigram"], big) if big else w["embed"][ids]
    reads = (lambda x, name: input_conv(x, w[name])) if (cfg.get("canon") or {}).get("taps") else (lambda x, name: x)
    kept = {}
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = reads(x, p + "canon1")
        if l["type"] == "latent_attention":
            src = l["mixer"].get("kv_from")
            y, kept[i] = latent_attention(h, w, p + "mix.", l["mixer"], eps, kept[src] if src is not None else None)
        elif l["type"] == "channel_delta":
            y = channel_delta(h, w, p + "mix.", l["mixer"], eps)
        else:
            raise ValueError(l["type"])
        x = x + layer_norm(y, w[p + "norm1"], w[p + "norm1.b"], eps)
        if l.get("mlp"):
            h = reads(x, p + "canon2")
            x = x + layer_norm(moe(h, w, p + "mlp.", l["mlp"]), w[p + "norm2"], w[p + "norm2.b"], eps)
        if taps is not None:
            taps.append(x.clone())
    return layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T * float(cfg["logit_scale"])

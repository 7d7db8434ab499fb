"""Pagonex models through the framework (loader, paged cache and state slots, ragged engine, scheduler,
kernels) against the plain implementation in ``pagonex_oracle`` (float64, written from the design's
equations; shares no code with the package).

Every test makes its own small configuration and random weights (checkpoint names and shapes are
produced here, saved as safetensors and read back by the package's loader).  ``dev`` runs each
case on the CPU (PyTorch forms of the ops) and, marked ``gpu``, on the HIP kernels.
"""
import json
import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import pagonex_oracle as oracle  # noqa: E402

from edgellm.engine.generate import SamplingParams  # noqa: E402
from edgellm.engine.paged import PagedCache  # noqa: E402
from edgellm.engine.ragged import RaggedEngine, RaggedGenerator  # noqa: E402
from edgellm.models.registry import load_model  # noqa: E402
from edgellm.ops import seqmix  # noqa: E402

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64
# a norm on each sublayer's output divides by the output's own spread, so tiny random models amplify fp32
# rounding a few hundred times at some rows (a relative weight perturbation of 1e-7 moves the oracle's
# own logits by up to 3e-4 there); a fault of a mechanism shows at 1e-2 and above
TOL = {"fp32": 1.5e-4, "bf16": 6e-2}


# --------------------------------------------------------------------------- configurations and weights
def latent(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=10, kv_rank=12, window=9, rot_dims=None, scaling=True, kv_from=None,
           scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim),
         "rot": {"dims": rot_dims if rot_dims is not None else rot_dim, "base": 100.0}}
    if scaling:
        m["rot"]["scaling"] = {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def delta(heads=4, kv_heads=2, dim=6, vdim=5, conv=3):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def moe(experts=5, top=2, ff=7, shared=9, scale=1.5, limit=1.2):
    m = {"kind": "moe", "router": {"experts": experts, "top": top, "scale": scale}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared, "limit": limit * 1.5}
    return m


def make_config(layers=None, mlps=None, width=20, vocab=53, taps=3, buckets=31, logit_scale=0.7):
    layers = layers if layers is not None else [latent(), delta(), latent(kv_from=0, window=5), delta(heads=2, kv_heads=2)]
    mlps = mlps if mlps is not None else [moe()] * len(layers)
    cfg = {"architecture": "Pagonex", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "logit_scale": logit_scale,
           "layers": [dict(l, mlp=m) for l, m in zip(layers, mlps)]}
    if taps:
        cfg["canon"] = {"taps": taps}
    if buckets:
        cfg["embedding"] = {"bigram": {"buckets": buckets, "mul_prev": 13, "mul_cur": 5}}
    return cfg


def make_weights(cfg, seed=0, decay_rank=3, gate_rank=4):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    bf = lambda t: t.to(torch.bfloat16)
    rn = lambda *s, k=1.0: bf(torch.randn(*s, generator=g) * k)
    lin = lambda o, i: rn(o, i, k=i ** -0.5)
    w = {"embed": rn(cfg["vocab"], W, k=0.7), "head": lin(cfg["vocab"], W), "final.norm": bf(1 + 0.2 * torch.randn(W, generator=g)),
         "final.norm.b": rn(W, k=0.1)}
    if cfg.get("embedding"):
        w["bigram"] = rn(cfg["embedding"]["bigram"]["buckets"] + 1, W, k=0.5)
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        for n in ("1", "2") if l["mlp"] else ("1",):
            w[p + "norm" + n], w[p + "norm" + n + ".b"] = bf(1 + 0.2 * torch.randn(W, generator=g)), rn(W, k=0.1)
            if taps:
                w[p + "canon" + n] = rn(W, taps, k=0.4)
        M = p + "mix."
        if l["type"] == "latent_attention":
            H, D, R, Dv, qr, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            w[M + "dq"], w[M + "dq.norm"] = lin(qr, W), bf(1 + 0.2 * torch.randn(qr, generator=g))
            w[M + "uq"] = lin(H * (D + R), qr)
            if m.get("kv_from") is None:
                w[M + "dkv"], w[M + "dkv.norm"] = lin(kr + R, W), bf(1 + 0.2 * torch.randn(kr, generator=g))
            w[M + "uk"], w[M + "uv"], w[M + "o"] = lin(H * D, kr), lin(H * Dv, kr), lin(W, H * Dv)
        else:
            H, G, N, P, c = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for n, rows in (("q", G * N), ("k", G * N), ("v", H * P)):
                w[M + n], w[M + n + ".conv"] = lin(rows, W), rn(rows, c, k=0.6)
            w[M + "b"], w[M + "A_log"] = lin(H, W), bf(torch.rand(H, generator=g) - 1.0)
            w[M + "a1"], w[M + "a2"], w[M + "dt_bias"] = lin(decay_rank, W), lin(H * N, decay_rank), rn(H * N, k=0.5)
            w[M + "g1"], w[M + "g2"] = lin(gate_rank, W), lin(H * P, gate_rank)
            w[M + "norm"], w[M + "o"] = bf(1 + 0.2 * torch.randn(P, generator=g)), lin(W, H * P)
        if l["mlp"]:
            F_, e = p + "mlp.", l["mlp"]
            w[F_ + "router"] = rn(e["router"]["experts"], W, k=0.8)
            names = [f"e{k}" for k in range(e["router"]["experts"])] + (["shared"] if e.get("shared") else [])
            for nm in names:
                ff = e["shared"]["ff"] if nm == "shared" else e["expert"]["ff"]
                w[F_ + nm + ".gate"], w[F_ + nm + ".up"], w[F_ + nm + ".down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return w


def load(tmp_path, cfg, w, dev, precision="fp32"):
    from safetensors.torch import save_file
    d = tmp_path / f"m{len(os.listdir(tmp_path))}"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
    model, _, src = load_model(str(d), precision=precision, device=torch.device(dev))
    assert src.startswith("checkpoint:")
    return model


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def replay(model, schedule, reqs, max_tokens, slots=4, graphs=None):
    """``schedule``: steps of [(request name, token count)]; every row's logits are collected.
    A request ends (slot and pages given back) with its last token."""
    eng = RaggedEngine(model, max_tokens, slots=slots, use_graphs=graphs)
    at = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    for step in schedule:
        entries = []
        for r, n in step:
            entries.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
        logits = eng.step(entries).cpu()
        o = 0
        for r, n in step:
            got[r].append(logits[o:o + n])
            o += n
            if at[r] == len(reqs[r]):
                eng.close(r)
    assert all(at[r] == len(reqs[r]) for r in reqs)
    return {r: torch.cat(v) for r, v in got.items()}, eng


def close(got, want, tol):
    d = got.double() - want
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().max().item() / want.std().item() < tol


def row_err(got, want):
    d = got.double() - want
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt() / want.std().item()


def close_conditioned(got, want, cfg, w, toks, tol):
    """``close`` with a per-row allowance for badly conditioned rows of a tiny random model: the larger
    of ``tol`` and twice what a relative perturbation of the weights by one part in 10^7 (about one
    fp32 rounding) does to the oracle's own logits."""
    g = torch.Generator().manual_seed(1)
    w2 = {k: (v.double() * (1 + 1e-7 * torch.randn(v.shape, generator=g, dtype=F64))) for k, v in w.items()}
    allow = torch.clamp(2 * row_err(oracle.forward(cfg, w2, toks), want), min=tol)
    return bool((row_err(got, want) < allow).all()) and bool((allow < 50 * tol).all())


def portions(total, first=2, mod=9):
    cuts, n = [], first
    while total:
        cuts.append(min(n, total))
        total -= cuts[-1]
        n = n % mod + 2
    return cuts


class _Spec:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def _meta(cache, seqs, dev):
    for slot, start, n in seqs:
        cache.extend(slot, start + n)
    return seqmix.RaggedMeta.build(seqs, cache.page_table, cache.page, dev)


def _state_cache(dev, width=0, taps=0, delta_spec=None, latent_spec=None, pages=8, prev=False):
    spec = _Spec(latent=latent_spec, delta=delta_spec, moe=_Spec(), attn=None, ssd=None)
    return PagedCache([spec], pages, slots=3, page=64, dtype=torch.float32, device=dev, width=width, canon_taps=taps,
                      prev_token=prev)


# --------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dev", DEVS)
def test_bigram_embedding_in_portions_over_used_slots(dev):
    """Portions of 1..5 tokens of two interleaved sequences; the slots held other tokens before."""
    torch.manual_seed(0)
    V, W, B = 17, 12, 7
    table, big = torch.randn(V, W), torch.randn(B + 1, W)
    consts = {"buckets": B, "mul_prev": 3, "mul_cur": 11}
    a, b = tokens(19, V, 1), tokens(11, V, 2)
    want = {0: oracle.embed(a, table.double(), big.double(), consts), 2: oracle.embed(b, table.double(), big.double(), consts)}
    cache = _state_cache(dev, prev=True)
    cache.prev_tok.fill_(5)                                   # what an earlier request left behind
    at, n, got = {0: 0, 2: 0}, 1, {0: [], 2: []}
    seqs = {0: a, 2: b}
    while any(at[s] < len(seqs[s]) for s in seqs):
        step = [(s, at[s], min(n + s, len(seqs[s]) - at[s])) for s in seqs if at[s] < len(seqs[s])]
        meta = _meta(cache, step, dev)
        ids = torch.tensor([t for s, st, k in step for t in seqs[s][st:st + k]], device=dev)
        out = seqmix.embedding_bigram(ids, meta, table.to(dev), big.to(dev), cache.prev_tok, B, 3, 11).cpu()
        o = 0
        for s, st, k in step:
            got[s].append(out[o:o + k])
            o += k
            at[s] += k
        n = n % 5 + 1
    for s in seqs:
        assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=1e-6)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("taps,W", [(3, 10), (1, 8), (2, 300), (5, 33)])
def test_input_convolution_in_portions(dev, taps, W):
    torch.manual_seed(taps)
    T = 23
    x, w = torch.randn(T, W), torch.randn(W, taps) * 0.5
    want = oracle.input_conv(x.double(), w.double())
    cache = _state_cache(dev, width=W, taps=taps)
    run = cache.run(0)
    run.canon1.normal_()                                      # stale rows of an earlier request
    out, at, n = [], 0, 1
    while at < T:
        n = min(n, T - at)
        meta = _meta(cache, [(1, at, n)], dev)
        out.append(seqmix.canon_conv(x[at:at + n].to(dev), w.to(dev), run.canon1, meta, torch.float32).cpu())
        at += n
        n = n % 6 + 1
    assert torch.allclose(torch.cat(out).double(), want, atol=1e-5)


@pytest.mark.parametrize("dev", DEVS)
def test_norms_activation_and_expert_sum(dev):
    torch.manual_seed(3)
    T, W, K = 7, 37, 3
    x, y = torch.randn(T, W) * 3 + 1, torch.randn(T, W)
    w, b = torch.randn(W), torch.randn(W)
    parts, pw = torch.randn(T, K, W), torch.rand(T, K)
    D = lambda t: t.to(dev)
    assert torch.allclose(seqmix.layer_norm_rows(D(x), D(w), D(b), 1e-5, torch.float32).cpu().double(),
                          oracle.layer_norm(x.double(), w.double(), b.double(), 1e-5), atol=1e-5)
    summed = y.double() + (pw.double()[..., None] * parts.double()).sum(1)
    for yy, pp, ref in ((y, None, y.double()), (y, parts, summed), (None, parts, summed - y.double())):
        got = seqmix.layer_norm_residual(D(x.clone()), None if yy is None else D(yy), D(w), D(b), 1e-5,
                                         None if pp is None else D(pp), None if pp is None else D(pw)).cpu().double()
        assert torch.allclose(got, x.double() + oracle.layer_norm(ref, w.double(), b.double(), 1e-5), atol=2e-5)
    u = torch.randn(T, 50)
    got = seqmix.rms_norm_cols(D(u), 9, 21, D(w[:21]), 1e-5, torch.float32).cpu().double()
    assert torch.allclose(got, oracle.rms(u[:, 9:30].double(), 1e-5) * w[:21].double(), atol=1e-5)
    gu = torch.randn(T, 22) * 2
    g, up = gu[:, :11].double().clamp(max=1.3), gu[:, 11:].double().clamp(-1.3, 1.3)
    assert torch.allclose(seqmix.glu_clamp(D(gu), 11, 1.3).cpu().double(), g * torch.sigmoid(1.702 * g) * (up + 1), atol=1e-5)
    yh, z, wn = torch.randn(T, 4 * 9), torch.randn(T, 4 * 9 + 5), torch.randn(9)
    want = (oracle.rms(yh.double().view(T, 4, 9), 1e-5) * wn.double()).reshape(T, 36) * torch.sigmoid(z[:, 5:].double())
    assert torch.allclose(seqmix.head_norm_gate(D(yh), D(z)[:, 5:], D(wn), 4, 1e-5, torch.float32).cpu().double(), want, atol=1e-5)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("H,G,N,P", [(4, 2, 6, 5), (2, 2, 40, 70), (3, 1, 64, 16), (1, 1, 130, 3), (2, 1, 100, 20)])
def test_delta_rule_in_portions_over_stale_state(dev, H, G, N, P):
    """The recurrence alone: two interleaved sequences fed in portions of 1..7 tokens into slots whose
    state an earlier request left behind; decays well below one, so a lost or stale state shows."""
    torch.manual_seed(N)
    T = {0: 29, 2: 17}
    GN = G * N
    data, want = {}, {}
    for s, n in T.items():
        qkv = torch.randn(n, 2 * GN + H * P)
        u = torch.randn(n, H + 3)
        a, dtb, A = torch.randn(n, H * N), torch.randn(H * N) * 0.5, torch.rand(H) - 1.0
        data[s] = (qkv, u, a, dtb, A)
        unit = lambda x: x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)
        q = unit(qkv[:, :GN].double().view(n, G, N)) * N ** -0.5
        k = unit(qkv[:, GN:2 * GN].double().view(n, G, N))
        v = qkv[:, 2 * GN:].double().view(n, H, P)
        g = torch.exp(-torch.exp(A.double())[None, :, None] * oracle.softplus(a.double() + dtb.double()).view(n, H, N))
        beta = torch.sigmoid(u[:, 2:2 + H].double())
        want[s] = torch.cat([oracle.delta_rule(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], g[:, h], beta[:, h])
                             for h in range(H)], -1)
    cache = _state_cache(dev, delta_spec=_Spec(heads=H, kv_heads=G, dim=N, vdim=P, conv=2, conv_channels=1))
    run = cache.run(0)
    run.ssm.normal_()
    at, n, got = {s: 0 for s in T}, 1, {s: [] for s in T}
    while any(at[s] < T[s] for s in T):
        step = [(s, at[s], min(n + s, T[s] - at[s])) for s in T if at[s] < T[s]]
        meta = _meta(cache, step, dev)
        outs = []
        for s, st, k in step:                                  # each sequence has its own constants: one call each
            m1 = seqmix.RaggedMeta.build([(s, st, k)], cache.page_table, cache.page, dev)
            qkv, u, a, dtb, A = (t.to(dev) for t in data[s])
            prep = seqmix.delta_prepare(qkv[st:st + k].contiguous(), u[st:st + k].contiguous(), 2, a[st:st + k].contiguous(),
                                        dtb, A, H, G, N)
            outs.append(seqmix.delta_rule_scan(prep, qkv[st:st + k].contiguous(), run.ssm, m1, H, G, N, P).cpu())
        for (s, st, k), o in zip(step, outs):
            got[s].append(o)
            at[s] += k
        n = n % 7 + 1
    for s in T:
        assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=2e-5, rtol=1e-4)


@pytest.mark.parametrize("dev", DEVS)
def test_delta_rule_batch_of_sequences_in_one_call(dev):
    """Three sequences of unequal length in one step (a 40-token portion, a single token, a portion of
    three) against each alone."""
    torch.manual_seed(5)
    H, G, N, P = 4, 2, 12, 20
    lens = [40, 1, 3]
    qkv, u, a = torch.randn(sum(lens), 2 * G * N + H * P), torch.randn(sum(lens), H), torch.randn(sum(lens), H * N)
    dtb, A = torch.randn(H * N) * 0.3, torch.rand(H) - 1.0
    D = lambda t: t.to(dev)
    cache = _state_cache(dev, delta_spec=_Spec(heads=H, kv_heads=G, dim=N, vdim=P, conv=2, conv_channels=1))
    meta = _meta(cache, [(s, 0, n) for s, n in enumerate(lens)], dev)
    prep = seqmix.delta_prepare(D(qkv), D(u), 0, D(a), D(dtb), D(A), H, G, N)
    both = seqmix.delta_rule_scan(prep, D(qkv), cache.run(0).ssm, meta, H, G, N, P).cpu()
    off = 0
    for s, n in enumerate(lens):
        c1 = _state_cache(dev, delta_spec=_Spec(heads=H, kv_heads=G, dim=N, vdim=P, conv=2, conv_channels=1))
        m1 = _meta(c1, [(1, 0, n)], dev)
        p1 = seqmix.delta_prepare(D(qkv[off:off + n]), D(u[off:off + n]), 0, D(a[off:off + n]), D(dtb), D(A), H, G, N)
        one = seqmix.delta_rule_scan(p1, D(qkv[off:off + n]), c1.run(0).ssm, m1, H, G, N, P).cpu()
        assert torch.allclose(both[off:off + n], one, atol=1e-6)
        assert torch.allclose(cache.run(0).ssm[s].cpu(), c1.run(0).ssm[1].cpu(), atol=1e-6)
        off += n


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("T,E,top", [(5, 6, 3), (90, 6, 3), (7, 70, 5), (130, 70, 5)])
def test_router_and_experts(dev, T, E, top):
    """Router choice and weights, and the experts' outputs, for a decode-sized and a prompt-sized step
    (the two expert paths), against the per-token loop."""
    torch.manual_seed(T)
    W, ff = 24, 10
    cfgm = {"router": {"experts": E, "top": top, "scale": 2.0}, "expert": {"ff": ff, "limit": 1.0}}
    w = {"router": torch.randn(E, W)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = torch.randn(ff, W) * 0.3, torch.randn(ff, W) * 0.3, torch.randn(W, ff) * 0.3
    h = torch.randn(T, W)
    want = oracle.moe(h.double(), {k: v.double() for k, v in w.items()}, "", cfgm)
    D = lambda t: t.to(dev)
    idx, wts = seqmix.moe_route(D(h), D(w["router"]), top, 2.0)
    w_gu = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)])
    w_down = torch.stack([w[f"e{e}.down"] for e in range(E)])
    parts = seqmix.moe_experts(D(h), idx, D(w_gu), D(w_down), 1.0)
    got = (wts[..., None] * parts.float()).sum(1).cpu().double()
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-4)
    assert torch.allclose(wts.sum(-1).cpu(), torch.full((T,), 2.0), atol=1e-5)
    # a skewed routing (nearly every token to the same experts) takes the per-expert path of prompt-sized steps
    skew = torch.arange(top, dtype=torch.int32).repeat(T, 1)
    skew[0] = torch.arange(E - top, E, dtype=torch.int32).flip(0)
    one = seqmix.moe_experts(D(h), D(skew), D(w_gu), D(w_down), 1.0).cpu().double()
    for t in (0, 1, T - 1):
        for k in range(top):
            e = int(skew[t, k])
            assert torch.allclose(one[t, k], oracle.expert(h[t:t + 1].double(), {n: v.double() for n, v in w.items()}, f"e{e}.", 1.0)[0],
                                  atol=2e-5, rtol=1e-4)


# --------------------------------------------------------------------------- whole models
CONFIGS = {
    "default": lambda: make_config(),
    # the delta layer first, two taps, one expert per token and no shared expert, a layer without a feed-forward,
    # rotation on a part of the rotated coordinates and no frequency blend, no window, equal q / k and value head counts
    "other": lambda: make_config(
        layers=[delta(heads=2, kv_heads=1, dim=10, vdim=4, conv=2), latent(heads=2, dim=4, rot_dim=6, vdim=8, window=None,
                                                                          rot_dims=4, scaling=False),
                delta(heads=3, kv_heads=3, dim=4, vdim=9, conv=5), latent(heads=2, dim=4, rot_dim=6, vdim=3, window=4,
                                                                          rot_dims=4, scaling=False, kv_from=1, kv_rank=12)],
        mlps=[moe(experts=3, top=1, shared=0), None, moe(experts=4, top=4, ff=5), moe(experts=2, top=1, shared=3)],
        width=24, taps=2, buckets=5, logit_scale=1.0),
    # no input convolution, no pair embedding, one layer of each kind
    "bare": lambda: make_config(layers=[latent(heads=1, window=3), delta(heads=1, kv_heads=1)], mlps=[None, moe(top=5)],
                                taps=0, buckets=0),
}


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_decode_and_portions(tmp_path, dev, name):
    """The residual stream after every layer and the logits of a whole prompt; the same logits from
    prompt + token-by-token decoding, and from portions of 2..9 tokens."""
    cfg = CONFIGS[name]()
    w = make_weights(cfg, seed=3)
    model = load(tmp_path, cfg, w, dev)
    toks = tokens(45, cfg["vocab"], 4)
    col = []
    want = oracle.forward(cfg, w, toks, col)
    eng = RaggedEngine(model, 64)
    taps = []
    got = eng.step([("a", toks, list(range(45)))], taps).cpu()
    for a, b in zip(taps, col):
        assert torch.allclose(a.cpu().double(), b, atol=3e-4, rtol=1e-4)
    assert close(got, want, TOL["fp32"])
    dec, _ = replay(model, [[("a", 12)]] + [[("a", 1)]] * 33, {"a": toks}, 64)
    assert close(dec["a"], want, TOL["fp32"])
    por, _ = replay(model, [[("a", c)] for c in portions(40)] + [[("a", 1)]] * 5, {"a": toks}, 64)
    assert close(por["a"], want, TOL["fp32"])
    two, _ = replay(model, [[("a", 2)]] * 22 + [[("a", 1)]], {"a": toks}, 64)
    assert close(two["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_random_geometries(tmp_path, dev):
    """Sizes drawn at random: head counts and ratios, key / value / latent sizes, windows, taps, expert counts."""
    rnd = torch.Generator().manual_seed(77)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rnd))
    for case in range(4):
        kvh = ri(1, 2)
        rot = 2 * ri(1, 3)
        lat0 = latent(heads=ri(1, 4), dim=ri(2, 9), rot_dim=rot, vdim=ri(2, 9), q_rank=ri(3, 9), kv_rank=ri(4, 14),
                      window=ri(2, 12), rot_dims=2 * ri(1, rot // 2), scaling=bool(case % 2))
        lat1 = latent(heads=ri(1, 4), dim=ri(2, 9), rot_dim=rot, vdim=ri(2, 9), q_rank=ri(3, 9), kv_rank=lat0["mixer"]["kv_rank"],
                      window=ri(2, 12), rot_dims=lat0["mixer"]["rot"]["dims"], scaling=bool(case % 2), kv_from=case % 2)
        dl = delta(heads=kvh * ri(1, 3), kv_heads=kvh, dim=ri(2, 11), vdim=ri(2, 11), conv=ri(1, 4))
        order = [lat0, dl, lat1] if case % 2 == 0 else [dl, lat0, dl, lat1]
        if case % 2:
            lat1["mixer"]["kv_from"] = 1
        cfg = make_config(layers=order, mlps=[moe(experts=ri(2, 7), top=1, ff=ri(2, 9), shared=ri(0, 1) * ri(2, 9))
                                              for _ in order], width=2 * ri(5, 12), taps=ri(1, 4), buckets=ri(2, 40))
        for l in cfg["layers"]:
            l["mlp"]["router"]["top"] = ri(1, l["mlp"]["router"]["experts"])
        w = make_weights(cfg, seed=case, decay_rank=ri(1, 5), gate_rank=ri(1, 5))
        model = load(tmp_path, cfg, w, dev)
        toks = tokens(30, cfg["vocab"], case)
        want = oracle.forward(cfg, w, toks)
        got, _ = replay(model, [[("a", c)] for c in portions(24, first=3, mod=7)] + [[("a", 1)]] * 6, {"a": toks}, 64)
        assert close_conditioned(got["a"], want, cfg, w, toks, TOL["fp32"]), cfg


@pytest.mark.parametrize("dev", DEVS)
def test_mixed_batches_reuse_pages_and_slots(tmp_path, dev):
    """Five unequal requests through three slots and six pages: portions beside single tokens, a request
    paused for a step, slots and pages handed on to later requests.  Page size 64 with requests up to
    150 tokens crosses page borders inside prompts and while decoding; the window (70) spans a border."""
    cfg = make_config(layers=[latent(window=70), delta(), latent(kv_from=0, window=66), delta(heads=2, kv_heads=1)])
    w = make_weights(cfg, seed=7)
    model = load(tmp_path, cfg, w, dev)
    reqs = {"a": tokens(150, cfg["vocab"], 1), "b": tokens(3, cfg["vocab"], 2), "c": tokens(66, cfg["vocab"], 3),
            "d": tokens(1, cfg["vocab"], 4), "e": tokens(130, cfg["vocab"], 5)}
    want = {r: oracle.forward(cfg, w, t) for r, t in reqs.items()}
    sched = [[("a", 60), ("b", 2), ("d", 1)], [("a", 5), ("b", 1), ("c", 64)], [("c", 1), ("a", 62)],
             [("a", 1), ("c", 1), ("e", 63)], [("e", 2), ("a", 20)], [("e", 64), ("a", 1)], [("a", 1), ("e", 1)]]
    got, eng = replay(model, sched, reqs, max_tokens=6 * 64, slots=3)
    for r in reqs:
        assert close(got[r], want[r], TOL["fp32"]), r
    assert eng.cache.stats()["free_pages"] == eng.cache.num_pages and eng.cache.stats()["free_slots"] == 3
    alone, _ = replay(model, [[("e", 130)]], {"e": reqs["e"]}, 192)
    assert close(got["e"], alone["e"].double(), TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_window_edges_with_sharp_scores(tmp_path, dev):
    """Window 8 with the softmax scale enlarged so that single keys carry the weight: the key just inside
    and just outside the window decides the logits, in a prompt and while decoding, at every cut near
    the edge; a window one token off is told apart by the oracle itself."""
    cfg = make_config(layers=[latent(window=8, scale=6.0, heads=2)], mlps=[None])
    w = make_weights(cfg, seed=9)
    model = load(tmp_path, cfg, w, dev)
    toks = tokens(30, cfg["vocab"], 10)
    want = oracle.forward(cfg, w, toks)
    off = json.loads(json.dumps(cfg))
    off["layers"][0]["mixer"]["mask"]["size"] = 9
    assert not close(oracle.forward(off, w, toks)[9:], want[9:], 1e-3)
    off["layers"][0]["mixer"]["mask"]["size"] = 7
    assert not close(oracle.forward(off, w, toks)[9:], want[9:], 1e-3)
    for cut in (6, 7, 8, 9, 10, 13):
        got, _ = replay(model, [[("a", cut)]] + [[("a", 1)]] * (30 - cut), {"a": toks}, 64)
        assert close(got["a"], want, TOL["fp32"]), cut


@pytest.mark.parametrize("dev", DEVS)
def test_far_token_through_the_recurrent_state(tmp_path, dev):
    """A delta-rule layer with slow decays keeps a token from 140 positions back: changing the first
    token moves the last logits (by the oracle), and the framework follows through prompt portions,
    page borders and 60 decoded tokens."""
    cfg = make_config(layers=[delta(heads=2, kv_heads=1, dim=8, vdim=8)], mlps=[None], taps=0, buckets=0)
    w = make_weights(cfg, seed=12)
    w["l0.mix.A_log"] = torch.full_like(w["l0.mix.A_log"], -6.0)             # decays close to one
    model = load(tmp_path, cfg, w, dev)
    toks = tokens(141, cfg["vocab"], 13)
    want = oracle.forward(cfg, w, toks)
    moved = oracle.forward(cfg, w, [(toks[0] + 1) % cfg["vocab"]] + toks[1:])
    assert not close(moved[-3:], want[-3:], 1e-3)
    got, _ = replay(model, [[("a", c)] for c in (50, 14, 17)] + [[("a", 1)]] * 60, {"a": toks}, 192)
    assert close(got["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_bf16_model_and_long_decoding(tmp_path, dev):
    """The 16-bit model against the oracle within rounding, 120 decoded tokens after a short prompt."""
    cfg = make_config(width=32)
    w = make_weights(cfg, seed=11)
    model = load(tmp_path, cfg, w, dev, precision="bf16")
    assert model.dtype == torch.bfloat16
    toks = tokens(128, cfg["vocab"], 12)
    want = oracle.forward(cfg, w, toks)
    got, _ = replay(model, [[("a", 8)]] + [[("a", 1)]] * 120, {"a": toks}, 128)
    # 16-bit rounding flips an expert choice at a few rows of a tiny model (the router sees a slightly
    # different stream): the bulk of the rows is held to rounding, the tail to a loose bound
    e = row_err(got["a"], want)
    assert e.median() < 4e-2 and e.quantile(0.9) < 0.2, (e.median(), e.quantile(0.9))
    m32 = load(tmp_path, cfg, w, dev)
    got32, _ = replay(m32, [[("a", 8)]] + [[("a", 1)]] * 120, {"a": toks}, 128)
    assert close(got32["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_greedy_generation_through_the_scheduler(tmp_path, dev):
    """Greedy tokens from ``RaggedGenerator.generate`` (more prompts than slots, chunked prompts) equal
    the oracle's argmax continuation."""
    cfg = make_config()
    w = make_weights(cfg, seed=13)
    model = load(tmp_path, cfg, w, dev)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (5, 19, 1, 33, 8)]
    new = 6

    def greedy(p):
        seq = list(p)
        for _ in range(new):
            lg = oracle.forward(cfg, w, seq)[-1]
            top = torch.topk(lg, 2).values
            if (top[0] - top[1]) < 1e-3:                       # a near tie is not a test of anything
                return None
            seq.append(int(lg.argmax()))
        return seq[len(p):]

    want = [greedy(p) for p in prompts]
    gen = RaggedGenerator(model, max_batch=2, max_seq=64, prefill_chunk=7)
    res = gen.generate(prompts, SamplingParams(max_new_tokens=new, do_sample=False, repetition_penalty=1.0))
    for g, x in zip(res.tokens, want):
        assert x is None or g == x
    assert gen.kv.stats()["free_pages"] == gen.kv.num_pages


def test_checkpoint_round_trip(tmp_path):
    """save -> load gives the same logits; the exported names and shapes are the checkpoint's."""
    from edgellm.models.hf import save_hf_model
    cfg = CONFIGS["other"]()
    w = make_weights(cfg, seed=2)
    model = load(tmp_path, cfg, w, "cpu")
    out = save_hf_model(model, str(tmp_path / "again"))
    from safetensors.torch import load_file
    back = load_file(os.path.join(out, "model.safetensors"))
    assert {k: tuple(v.shape) for k, v in back.items()} == {k: tuple(v.shape) for k, v in w.items()}
    again, _, _ = load_model(out, precision="fp32", device=torch.device("cpu"))
    toks = tokens(12, cfg["vocab"], 1)
    a = RaggedEngine(model, 64).step([("a", toks, list(range(12)))])
    b = RaggedEngine(again, 64).step([("a", toks, list(range(12)))])
    assert torch.allclose(a, b, atol=1e-6)


def test_evaluate_cli_runs_a_pagonex_checkpoint(tmp_path):
    """The evaluation command line on a checkpoint folder of this design (vocabulary wide enough for the
    byte tokenizer): loader by config.json, paged engine and scheduler, the sampling configuration, the
    confidence metric through the model's own prompt pass."""
    from safetensors.torch import save_file
    from edgellm.cli import evaluate
    cfg = make_config(vocab=300, width=24)
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file(make_weights(cfg, seed=3), str(d / "model.safetensors"))
    y = tmp_path / "c.yaml"
    y.write_text(f"""
max_new_tokens: 4
temperature: 0.7
top_k: 50
top_p: 0.9
repetition_penalty: 1.1
dataset_name: sentence-transformers/natural-questions
dataset_split: train[:2]
embedder_model: "none"
models: ["{d}"]
""")
    out = evaluate.main(["--config", str(y), "--devices", "cpu", "--num_samples", "2", "--max_seq", "256",
                         "--batch_size", "2", "--prefill_chunk", "16", "--precision", "fp32"])
    assert out[str(d)]["tps"] > 0 and 0 < out[str(d)]["confidence"] <= 1


def test_trace_runner_program_on_a_pagonex_checkpoint(tmp_path):
    """``bin/trace_run`` as a program: steps on standard input, logits files and ``done`` lines out; a
    request cut into portions gives the logits of the same request in one step."""
    import subprocess
    import numpy as np
    from safetensors.torch import save_file
    cfg = make_config()
    d = tmp_path / "ckpt"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file(make_weights(cfg, seed=5), str(d / "model.safetensors"))
    toks = tokens(20, cfg["vocab"], 6)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks, "want": [3, 19]}], "end": ["a"]},
             {"step": 1, "entries": [{"id": "b", "tokens": toks[:7], "want": [3]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": toks[7:19], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "b", "tokens": toks[19:], "want": [0]}], "end": ["b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(d), "--dtype", "float32", "--out",
                        str(tmp_path / "out"), "--max-tokens", "64", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = cfg["vocab"]
    whole = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(2, V)
    first = np.fromfile(tmp_path / "out" / "1.f32", dtype="<f4").reshape(1, V)
    last = np.fromfile(tmp_path / "out" / "3.f32", dtype="<f4").reshape(1, V)
    assert not (tmp_path / "out" / "2.f32").exists()
    assert np.allclose(whole[0], first[0], atol=1e-4) and np.allclose(whole[1], last[0], atol=1e-4)
    want = oracle.forward(cfg, make_weights(cfg, seed=5), toks)
    assert close(torch.from_numpy(whole.copy()), want[[3, 19]], TOL["fp32"])


# --------------------------------------------------------------------------- GPU only
@pytest.mark.gpu
def test_decode_graph_replays_match_eager(tmp_path):
    """Decode steps through the captured graph (replayed many times, eager prompt steps and batch-size
    changes between the replays) equal the same steps run eagerly."""
    cfg = make_config(width=64)
    w = make_weights(cfg, seed=21)
    reqs = {"a": tokens(40, cfg["vocab"], 1), "b": tokens(25, cfg["vocab"], 2), "c": tokens(30, cfg["vocab"], 3)}
    sched = [[("a", 10), ("b", 4)]] + [[("a", 1), ("b", 1)]] * 12 + [[("a", 1), ("b", 1), ("c", 11)]] + \
        [[("a", 1), ("b", 1), ("c", 1)]] * 8 + [[("a", 1), ("c", 1)]] * 9 + [[("c", 1)]] * 2
    outs = {}
    for graphs in (False, True):
        model = load(tmp_path, cfg, w, "cuda", precision="bf16")
        outs[graphs], eng = replay(model, sched, reqs, 256, graphs=graphs)
        assert eng.graphs_used == graphs
    for r in reqs:
        assert torch.allclose(outs[True][r], outs[False][r], atol=1e-5), r


@pytest.mark.gpu
@pytest.mark.parametrize("N,P", [(64, 64), (128, 48), (256, 16), (33, 130)])
def test_delta_rule_long_portions_kernel_against_the_token_loop(N, P):
    """Portions of 300, 65 and 1 tokens in one step, then a second step continuing each from the slots'
    state: the kernel (many staged chunks, every register layout) against the token-by-token PyTorch form."""
    torch.manual_seed(N)
    H, G = 2, 1
    res = {}
    steps = [[300, 65, 1], [40, 200, 7]]
    data = [(torch.randn(sum(l), 2 * G * N + H * P), torch.randn(sum(l), H), torch.randn(sum(l), H * N)) for l in steps]
    dtb, A = torch.randn(H * N) * 0.3, torch.rand(H) - 1.5
    for dev in ("cpu", "cuda"):
        cache = _state_cache(dev, delta_spec=_Spec(heads=H, kv_heads=G, dim=N, vdim=P, conv=2, conv_channels=1), pages=24)
        outs, at = [], [0, 0, 0]
        for lens, (qkv, u, a) in zip(steps, data):
            meta = _meta(cache, [(s, at[s], n) for s, n in enumerate(lens)], dev)
            prep = seqmix.delta_prepare(qkv.to(dev), u.to(dev), 0, a.to(dev), dtb.to(dev), A.to(dev), H, G, N)
            outs.append(seqmix.delta_rule_scan(prep, qkv.to(dev), cache.run(0).ssm, meta, H, G, N, P).cpu())
            at = [x + n for x, n in zip(at, lens)]
        res[dev] = (torch.cat(outs), cache.run(0).ssm.cpu())
    assert torch.allclose(res["cuda"][0], res["cpu"][0], atol=2e-5, rtol=1e-4)
    assert torch.allclose(res["cuda"][1], res["cpu"][1], atol=2e-5, rtol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kv_rank,rot_dim,heads,window", [(24, 8, 6, 600), (64, 32, 16, None), (40, 8, 5, 300), (128, 32, 3, 1000)])
def test_decode_attention_over_long_latent_windows(kv_rank, rot_dim, heads, window, dt):
    """One-token steps of three sequences holding 700-1100 cached latent rows: every query's keys are
    split over several workgroups and the heads of the one kv head over several more; against the same op
    on the CPU in fp32."""
    torch.manual_seed(heads)
    Dc, lens = kv_rank + rot_dim, [700, 1100, 901]
    rows = {s: torch.randn(n, Dc).to(dt).float() for s, n in enumerate(lens)}
    q = (torch.randn(3, heads, Dc) * 0.5).to(dt).float()
    res = {}
    for dev, d in (("cpu", torch.float32), ("cuda", dt)):
        spec = _Spec(heads=heads, kv_rank=kv_rank, rot_dim=rot_dim, cache_dim=Dc, kv_from=None)
        cache = PagedCache([_Spec(latent=spec, delta=None, moe=None, attn=None, ssd=None)], 48, slots=3, page=64, dtype=d,
                           device=dev)
        lat = cache.run(0).lat
        for s, n in enumerate(lens):
            cache.extend(s, n)
            pos = torch.arange(n)
            pid = cache.page_table[s, (pos // 64).to(dev)].long()
            lat[pid, (pos % 64).to(dev), 0] = rows[s].to(dev, d)
        meta = seqmix.RaggedMeta.build([(s, n - 1, 1) for s, n in enumerate(lens)], cache.page_table, 64, dev)
        res[dev] = seqmix.window_pool_attention(q.to(dev, d).contiguous(), None, lat, lat[..., :kv_rank], None, None, meta,
                                                0.2, window, None).float().cpu()
    tol = 1e-4 if dt == torch.float32 else 2e-2
    assert torch.allclose(res["cuda"], res["cpu"], atol=tol, rtol=tol)


@pytest.mark.gpu
@pytest.mark.parametrize("width,heads,dim,rot,vdim,kvr,qr,dh,dn,dp,ff,E", [(34, 3, 5, 2, 7, 9, 11, 3, 7, 5, 9, 3), (66, 5, 6, 6, 3, 13, 7, 5, 9, 11, 13, 1),
                                                                          (96, 12, 16, 16, 8, 48, 40, 6, 32, 24, 40, 9)])
def test_bf16_odd_sizes(tmp_path, width, heads, dim, rot, vdim, kvr, qr, dh, dn, dp, ff, E):
    """16-bit storage with sizes that are not multiples of 8 (unaligned slices of the fused projections,
    scalar paths of the kernels) and one with aligned sizes, prompt-sized and decode-sized steps: the bulk of
    the rows within 16-bit rounding of the oracle."""
    cfg = make_config(layers=[latent(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=qr, kv_rank=kvr, window=40),
                              delta(heads=dh, kv_heads=dh, dim=dn, vdim=dp, conv=3),
                              latent(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=qr, kv_rank=kvr, window=70, kv_from=0)],
                      mlps=[moe(experts=E, top=min(2, E), ff=ff, shared=ff + 1)] * 3, width=width, vocab=97)
    w = make_weights(cfg, seed=width, decay_rank=5, gate_rank=3)
    model = load(tmp_path, cfg, w, "cuda", precision="bf16")
    toks = tokens(150, cfg["vocab"], 3)
    want = oracle.forward(cfg, w, toks)
    got, _ = replay(model, [[("a", 100)], [("a", 30)]] + [[("a", 1)]] * 20, {"a": toks}, 192)
    e = row_err(got["a"], want)
    assert torch.isfinite(got["a"]).all() and e.median() < 5e-2 and e.quantile(0.9) < 0.3, (e.median(), e.quantile(0.9))


@pytest.mark.gpu
def test_bf16_prompt_sized_experts_against_the_decode_sized_path():
    """The sorted path of prompt-sized steps (bf16: the library's grouped product; an expert that no token
    chose among them) against the per-pair kernels of decode-sized steps."""
    torch.manual_seed(4)
    T, W, E, top, ff = 150, 64, 7, 2, 48
    h = torch.randn(T, W, device="cuda").bfloat16()
    w_gu = (torch.randn(E, 2 * ff, W, device="cuda") * 0.2).bfloat16()
    w_down = (torch.randn(E, W, ff, device="cuda") * 0.2).bfloat16()
    idx = torch.randint(0, E - 1, (T, top), device="cuda", dtype=torch.int32)      # expert E - 1 stays idle
    idx[:, 1] = (idx[:, 0] + 1) % (E - 1)
    big = seqmix.moe_experts(h, idx, w_gu, w_down, 1.5).float()
    small = torch.cat([seqmix.moe_experts(h[a:a + 50].contiguous(), idx[a:a + 50].contiguous(), w_gu, w_down, 1.5)
                       for a in range(0, T, 50)]).float()
    assert torch.allclose(big, small, atol=3e-2, rtol=3e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("T,window,cuts", [(200, 70, (130, 70)), (900, 600, (500, 336, 64)), (500, None, (257, 243))])
@pytest.mark.parametrize("kv_rank,rot_dim,heads", [(96, 32, 4), (128, 64, 16), (24, 8, 3), (128, 32, 4), (256, 64, 8), (512, 64, 2)])
def test_bf16_prompt_attention_over_latent_rows(kv_rank, rot_dim, heads, T, window, cuts):
    """The attention op on bf16 latent rows (value = the first kv_rank numbers of the key row) for prompt
    portions (the matrix-core kernel where it takes the sizes) against the same op in fp32 on the CPU."""
    torch.manual_seed(kv_rank)
    Dc = kv_rank + rot_dim
    q = (torch.randn(T, heads, Dc) * 0.5).bfloat16().float()
    rows = torch.randn(T, Dc).bfloat16().float()
    res = {}
    for dev, dt in (("cpu", torch.float32), ("cuda", torch.bfloat16)):
        spec = _Spec(heads=heads, kv_rank=kv_rank, rot_dim=rot_dim, cache_dim=Dc, kv_from=None)
        cache = PagedCache([_Spec(latent=spec, delta=None, moe=None, attn=None, ssd=None)], 16, slots=3, page=64, dtype=dt,
                           device=dev)
        lat = cache.run(0).lat
        out, at = [], 0
        for n in cuts:
            meta = _meta(cache, [(1, at, n)], dev)
            pos = torch.arange(at, at + n)
            pid = cache.page_table[1, (pos // 64).to(dev)].long()
            lat[pid, (pos % 64).to(dev), 0] = rows[at:at + n].to(dev, dt)
            qq = q[at:at + n].to(dev, dt).contiguous()
            out.append(seqmix.window_pool_attention(qq, None, lat, lat[..., :kv_rank], None, None, meta, 0.2, window,
                                                    None).float().cpu())
            at += n
        res[dev] = torch.cat(out)
    assert torch.allclose(res["cuda"], res["cpu"], atol=3e-2, rtol=3e-2)

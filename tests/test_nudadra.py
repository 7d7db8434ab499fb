"""Nudadra models through the framework (loader, paged cache, ragged engine, scheduler, kernels)
against the plain implementation in ``nudadra_oracle`` (float64, written from the design's
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
import nudadra_oracle as oracle  # noqa: E402

from edgellm.engine.generate import SamplingParams  # noqa: E402
from edgellm.engine.paged import PagedCache  # noqa: E402
from edgellm.engine.ragged import RaggedEngine, RaggedGenerator  # noqa: E402
from edgellm.models.registry import load_model  # noqa: E402
from edgellm.ops import seqmix  # noqa: E402
from edgellm import ops  # noqa: E402

DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def make_config(width=32, vocab=61, n_layers=2, heads=4, kv_heads=2, dim=8, vdim=8, window=6, pool=3, rot_dims=8,
                scaling=True, s_heads=2, s_vdim=8, state=4, groups=1, conv=4, norm_groups=2, ff=40, loop=None,
                per_layer=None):
    layers = []
    for i in range(n_layers):
        left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 1.0 / math.sqrt(dim),
                "mask": {"size": window, "pool": pool} if window else None,
                "rot": {"dims": rot_dims, "base": 100.0,
                        "scaling": {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0} if scaling else None}
                if rot_dims else None}
        right = {"heads": s_heads, "vdim": s_vdim, "state": state, "groups": groups, "conv": conv,
                 "norm_groups": norm_groups}
        l = {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": {"kind": "dense", "ff": ff} if ff else None}
        if per_layer and i in per_layer:
            for side, kv in per_layer[i].items():
                if side == "mlp":
                    l["mlp"] = kv
                else:
                    l["mixer"][side].update(kv)
        layers.append(l)
    cfg = {"architecture": "Nudadra", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": 1e-5},
           "embedding": {"scale": 3.0}}
    if loop:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    bf = lambda t: t.to(torch.bfloat16)
    rn = lambda *s, k=1.0: bf(torch.randn(*s, generator=g) * k)
    w = {"embed": rn(cfg["vocab"], W, k=0.5), "final.norm": bf(torch.tensor(1.1)), "head": rn(cfg["vocab"], W, k=W ** -0.5)}
    if cfg.get("loop"):
        w["loop.in"] = rn(W, 2 * W, k=(2 * W) ** -0.5)
        w["loop.step"] = rn(cfg["loop"]["times"], W, k=0.3)
    for i, l in enumerate(cfg["layers"]):
        a, r, p = l["mixer"]["left"], l["mixer"]["right"], f"l{i}."
        w[p + "norm1"] = bf(torch.tensor(0.9 + 0.05 * i))
        for nm, rows in (("q", a["heads"] * a["dim"]), ("k", a["kv_heads"] * a["dim"]), ("v", a["kv_heads"] * a["vdim"]),
                         ("g", a["heads"])):
            w[p + "mix.left." + nm] = rn(rows, W, k=W ** -0.5)
        w[p + "mix.left.o"] = rn(W, a["heads"] * a["vdim"], k=(a["heads"] * a["vdim"]) ** -0.5)
        inner = r["heads"] * r["vdim"]
        ch = inner + 2 * r["groups"] * r["state"]
        w[p + "mix.right.in"] = rn(2 * inner + 2 * r["groups"] * r["state"] + r["heads"], W, k=W ** -0.5)
        w[p + "mix.right.conv"] = rn(ch, r["conv"], k=0.5)
        w[p + "mix.right.conv.b"] = rn(ch, k=0.2)
        w[p + "mix.right.dt_bias"] = rn(r["heads"], k=0.5)
        w[p + "mix.right.A_log"] = bf(torch.rand(r["heads"], generator=g) - 0.5)
        w[p + "mix.right.D"] = rn(r["heads"])
        w[p + "mix.right.norm"] = bf(1.0 + 0.2 * torch.randn(inner, generator=g))
        w[p + "mix.right.o"] = rn(W, inner, k=inner ** -0.5)
        w[p + "mix.left.out"] = bf(1.0 + 0.2 * torch.randn(W, generator=g))
        w[p + "mix.right.out"] = bf(1.0 + 0.2 * torch.randn(W, generator=g))
        if l["mlp"]:
            w[p + "mlp.up"] = rn(l["mlp"]["ff"], W, k=W ** -0.5)
            w[p + "mlp.down"] = rn(W, l["mlp"]["ff"], k=l["mlp"]["ff"] ** -0.5)
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


def replay(model, schedule, reqs, max_tokens, slots=4):
    """``schedule``: steps of [(request name, token count)]; every row's logits are collected.
    A request ends (slot and pages given back) with its last token."""
    eng = RaggedEngine(model, max_tokens, slots=slots)
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
    d = (got.double() - want)
    scale = want.std().item()
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt().max().item() / scale < tol


TOL = {"fp32": 2e-5, "bf16": 6e-2}


# --------------------------------------------------------------------------- mechanisms alone
def test_yarn_table_matches_the_blend():
    rot = {"dims": 12, "base": 50.0, "scaling": {"factor": 6.0, "original": 32, "fast": 4.0, "slow": 0.5}}
    f, mult = oracle.rotary_frequencies(rot)
    tab = ops.rope_tables(12, 40, 50.0, dict(rot["scaling"], rope_type="yarn")).double()
    pos = torch.arange(40, dtype=torch.float64)
    assert torch.allclose(tab[..., 0], torch.cos(pos[:, None] * f) * mult, atol=1e-6)
    assert torch.allclose(tab[..., 1], torch.sin(pos[:, None] * f) * mult, atol=1e-6)
    assert not torch.allclose(f, oracle.rotary_frequencies({"dims": 12, "base": 50.0})[0])


def _meta(cache, seqs, dev):
    for slot, start, n in seqs:
        cache.extend(slot, start + n)
    return seqmix.RaggedMeta.build(seqs, cache.page_table, cache.page, dev)


class _Spec:
    def __init__(self, **kw):
        self.__dict__.update(kw)


def _attn_cache(G, D, Dv, window, pool, pages, dev, dtype=torch.float32, page=64, Hs=1):
    a = _Spec(kv_heads=G, dim=D, vdim=Dv, window=window, pool=pool)
    m = _Spec(conv=2, conv_channels=1, heads=Hs, state=1, vdim=1)
    return PagedCache([_Spec(attn=a, ssd=m)], pages, slots=3, page=page, dtype=dtype, device=dev)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("window,pool,H,G,D,Dv,page", [(5, 2, 4, 2, 6, 4, 64), (7, 3, 3, 1, 8, 10, 8), (None, None, 2, 2, 4, 4, 64),
                                                       (9, 1, 6, 3, 4, 6, 16), (4, 9, 2, 1, 16, 8, 8)])
def test_attention_op_portions_and_a_far_key(dev, window, pool, H, G, D, Dv, page):
    """The op alone, fed in portions of 1..7 tokens into slot 2, with one early key and one query
    scaled so that a single score dominates: the far key is seen only through its block's mean."""
    torch.manual_seed(1)
    T = 41
    q, k, v = torch.randn(T, H, D, dtype=torch.float64), torch.randn(T, G, D, dtype=torch.float64), torch.randn(T, G, Dv, dtype=torch.float64)
    k[3] *= 4.0
    q[T - 2] = k[3, 0] * 1.5                                  # the late query looks for position 3
    v[3] += 5.0
    want = oracle.window_pool_attention(q, k, v, 0.3, window, pool)
    cache = _attn_cache(G, D, Dv, window, pool, 24, dev, page=page)
    slot, other = 2, 0
    run = cache.run(0)
    proj = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).float().to(dev)
    out, at, n = [], 0, 1
    meta = _meta(cache, [(other, 0, 5)], dev)                  # another sequence takes the first pages
    seqmix.rope_paged_write(torch.randn(5, proj.shape[1], device=dev), meta, None, run.k, run.v, H, 0)
    while at < T:
        n = min(n, T - at)
        meta = _meta(cache, [(slot, at, n)], dev)
        qq = seqmix.rope_paged_write(proj[at:at + n], meta, None, run.k, run.v, H, 0)
        if window and pool:
            seqmix.pool_blocks(run.k, run.v, run.k_pool, run.v_pool, meta, pool)
        out.append(seqmix.window_pool_attention(qq, None, run.k, run.v, run.k_pool, run.v_pool, meta, 0.3, window,
                                                pool if window else None))
        at += n
        n = n % 7 + 1
    got = torch.cat(out).cpu().double().view(T, H, Dv)
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-4)
    if window and pool and pool <= 4:
        # the far key matters: without the pooled blocks the late query's output differs
        assert not torch.allclose(want[T - 2], oracle.window_pool_attention(q, k, v, 0.3, window, None)[T - 2], atol=1e-2)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("Hs,P,N,groups,taps,sizes", [
    (2, 4, 3, 1, 4, (1, 2, 3, 4, 5)), (4, 8, 16, 2, 2, (1, 2, 3, 4, 5)), (3, 5, 20, 3, 5, (1, 2, 3, 4, 5)),
    (1, 70, 33, 1, 3, (1, 2, 3, 4, 5)), (2, 70, 67, 2, 4, (64, 1, 33, 65, 2, 130)), (3, 16, 8, 1, 3, (40, 100, 7)),
    (8, 8, 8, 1, 4, (1, 2, 3, 4, 5)), (8, 8, 8, 1, 4, (40, 100, 7)), (8, 8, 8, 1, 4, (1030, 70, 5)),
    (3, 5, 20, 3, 5, (1030, 70, 5))])
def test_state_space_ops_in_portions(dev, Hs, P, N, groups, taps, sizes):
    """Convolution tail and state matrix carried over portions of ``sizes`` tokens (short ones step
    token by token, long ones take the chunked form; chunk borders inside and at the end of a
    portion), two sequences interleaved in the same steps, against one pass of the oracle over each
    whole sequence."""
    torch.manual_seed(2)
    inner, C = Hs * P, Hs * P + 2 * groups * N
    Ts = {0: 23, 2: 17} if max(sizes) < 10 else ({0: 300, 2: 171} if max(sizes) < 1000 else {0: 1105, 2: 171})
    u = {s: torch.randn(T, 2 * inner + 2 * groups * N + Hs, dtype=torch.float64) for s, T in Ts.items()}
    cw, cb = torch.randn(C, taps, dtype=torch.float64) * 0.5, torch.randn(C, dtype=torch.float64) * 0.2
    dtb, A_log, Dp = torch.randn(Hs, dtype=torch.float64), torch.rand(Hs, dtype=torch.float64) - 0.5, torch.randn(Hs, dtype=torch.float64)
    nw = 1 + 0.1 * torch.randn(inner, dtype=torch.float64)
    want = {}
    for s, T in Ts.items():
        xbc = oracle.silu(oracle.causal_conv(u[s][:, inner:inner + C], cw, cb))
        y = oracle.ssd_scan(xbc[:, :inner].view(T, Hs, P), xbc[:, inner:inner + groups * N].view(T, groups, N),
                            xbc[:, inner + groups * N:].view(T, groups, N), oracle.softplus(u[s][:, inner + C:] + dtb),
                            A_log, Dp, groups).reshape(T, inner)
        want[s] = oracle.group_norm(y * oracle.silu(u[s][:, :inner]), nw, Hs, 1e-5)
    f = lambda t: t.float().to(dev)
    conv = torch.full((3, max(taps - 1, 1), C), 7.0, device=dev)       # stale rows of an earlier tenant
    ssm = torch.full((3, Hs, N, P), -3.0, device=dev)
    at, got, k = {s: 0 for s in Ts}, {s: [] for s in Ts}, 0
    pt = torch.zeros(3, 4, dtype=torch.int32, device=dev)
    while any(at[s] < Ts[s] for s in Ts):
        n = sizes[k % len(sizes)]
        k += 1
        seqs = [(s, at[s], min(n + (s == 2), Ts[s] - at[s])) for s in Ts if at[s] < Ts[s]]
        meta = seqmix.RaggedMeta.build(seqs, pt, 64, dev)
        uu = f(torch.cat([u[s][a:a + m] for s, a, m in seqs]))
        xbc = seqmix.conv_silu(uu, inner, C, f(cw), f(cb), conv, meta)
        y = seqmix.ssd_scan(xbc, uu, inner + C, f(dtb), f(A_log), f(Dp), ssm, meta, Hs, P, N, groups)
        o = seqmix.gated_group_norm(y, uu[:, :inner], f(nw), Hs, 1e-5, torch.float32).cpu().double()
        off = 0
        for s, a, m in seqs:
            got[s].append(o[off:off + m])
            off += m
            at[s] += m
    for s in Ts:
        g = torch.cat(got[s])
        # fp32 sums regrouped per 64-token chunk against float64: the error grows with the state's size
        err = ((g - want[s]).abs() / (1.0 + want[s].abs())).max().item()
        assert err < (3e-5 if max(sizes) < 1000 else 1e-4), (s, err)


@pytest.mark.parametrize("dev", DEVS)
def test_norms_and_combine(dev):
    torch.manual_seed(3)
    T, W = 5, 37
    x, l, r, e = (torch.randn(T, W, dtype=torch.float64) * 2 for _ in range(4))
    wl, wr = torch.randn(W, dtype=torch.float64), torch.randn(W, dtype=torch.float64)
    f = lambda t: t.float().to(dev)
    y = seqmix.scalar_rms_norm(f(x), torch.tensor([1.3], device=dev), 1e-3, torch.float32)
    assert torch.allclose(y.cpu().double(), oracle.scalar_norm(x, 1.3, 1e-3), atol=1e-5)
    want = x + 0.5 * (oracle.rms(l, 1e-3) * wl + oracle.rms(r, 1e-3) * wr) + e
    got = seqmix.combine_residual(f(x), f(l), f(r), f(wl), f(wr), 1e-3, f(e))
    assert torch.allclose(got.cpu().double(), want, atol=2e-5)
    u = f(torch.cat([x, l], 1))
    assert torch.allclose(seqmix.relu2(u, W, W).cpu().double(), torch.relu(l.float().double()) ** 2, atol=1e-5)
    assert torch.equal(seqmix.cat_cast(f(x), f(l), torch.float32).cpu(), torch.cat([x, l], 1).float())
    emb = torch.randn(11, W).to(torch.bfloat16)
    ids = torch.tensor([3, 0, 10], device=dev)
    assert torch.equal(seqmix.embedding_scaled(ids, emb.to(dev), 4.0).cpu(), emb[ids.cpu()].float() * 4.0)


# --------------------------------------------------------------------------- whole models
CONFIGS = {
    "loop": dict(n_layers=3, loop=(1, 3, 2)),
    "plain": dict(n_layers=2, kv_heads=4, norm_groups=1, groups=2, s_heads=4, state=3, ff=None, rot_dims=4, vdim=12, conv=2),
    "mixed": dict(n_layers=3, loop=(0, 2, 3), scaling=False, pool=1, window=4,
                  per_layer={1: {"left": {"heads": 2, "kv_heads": 1, "dim": 16, "vdim": 4, "scale": 0.2,
                                          "mask": {"size": 9, "pool": 4}, "rot": None},
                                 "right": {"heads": 1, "vdim": 24, "state": 9, "groups": 1, "conv": 3, "norm_groups": 3},
                                 "mlp": None},
                             2: {"left": {"mask": None}}}),
}


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompt_decode_and_portions_match_the_oracle(tmp_path, dev, name):
    """One request three ways (whole prompt; a prompt then token-by-token decoding; portions of
    2..9 tokens then single tokens), plus the residual stream after every layer run."""
    cfg = make_config(**CONFIGS[name])
    w = make_weights(cfg, seed=5)
    model = load(tmp_path, cfg, w, dev)
    toks = tokens(45, cfg["vocab"], 6)
    col = []
    want = oracle.forward(cfg, w, toks, col)
    whole, _ = replay(model, [[("a", 45)]], {"a": toks}, 64)
    assert close(whole["a"], want, TOL["fp32"])
    dec, _ = replay(model, [[("a", 11)]] + [[("a", 1)]] * 34, {"a": toks}, 64)
    assert close(dec["a"], want, TOL["fp32"])
    cuts, left, n = [], 40, 2
    while left:
        cuts.append(min(n, left))
        left -= cuts[-1]
        n = n % 9 + 2
    por, _ = replay(model, [[("a", c)] for c in cuts] + [[("a", 1)]] * 5, {"a": toks}, 64)
    assert close(por["a"], want, TOL["fp32"])
    eng = RaggedEngine(model, 64)
    taps = []
    eng.step([("a", toks, [])], taps)
    assert len(taps) == len(col)
    for a, b in zip(taps, col):
        assert torch.allclose(a.cpu().double(), b, atol=2e-4, rtol=1e-4)


@pytest.mark.parametrize("dev", DEVS)
def test_mixed_batches_reuse_pages_and_slots(tmp_path, dev):
    """Five unequal requests through two slots' worth of pages: portions beside single tokens, a
    request paused for a step, slots and pages handed on to later requests.  Page size 64 with
    requests up to 150 tokens crosses page borders inside prompts and while decoding."""
    cfg = make_config(n_layers=2, loop=(0, 1, 2), window=70, pool=8)
    w = make_weights(cfg, seed=7)
    model = load(tmp_path, cfg, w, dev)
    reqs = {"a": tokens(150, cfg["vocab"], 1), "b": tokens(3, cfg["vocab"], 2), "c": tokens(66, cfg["vocab"], 3),
            "d": tokens(1, cfg["vocab"], 4), "e": tokens(130, cfg["vocab"], 5)}
    want = {r: oracle.forward(cfg, w, t) for r, t in reqs.items()}
    sched = [[("a", 60), ("b", 2), ("d", 1)], [("a", 5), ("b", 1), ("c", 64)], [("c", 1), ("a", 62)],
             [("a", 1), ("c", 1), ("e", 63)], [("e", 2), ("a", 20)], [("e", 64), ("a", 1)], [("a", 1), ("e", 1)]]
    got, eng = replay(model, sched, reqs, max_tokens=3 * 64 + 3 * 64, slots=3)
    for r in reqs:
        assert close(got[r], want[r], TOL["fp32"]), r
    assert eng.cache.stats()["free_pages"] == eng.cache.num_pages and eng.cache.stats()["free_slots"] == 3
    alone, _ = replay(model, [[("e", 130)]], {"e": reqs["e"]}, 192)
    assert close(got["e"], alone["e"].double(), 1e-5)


@pytest.mark.parametrize("dev", DEVS)
def test_window_and_block_edges_with_planted_keys(tmp_path, dev):
    """Window 8, blocks of 4: the queries right at the edges (a key just inside / just outside
    the window, a block just complete / not yet seen) in a prompt and while decoding.  The key
    projection of one early token is enlarged so that losing or keeping it moves the logits."""
    cfg = make_config(n_layers=1, window=8, pool=4, heads=2, kv_heads=1, ff=None)
    w = make_weights(cfg, seed=9)
    w["l0.mix.left.k"] = (w["l0.mix.left.k"].float() * 3).to(torch.bfloat16)
    w["l0.mix.left.v"] = (w["l0.mix.left.v"].float() * 3).to(torch.bfloat16)
    model = load(tmp_path, cfg, w, dev)
    toks = tokens(30, cfg["vocab"], 10)
    want = oracle.forward(cfg, w, toks)
    other = oracle.forward(dict(cfg, layers=[dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"], left=dict(
        cfg["layers"][0]["mixer"]["left"], mask={"size": 9, "pool": 4})))]), w, toks)
    assert not close(other[9:], want[9:], 1e-3)                # a window one token off shows
    for cut in (7, 8, 9, 11, 12, 13):
        got, _ = replay(model, [[("a", cut)]] + [[("a", 1)]] * (30 - cut), {"a": toks}, 64)
        assert close(got["a"], want, TOL["fp32"]), cut


@pytest.mark.parametrize("dev", DEVS)
def test_bf16_model_and_long_decoding(tmp_path, dev):
    """The 16-bit model against the oracle within rounding, 120 decoded tokens after a short prompt
    (the recurrent state and the pooled blocks carry everything older than the window)."""
    cfg = make_config(n_layers=2, loop=(1, 2, 2), window=16, pool=4)
    w = make_weights(cfg, seed=11)
    model = load(tmp_path, cfg, w, dev, precision="bf16")
    assert model.dtype == torch.bfloat16
    toks = tokens(128, cfg["vocab"], 12)
    want = oracle.forward(cfg, w, toks)
    got, _ = replay(model, [[("a", 8)]] + [[("a", 1)]] * 120, {"a": toks}, 128)
    assert close(got["a"], want, TOL["bf16"])
    m32 = load(tmp_path, cfg, w, dev)
    got32, _ = replay(m32, [[("a", 8)]] + [[("a", 1)]] * 120, {"a": toks}, 128)
    assert close(got32["a"], want, TOL["fp32"])


@pytest.mark.parametrize("dev", DEVS)
def test_greedy_generation_through_scheduler_and_server(tmp_path, dev):
    """Greedy tokens from ``RaggedGenerator.generate`` (more prompts than slots, chunked prompts)
    and from the serving engine's continuous loop equal the oracle's argmax continuation."""
    cfg = make_config(n_layers=2, loop=(0, 2, 2), window=12, pool=3)
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
    sp = SamplingParams(max_new_tokens=new, do_sample=False, repetition_penalty=1.0)
    res = gen.generate(prompts, sp)
    for g, x in zip(res.tokens, want):
        assert x is None or g == x
    assert gen.kv.stats()["free_pages"] == gen.kv.num_pages
    from edgellm.serve.server import ServingEngine
    from edgellm.utils.tokenizer import ByteTokenizer
    srv = ServingEngine(gen, ByteTokenizer(259), max_batch=2)
    try:
        futs = [srv.submit(p, sp) for p in prompts]
        for f, x in zip(futs, want):
            assert x is None or f.result(timeout=120)["tokens"] == x
    finally:
        srv.close()


@pytest.mark.gpu
def test_decode_graph_replays_match_eager(tmp_path):
    """Decode steps through the captured graph (replayed many times, host work and other eager
    steps between the replays, batch sizes changing) equal the same steps run eagerly."""
    cfg = make_config(n_layers=2, loop=(0, 2, 2), window=12, pool=3, width=64, heads=4, kv_heads=1, dim=16, vdim=8)
    w = make_weights(cfg, seed=21)
    outs = {}
    for graphs in (False, True):
        model = load(tmp_path, cfg, w, "cuda", precision="bf16")
        eng = RaggedEngine(model, 4 * 128, slots=4, use_graphs=graphs)
        reqs = {r: tokens(90, cfg["vocab"], 30 + i) for i, r in enumerate("abc")}
        got = []
        got.append(eng.step([("a", reqs["a"][:20], [19]), ("b", reqs["b"][:3], [2])]).cpu())
        at = {"a": 20, "b": 3, "c": 0}
        for k in range(40):
            live = ["a", "b"] if k < 10 or k > 25 else ["a", "b", "c"]
            if k == 10:
                got.append(eng.step([("c", reqs["c"][:7], [6])]).cpu())
                at["c"] = 7
            got.append(eng.step([(r, [reqs[r][at[r]]], [0]) for r in live]).cpu())
            for r in live:
                at[r] += 1
        assert eng.graphs_used == graphs
        outs[graphs] = torch.cat(got)
    assert torch.allclose(outs[True], outs[False], atol=2e-2, rtol=2e-2)
    assert (outs[True] - outs[False]).abs().max() < 0.05


@pytest.mark.gpu
@pytest.mark.parametrize("window,pool,H,G,D,Dv", [(40, 8, 4, 2, 32, 32), (100, 16, 2, 1, 64, 64), (None, None, 2, 2, 32, 32),
                                                  (70, 3, 3, 1, 96, 96), (33, 70, 2, 2, 128, 64), (300, 2, 4, 2, 32, 32), (64, 8, 8, 2, 32, 32), (50, 4, 4, 1, 64, 64)])
def test_attention_bf16_prompt_kernel(window, pool, H, G, D, Dv):
    """The matrix-core prompt kernel (bf16 portions of 16 tokens or more): two sequences in the
    same steps, portions that start and end inside pages, a planted far key, against the oracle on
    the bf16-rounded inputs; decode-sized steps in between take the general kernel."""
    dev = "cuda"
    torch.manual_seed(4)
    Ts = {0: 333, 2: 150}
    rnd = lambda *s: torch.randn(*s).to(torch.bfloat16).double()
    data, want = {}, {}
    for s, T in Ts.items():
        q, k, v = rnd(T, H, D), rnd(T, G, D), rnd(T, G, Dv)
        k[5] = (k[5] * 3).to(torch.bfloat16).double()
        q[T - 3] = (k[5, 0] * 0.5).to(torch.bfloat16).double()
        v[5] = (v[5] + 4).to(torch.bfloat16).double()
        data[s] = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).to(torch.bfloat16).to(dev)
        want[s] = oracle.window_pool_attention(q, k, v, D ** -0.5, window, pool)
    cache = _attn_cache(G, D, Dv, window, pool, 12, dev, dtype=torch.bfloat16)
    run = cache.run(0)
    sizes, at, got, kk = (70, 1, 64, 17, 2, 130, 16), {s: 0 for s in Ts}, {s: [] for s in Ts}, 0
    while any(at[s] < Ts[s] for s in Ts):
        n = sizes[kk % len(sizes)]
        kk += 1
        seqs = [(s, at[s], min(n + 3 * (s == 2), Ts[s] - at[s])) for s in Ts if at[s] < Ts[s]]
        meta = _meta(cache, seqs, dev)
        proj = torch.cat([data[s][a:a + m] for s, a, m in seqs])
        qq = seqmix.rope_paged_write(proj, meta, None, run.k, run.v, H, 0)
        if window and pool:
            seqmix.pool_blocks(run.k, run.v, run.k_pool, run.v_pool, meta, pool)
        o = seqmix.window_pool_attention(qq, None, run.k, run.v, run.k_pool, run.v_pool, meta, D ** -0.5, window,
                                         pool if window else None).cpu().double()
        off = 0
        for s, a, m in seqs:
            got[s].append(o[off:off + m])
            off += m
            at[s] += m
    for s, T in Ts.items():
        g = torch.cat(got[s]).view(T, H, Dv)
        assert torch.allclose(g, want[s], atol=3e-2, rtol=3e-2), (s, (g - want[s]).abs().max())


def test_evaluate_cli_runs_a_nudadra_checkpoint(tmp_path):
    """The evaluation command line on a checkpoint folder of this design (vocabulary wide enough
    for the byte tokenizer): loader by config.json, paged engine, the reference's sampling
    configuration, the confidence metric through the model's own prompt pass."""
    from safetensors.torch import save_file
    from edgellm.cli import evaluate
    cfg = make_config(vocab=300, n_layers=2, loop=(1, 2, 2), window=20, pool=4)
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


def _random_config(seed):
    import random
    r = random.Random(seed)
    kv = r.choice([1, 2, 3])
    heads = kv * r.choice([1, 2, 4])
    dim = r.choice([4, 8, 12, 16, 32])
    s_heads = r.choice([1, 2, 4])
    groups = r.choice([g for g in (1, 2, 4) if s_heads % g == 0])
    s_vdim = r.choice([4, 8, 12])
    n_layers = r.choice([1, 2, 3])
    loop = None
    if r.random() < 0.6:
        a = r.randrange(0, n_layers)
        loop = (a, r.randrange(a + 1, n_layers + 1), r.choice([1, 2, 3]))
    return make_config(width=r.choice([24, 40, 64]), vocab=r.choice([37, 64, 101]), n_layers=n_layers, heads=heads,
                       kv_heads=kv, dim=dim, vdim=r.choice([dim, 8, 20]), window=r.choice([3, 5, 16, 33, None]),
                       pool=r.choice([1, 2, 5, 8]), rot_dims=r.choice([0, dim, dim // 2]), scaling=r.random() < 0.5,
                       s_heads=s_heads, s_vdim=s_vdim, state=r.choice([1, 4, 7, 16]), groups=groups,
                       conv=r.choice([1, 2, 3, 4, 6]), norm_groups=r.choice([g for g in (1, 2, 4) if (s_heads * s_vdim) % g == 0]),
                       ff=r.choice([None, 16, 56]), loop=loop)


@pytest.mark.parametrize("dev", DEVS)
@pytest.mark.parametrize("seed", range(8))
def test_random_geometries(tmp_path, dev, seed):
    """Sizes drawn at random (head counts and ratios, key / value sizes, windows, pools, rotation
    share, state sizes, taps, norm groups, loops, missing feed-forward): a prompt in portions with
    token-by-token decoding and a second request beside it, against the oracle."""
    cfg = _random_config(100 + seed)
    w = make_weights(cfg, seed=seed)
    model = load(tmp_path, cfg, w, dev)
    reqs = {"a": tokens(50, cfg["vocab"], seed), "b": tokens(21, cfg["vocab"], seed + 50)}
    want = {r: oracle.forward(cfg, w, t) for r, t in reqs.items()}
    sched = [[("a", 17)], [("a", 2), ("b", 20)], [("a", 18), ("b", 1)]] + [[("a", 1)]] * 13
    got, _ = replay(model, sched, reqs, 128, slots=2)
    for r in reqs:
        assert close(got[r], want[r], TOL["fp32"]), (r, cfg)


@pytest.mark.gpu
@pytest.mark.parametrize("dim,heads,kv", [(32, 2, 1), (64, 4, 2)])
def test_bf16_model_on_the_matrix_core_prompt_kernel(tmp_path, dim, heads, kv):
    """A bf16 model whose head sizes the matrix-core prompt kernel takes: prompts in portions of 16+
    tokens (that kernel) and decoded tokens (the general kernel) agree with the oracle within rounding."""
    cfg = make_config(width=64, n_layers=2, loop=(1, 2, 2), heads=heads, kv_heads=kv, dim=dim, vdim=dim, rot_dims=dim,
                      window=48, pool=8, s_heads=2, s_vdim=16, state=8, ff=64)
    w = make_weights(cfg, seed=31)
    model = load(tmp_path, cfg, w, "cuda", precision="bf16")
    reqs = {"a": tokens(200, cfg["vocab"], 1), "b": tokens(90, cfg["vocab"], 2)}
    want = {r: oracle.forward(cfg, w, t) for r, t in reqs.items()}
    sched = [[("a", 70), ("b", 33)], [("a", 64), ("b", 1)], [("a", 50), ("b", 40)]] + [[("a", 1), ("b", 1)]] * 16
    got, _ = replay(model, sched, reqs, 512, slots=2)
    for r in reqs:
        assert close(got[r], want[r], TOL["bf16"]), r


def test_trace_runner_program(tmp_path):
    """``bin/trace_run`` as a program: steps on standard input, a flushed ``done <step>`` per step,
    logits files only for steps that want rows (little-endian fp32 [wanted, vocab], entry order),
    requests ended and their slot reused, exit code 0 at end of input."""
    import subprocess
    import numpy as np
    from safetensors.torch import save_file
    cfg = make_config(n_layers=2, loop=(1, 2, 2), window=10, pool=4)
    w = make_weights(cfg, seed=41)
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(cfg))
    save_file(w, str(d / "model.safetensors"))
    a, b, c = tokens(30, cfg["vocab"], 1), tokens(9, cfg["vocab"], 2), tokens(12, cfg["vocab"], 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [0, 19]}, {"id": "b", "tokens": b, "want": [8]}],
              "end": ["b"]},
             {"step": 1, "entries": [{"id": "a", "tokens": a[20:29], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "c", "tokens": c, "want": [11]}, {"id": "a", "tokens": a[29:], "want": [0]}],
              "end": ["a", "c"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(d), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128", "--slots", "2", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32"]
    V = cfg["vocab"]
    wa, wb, wc = (oracle.forward(cfg, w, t) for t in (a, b, c))
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    assert close(g0, torch.stack([wa[0], wa[19], wb[8]]), TOL["fp32"])
    assert close(g2, torch.stack([wc[11], wa[29]]), TOL["fp32"])

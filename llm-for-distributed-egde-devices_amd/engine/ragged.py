"""Ragged-step engine: several sequences per step, prompt portions beside decode tokens.

``RaggedEngine`` is the step function: it owns a ``PagedCache`` sized for the tokens alive at
one time, maps request ids to state slots, and runs one model call per step over whatever each
request brings (a whole prompt, a cut of one, one decoded token), returning the logits of the
rows asked for.  Nothing in a step depends on how a prompt was cut or on the other requests
of the batch: every kernel addresses a token by (sequence, position) through the page table.

``RaggedScheduler`` is iteration-level batching on top of it, with the interface the serving
loop drives (``admit`` / ``step`` / ``poll``, as ``engine.continuous.SlotDecoder``): a request is
admitted into a free slot at any step, its prompt is fed in portions of at most
``prefill_chunk`` tokens beside the other requests' decode tokens, the fused sampler draws one
token per sequence whose portion reached its last prompt token, and a finished request gives
its slot and pages back at once.  ``RaggedGenerator`` is the ``Generator`` surface over it
(``generate`` / ``slot_decoder``) for the CLIs and the serving engine.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import ops
from ..ops.seqmix import RaggedMeta
from ..utils.tracing import trace_range
from .generate import GenerationResult, SamplingParams
from .paged import PagedCache


class _DecodeGraph:
    """A captured decode step for ``n`` sequences (one token each): static token / metadata buffers
    filled from pinned host rows before every replay; the first call runs eagerly (lazy weight packs
    and rotary tables are built outside any capture)."""
    RING = 8

    def __init__(self, eng: "RaggedEngine", n: int):
        dev = eng.device
        self.eng, self.n = eng, n
        self.buf = torch.zeros(6 * n, dtype=torch.int32, device=dev)
        self.ids = torch.zeros(n, dtype=torch.long, device=dev)
        self.host = [(torch.zeros(6 * n, dtype=torch.int32).pin_memory(), torch.zeros(n, dtype=torch.long).pin_memory(),
                      torch.cuda.Event()) for _ in range(self.RING)]
        self.turn = 0
        b = self.buf
        cap = eng.cache.num_pages * eng.page
        self.meta = RaggedMeta(n, n, b[0:n], b[n:2 * n], b[2 * n:3 * n], b[3 * n:4 * n], b[4 * n:5 * n], b[5 * n:6 * n],
                               eng.cache.page_table, eng.page, [(0, 1, 1, i) for i in range(n)], 1, cap)
        self.rows = torch.arange(n, dtype=torch.long, device=dev)
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.out: Optional[torch.Tensor] = None
        self.warm = False

    def run(self, seqs, ids) -> torch.Tensor:
        n = self.n
        hb, hi, ev = self.host[self.turn]
        self.turn = (self.turn + 1) % self.RING
        ev.synchronize()                           # the copy that last read this pinned row is done
        flat = [s[0] for s in seqs] + [s[1] for s in seqs] + [1] * n + list(range(n)) + list(range(n)) + \
            [s[1] for s in seqs]
        hb.copy_(torch.tensor(flat, dtype=torch.int32))
        hi.copy_(torch.tensor(ids, dtype=torch.long))
        self.buf.copy_(hb, non_blocking=True)
        self.ids.copy_(hi, non_blocking=True)
        ev.record()
        eng = self.eng
        if not self.warm:
            self.warm = True
            return eng.model(self.ids, self.meta, eng.cache, self.rows)
        if self.graph is None:
            # no cyclic garbage collection while the stream captures: a collected engine of an earlier
            # request frees pinned buffers and graphs, which the runtime refuses during a capture; what
            # is garbage already goes first
            import gc
            gc.collect()
            g = torch.cuda.CUDAGraph()
            torch.cuda.synchronize()
            gc_was_on = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(g, pool=eng._pool):
                    self.out = eng.model(self.ids, self.meta, eng.cache, self.rows)
            except Exception as e:  # noqa: BLE001 - an op that cannot be captured: this engine steps eagerly
                from ..utils.log import get_logger
                get_logger("ragged").warning(f"decode step not graph-capturable ({e!r}): running eagerly")
                torch.cuda.synchronize()
                eng.use_graphs = False
                return eng.model(self.ids, self.meta, eng.cache, self.rows)
            finally:
                if gc_was_on:
                    gc.enable()
            if eng._pool is None:
                eng._pool = g.pool()
            self.graph = g
        self.graph.replay()
        return self.out


class RaggedEngine:
    def __init__(self, model, max_tokens: int, slots: int = 4, page: int = 64, use_graphs: Optional[bool] = None):
        assert getattr(model, "ragged", False), "RaggedEngine runs layer-spec (ragged-step) models"
        self.model, self.cfg, self.device = model, model.cfg, model.device
        self.page = page
        pages = max(1, (int(max_tokens) + page - 1) // page)
        cfg = model.cfg
        self.cache = PagedCache(model.run_specs(), pages, slots, page, dtype=model.dtype, device=self.device,
                                width=cfg.hidden_size, canon_taps=cfg.canon_taps, prev_token=bool(cfg.bigram),
                                run_layers=[i for i, _ in model.runs])
        self.live: Dict[object, int] = {}
        # decode-only steps (every sequence brings one token) replay a HIP graph per batch size
        self.use_graphs = (self.device.type == "cuda" and ops.gpu_path(model.embed)) if use_graphs is None \
            else bool(use_graphs)
        self._graphs: Dict[int, _DecodeGraph] = {}
        self._pool = None
        self.graphs_used = False

    # ------------------------------------------------------------------ requests
    def open(self, rid) -> int:
        assert rid not in self.live, f"request {rid!r} is already live"
        self.live[rid] = self.cache.acquire()
        return self.live[rid]

    def close(self, rid) -> None:
        self.cache.release(self.live.pop(rid))

    def length(self, rid) -> int:
        return self.cache.lens[self.live[rid]]

    def can_open(self) -> bool:
        return bool(self.cache.free_slots)

    # ------------------------------------------------------------------ the step
    @torch.no_grad()
    def step(self, entries: Sequence[Tuple[object, Sequence[int], Sequence[int]]],
             taps: Optional[list] = None) -> torch.Tensor:
        """``entries``: (request id, its next tokens, indices among them whose logits are wanted).
        A request not yet live is opened.  Returns fp32 logits [wanted rows, vocab] in entry order."""
        seqs, ids, rows, off = [], [], [], 0
        for rid, toks, want in entries:
            if len(toks) == 0:
                continue
            slot = self.live[rid] if rid in self.live else self.open(rid)
            start = self.cache.lens[slot]
            self.cache.extend(slot, start + len(toks))
            seqs.append((slot, start, len(toks)))
            ids.extend(toks)
            rows.extend(off + int(w) for w in want)
            off += len(toks)
        if not seqs:
            return torch.empty(0, self.cfg.vocab_size, dtype=torch.float32, device=self.device)
        if self.use_graphs and taps is None and len(ids) == len(seqs):
            dg = self._graphs.get(len(seqs))
            if dg is None:
                dg = self._graphs[len(seqs)] = _DecodeGraph(self, len(seqs))
            with trace_range(f"ragged.decode.n{len(seqs)}"):
                out = dg.run(seqs, ids)
            self.graphs_used = self.graphs_used or dg.graph is not None
            if rows == list(range(len(seqs))):
                return out.clone()
            return out.index_select(0, torch.tensor(rows, dtype=torch.long, device=self.device))
        meta = RaggedMeta.build(seqs, self.cache.page_table, self.page, self.device)
        ids_t = torch.from_numpy(np.asarray(ids, dtype=np.int64))
        rows_t = torch.from_numpy(np.asarray(rows, dtype=np.int64))
        if self.device.type == "cuda":
            ids_t = ids_t.pin_memory().to(self.device, non_blocking=True)
            rows_t = rows_t.pin_memory().to(self.device, non_blocking=True)
        with trace_range(f"ragged.step.n{meta.n}.T{meta.T}"):
            return self.model(ids_t, meta, self.cache, rows_t, taps)


@dataclass
class _Req:
    tag: object
    prompt: List[int]
    max_new: int
    eos: Optional[int]
    fed: int = 0
    tokens: List[int] = field(default_factory=list)
    t0: float = 0.0
    t_first: float = 0.0
    done: bool = False
    row: int = 0                     # admission order
    rid: object = None               # the engine's request id


class RaggedScheduler:
    def __init__(self, engine: RaggedEngine, sampling: SamplingParams, seed: int = 0, prefill_chunk: int = 512,
                 max_step_tokens: int = 2048, max_batch: Optional[int] = None, width: int = 1 << 30):
        self.eng, self.sp = engine, sampling
        self.B = min(int(max_batch), engine.cache.slots) if max_batch else engine.cache.slots
        self.prefill_chunk, self.max_step_tokens = int(prefill_chunk), int(max_step_tokens)
        V = engine.cfg.vocab_size
        self.seen = torch.zeros(engine.cache.slots, V, dtype=torch.uint8, device=engine.device)
        self.rng = torch.zeros(2, dtype=torch.int32, device=engine.device)
        self.rng[0] = seed & 0x7FFFFFFF
        self.reqs: Dict[int, _Req] = {}            # slot -> request
        self.reserved = 0                          # pages promised to admitted requests
        self.col, self.width = 1, width            # session bookkeeping the serving loop reads
        self.steps = 0
        self._n = 0

    # ------------------------------------------------------------------ slots
    @property
    def slots(self) -> List[Optional[_Req]]:
        return [self.reqs.get(s) for s in range(self.eng.cache.slots)]

    def free_slots(self) -> List[int]:
        return list(self.eng.cache.free_slots)[:max(0, self.B - len(self.reqs))]

    def busy(self) -> bool:
        return bool(self.reqs)

    def can_admit(self, prompt_len: int, max_new: int) -> bool:
        c = self.eng.cache
        return bool(self.free_slots()) and \
            c.pages_for(prompt_len + max_new) + self.reserved <= c.num_pages

    def admit(self, ids: Sequence[int], max_new: int, eos: Optional[int] = None, tag=None) -> int:
        assert self.can_admit(len(ids), max_new), "no slot / page room for this request"
        rid = ("sched", id(self), self._n)
        slot = self.eng.open(rid)
        self.seen[slot].zero_()
        self.reqs[slot] = _Req(tag, [int(t) for t in ids], int(max_new), eos, t0=time.perf_counter(), row=self._n,
                               rid=rid)
        self.reserved += self.eng.cache.pages_for(len(ids) + max_new)
        self._n += 1
        return slot

    # ------------------------------------------------------------------ stepping
    @torch.no_grad()
    def step(self, n: int = 1) -> int:
        """``n`` engine steps: every live request brings its next prompt portion or its last
        sampled token.  Stops early once a request finishes (the caller polls)."""
        done = 0
        for _ in range(n):
            entries, sampled, budget = [], [], self.max_step_tokens
            for slot, r in self.reqs.items():
                if r.done:
                    continue
                if r.fed < len(r.prompt):
                    take = min(self.prefill_chunk, len(r.prompt) - r.fed, max(budget, 1))
                    toks = r.prompt[r.fed:r.fed + take]
                    r.fed += take
                    last = r.fed == len(r.prompt)
                    entries.append((r.rid, toks, [take - 1] if last else []))
                    if last:
                        sampled.append(slot)
                else:
                    toks = [r.tokens[-1]]
                    entries.append((r.rid, toks, [0]))
                    sampled.append(slot)
                budget -= len(toks)
            if not entries:
                break
            logits = self.eng.step(entries)
            if sampled:
                self._sample(logits, sampled)
            self.steps += 1
            done += 1
            if any(r.done for r in self.reqs.values()):
                break
        return done

    def _sample(self, logits: torch.Tensor, slots: List[int]) -> None:
        sp = self.sp
        idx = torch.tensor(slots, dtype=torch.long, device=logits.device)
        for s in slots:                                  # prompt tokens count for the repetition penalty
            r = self.reqs[s]
            if not r.tokens:
                self.seen[s, torch.tensor(r.prompt, dtype=torch.long, device=logits.device)] = 1
        seen = self.seen.index_select(0, idx)
        self.rng[1] = self.steps + 1
        nxt = ops.sample(logits, seen, sp.temperature, sp.top_k, sp.top_p, sp.repetition_penalty, self.rng,
                         sp.do_sample)
        self.seen[idx, nxt] = 1
        now = time.perf_counter()
        for s, t in zip(slots, nxt.tolist()):
            r = self.reqs[s]
            if not r.tokens:
                r.t_first = now
            r.tokens.append(int(t))
            if len(r.tokens) >= r.max_new or (r.eos is not None and int(t) == r.eos):
                r.done = True

    def poll(self) -> List[tuple]:
        """Release finished requests: [(tag, GenerationResult)]."""
        out, now = [], time.perf_counter()
        for slot in [s for s, r in self.reqs.items() if r.done]:
            r = self.reqs.pop(slot)
            self.eng.close(r.rid)
            self.reserved -= self.eng.cache.pages_for(len(r.prompt) + r.max_new)
            out.append((r.tag, GenerationResult([r.tokens], [len(r.prompt)], now - r.t0, r.t_first - r.t0,
                                                now - r.t_first, [])))
        return out


class RaggedGenerator:
    """The ``Generator`` surface (``generate``, ``slot_decoder``, ``max_seq``, ``kv.max_batch``) for
    ragged-step models: every call goes through a ``RaggedScheduler``."""

    attn_hook = None
    use_graphs = False

    def __init__(self, model, max_batch: int = 4, max_seq: int = 2048, max_tokens: Optional[int] = None,
                 page: int = 64, prefill_chunk: int = 512):
        self.model, self.cfg, self.device = model, model.cfg, model.device
        self.max_seq = int(max_seq)
        tokens = int(max_tokens) if max_tokens else max_batch * ((self.max_seq + page - 1) // page) * page
        self.engine = RaggedEngine(model, tokens, slots=max_batch, page=page)
        self.kv = self.engine.cache
        self.kv.max_batch = max_batch
        self.prefill_chunk = prefill_chunk

    def slot_decoder(self, sampling: SamplingParams, seed: int = 0, width: int = 1 << 30,
                     max_batch: Optional[int] = None) -> RaggedScheduler:
        return RaggedScheduler(self.engine, sampling, seed, self.prefill_chunk, max_batch=max_batch, width=1 << 30)

    @torch.no_grad()
    def generate(self, prompts: Sequence[Sequence[int]], sampling: SamplingParams, seed: int = 0,
                 eos_token_id: Optional[int] = None, stop_at_eos: bool = True,
                 record_step_latency: bool = True) -> GenerationResult:
        """Every prompt through the scheduler (more prompts than slots queue up and start as
        slots free); tokens come back in prompt order."""
        sched = self.slot_decoder(sampling, seed)
        cuda = self.device.type == "cuda"
        if cuda:
            torch.cuda.synchronize()
        t0 = time.perf_counter()
        queue = list(enumerate(prompts))
        results: Dict[int, GenerationResult] = {}
        step_ms: List[float] = []
        t_first = None
        while queue or sched.busy():
            while queue and sched.can_admit(len(queue[0][1]), sampling.max_new_tokens):
                i, p = queue.pop(0)
                sched.admit(p, sampling.max_new_tokens, eos_token_id if stop_at_eos else None, tag=i)
            if not sched.busy():
                raise RuntimeError("a prompt does not fit the page pool")
            ts = time.perf_counter()
            sched.step(1)
            if record_step_latency:
                step_ms.append((time.perf_counter() - ts) * 1e3)
            for tag, res in sched.poll():
                results[tag] = res
                t_first = t_first or (time.perf_counter() - t0 - res.decode_s)
        if cuda:
            torch.cuda.synchronize()
        el = time.perf_counter() - t0
        pre = min((r.prefill_s for r in results.values()), default=0.0)
        return GenerationResult([results[i].tokens[0] for i in range(len(prompts))], [len(p) for p in prompts], el,
                                pre, el - pre, step_ms)

"""Execution backend for hybrid models (``models.hybrid``): the step function over the
sequence cache, and on top of it the same surface the Llama ``Engine`` offers to the
scheduler and servers (``prefill`` / ``decode_steps`` / ``generate``).

``step`` is the one entry everything goes through: a list of (sequence key, next tokens,
wanted positions).  Unknown keys are admitted (a state slot), pages are reserved as the
sequence grows, the whole list runs as one batch -- portions of prompts beside single
decoded tokens -- and ``release`` hands a sequence's pages and slot back.

When a scheduler owns the pages (``engine.server``: the native ``Scheduler`` allocates them)
``prefill`` / ``decode_steps`` take its block tables; the state slot of such a sequence is
keyed by its first page, which is unique among live sequences, and is handed back by
``release_sequence`` when the scheduler retires the request.
"""
from __future__ import annotations

import os
import time

import torch

from ..models.hybrid import HybridConfig, HybridModel, HybridWeights, StepBatch
from ..ops import PAGE
from .engine import GenResult
from .seq_cache import SequenceCache, layer_specs


DECODE_BUCKETS = (1, 2, 4, 8, 16, 32, 64, 128, 256)


def _bucket(x: int, buckets=DECODE_BUCKETS) -> int:
    for b in buckets:
        if x <= b:
            return b
    return x


class HybridDecodeGraph:
    """One decode step of ``rows`` single-token entries (block tables ``maxp`` pages wide) as
    a captured hipGraph: forward + greedy argmax.  A step loads its metadata into the batch's
    device tensors with one copy and replays; rows beyond the live ones are padding on the
    null page and the null state slot."""

    def __init__(self, model: HybridModel, rows: int, maxp: int):
        self.model, self.rows, self.maxp = model, rows, maxp
        self.pad = (model.cache.null_slot, [0] * maxp, 0, [0])
        self.batch = StepBatch([self.pad] * rows, [[0]] * rows, model.device, min_pages=maxp)
        self.batch.max_keys = maxp * PAGE   # a captured step must not depend on the positions
        self.tokens = torch.zeros(rows, dtype=torch.int32, device=model.device)
        self.logits = None
        self.graph = None

    def _body(self):
        from .. import ops

        self.logits = self.model.forward(self.batch)
        ops.argmax(self.logits, out=self.tokens)

    def capture(self, warmup: int = 2):
        cur = torch.cuda.current_stream(self.model.device)
        side = torch.cuda.Stream(self.model.device)
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            for _ in range(warmup):  # also builds everything a step creates lazily
                self._body()
        cur.wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self._body()
        self.graph = g
        return self

    def step(self, rows: list) -> list:
        """rows: (slot, pages, position, token) per live sequence -> their next tokens."""
        n = len(rows)
        ent = [(s, list(pg) + [0] * (self.maxp - len(pg)), p, [t]) for s, pg, p, t in rows]
        self.batch.reload(ent + [self.pad] * (self.rows - n), [[0]] * self.rows)
        if self.batch.max_pos >= self.model.cfg.max_pos:
            raise ValueError("position %d exceeds the model's %d positions"
                             % (self.batch.max_pos, self.model.cfg.max_pos))
        self.graph.replay()
        return self.tokens[:n].cpu().tolist()


class HybridEngine:
    def __init__(self, cfg: HybridConfig, weights: HybridWeights | None = None, device="cuda",
                 seed: int = 0, kv_pages: int | None = None, max_batch: int = 16,
                 max_prefill_tokens: int = 1024, dtype=torch.bfloat16, num_slots: int | None = None,
                 kv_fraction: float = 0.85, use_graph: bool = True):
        self.cfg = cfg
        self.device = torch.device(device)
        if weights is None:
            weights = HybridWeights.random(cfg, self.device, seed=seed, dtype=dtype)
        self.weights = weights
        self.dtype = weights.dtype
        self.max_batch = max_batch
        self.max_prefill_tokens = max_prefill_tokens
        slots = num_slots or max_batch
        specs = weights.cache_specs()
        if kv_pages is None:
            per_page = max(1, sum(int(what) for _i, kind, what in layer_specs(specs) if kind == "paged")
                           * PAGE * (4 if self.dtype == torch.float32 else 2))
            if self.device.type == "cuda":
                free, _ = torch.cuda.mem_get_info(self.device)
                kv_pages = max(2, int(max(0, free - (4 << 30)) * kv_fraction) // per_page)
                kv_pages = min(kv_pages, 2 + max_batch * (cfg.max_pos + PAGE - 1) // PAGE)
            else:
                kv_pages = 256
        self.cache = self.kv = SequenceCache(specs, kv_pages, slots, self.device, self.dtype)
        self.model = HybridModel(weights, self.cache)
        self._page_slot = {}  # first page of a scheduler-owned sequence -> state slot
        # greedy decode steps replay a captured hipGraph per (rows, table width) bucket
        # (P2P_HYBRID_GRAPH=0: every step eager)
        self.use_graph = (use_graph and self.device.type == "cuda"
                          and os.environ.get("P2P_HYBRID_GRAPH", "1") != "0")
        self._graphs = {}

    # ------------------------------------------------------------------ step
    def step(self, entries: list, return_layers=None):
        """entries: (key, tokens, want) per sequence.  Returns fp32 logits
        [sum(len(want)), vocab] in entry order (None when nothing is wanted)."""
        cache, rows, want = self.cache, [], []
        for key, toks, w in entries:
            seq = cache.get(key) if key in cache else cache.open(key)
            cache.reserve(seq, seq.length + len(toks))
            rows.append((seq.slot, seq.pages, seq.length, toks))
            want.append(list(w))
        b = StepBatch(rows, want, self.device)
        logits = self.model.forward(b, return_layers)
        for key, toks, _w in entries:
            cache.get(key).length += len(toks)
        return logits

    def release(self, key):
        self.cache.close(key)

    def decode_graph(self, rows: int, pages: int) -> HybridDecodeGraph:
        key = (_bucket(rows), _bucket(pages))
        g = self._graphs.get(key)
        if g is None:
            g = self._graphs[key] = HybridDecodeGraph(self.model, *key).capture()
        return g

    def _decode_rows(self, rows: list, params, pos) -> list:
        """One token for each of rows = (slot, pages, position, token): the captured graph
        when every row is greedy, else an eager step + the sampler."""
        if self.use_graph and (params is None or all(p.greedy for p in params)):
            return self.decode_graph(len(rows), max(len(r[1]) for r in rows)).step(rows)
        b = StepBatch([(s, pg, p, [t]) for s, pg, p, t in rows], [[0]] * len(rows), self.device)
        return self._pick(self.model.forward(b), params, pos).cpu().tolist()

    # ------------------------------------------------------------------ sampling
    def _pick(self, logits, params, pos):
        from .. import ops
        from .sampling import sample

        if params is None or all(p.greedy for p in params):
            return ops.argmax(logits.contiguous())
        return sample(logits.contiguous(), params, pos)

    # ------------------------------------------------- scheduler-owned pages
    def _slot_for(self, pages, start: int) -> int:
        first = pages[0]
        s = self._page_slot.get(first)
        if s is None or start == 0:
            if s is None:
                s = self._page_slot[first] = self.cache.slots.alloc()
        return s

    def release_sequence(self, pages):
        """The scheduler retired the sequence that owned ``pages``: free its state slot."""
        if pages and pages[0] in self._page_slot:
            self.cache.slots.free(self._page_slot.pop(pages[0]))

    def check_comm(self):
        pass

    def prefill(self, prompts: list, block_tables: list, return_logits: bool = False,
                sampling: list | None = None, starts: list | None = None, **_kw):
        """First tokens (int32 [B], device) of the prompts, run from ``starts`` (a running
        sequence rides along as one row at its last position), in chunks of at most
        ``max_prefill_tokens`` rows; prompts may be cut at a chunk's end."""
        B = len(prompts)
        todo = []
        for bi, p in enumerate(prompts):
            s0 = starts[bi] if starts else 0
            todo.append([bi, s0, len(p)])
        first = torch.zeros(B, dtype=torch.int32, device=self.device)
        all_logits = None
        while todo:
            budget, rows, want, seqs = self.max_prefill_tokens, [], [], []
            while todo and budget > 0:
                bi, s0, end = todo[0]
                n = min(end - s0, budget)
                p = prompts[bi]
                toks = [p[i] for i in range(s0, s0 + n)]
                rows.append((self._slot_for(block_tables[bi], s0), list(block_tables[bi]), s0, toks))
                done = s0 + n == end
                want.append([n - 1] if done else [])
                if done:
                    seqs.append(bi)
                    todo.pop(0)
                else:
                    todo[0][1] = s0 + n
                budget -= n
            logits = self.model.forward(StepBatch(rows, want, self.device))
            if not seqs:
                continue
            params = [sampling[bi] for bi in seqs] if sampling is not None else None
            toks = self._pick(logits, params, [len(prompts[bi]) - 1 for bi in seqs])
            sel = torch.tensor(seqs, dtype=torch.long, device=self.device)
            first.index_copy_(0, sel, toks)
            if return_logits:
                if all_logits is None:
                    all_logits = torch.zeros(B, self.cfg.vocab, dtype=torch.float32, device=self.device)
                all_logits.index_copy_(0, sel, logits)
        return (first, all_logits) if return_logits else first

    def decode_steps(self, last_ids: list, pos: list, block_tables: list, ctx: int, k: int,
                     params: list | None = None, **_kw) -> list:
        """k decode steps of running sequences: row b continues from ``last_ids[b]`` at
        position ``pos[b]``.  Returns each row's k new tokens."""
        ids, hist = list(last_ids), [[] for _ in last_ids]
        for j in range(k):
            rows = [(self._slot_for(block_tables[b], pos[b] + j), list(block_tables[b]), pos[b] + j,
                     ids[b]) for b in range(len(ids))]
            ids = self._decode_rows(rows, params, [p + j for p in pos])
            for b, t in enumerate(ids):
                hist[b].append(int(t))
        return hist

    # ------------------------------------------------------------------ generate
    def generate(self, prompts: list, max_new_tokens: int = 64, stop_on_eos: bool = True,
                 sampling: list | None = None) -> list:
        """Reply to a static batch of prompts (token id lists); greedy unless ``sampling``
        gives per-prompt SamplingParams.  Pages and slots are the engine's own."""
        t0 = time.perf_counter_ns()
        B = len(prompts)
        assert 0 < B <= self.cache.slots.free_slots
        keys = [("gen", time.monotonic_ns(), b) for b in range(B)]
        out = [[] for _ in range(B)]
        try:
            # prompts in portions of max_prefill_tokens rows, last tokens wanted
            pending = [[b, 0] for b in range(B)]
            firsts = {}
            while pending:
                budget, ent, owners = self.max_prefill_tokens, [], []
                while pending and budget > 0:
                    b, s0 = pending[0]
                    n = min(len(prompts[b]) - s0, budget)
                    done = s0 + n == len(prompts[b])
                    ent.append((keys[b], prompts[b][s0:s0 + n], [n - 1] if done else []))
                    if done:
                        owners.append(b)
                        pending.pop(0)
                    else:
                        pending[0][1] = s0 + n
                    budget -= n
                logits = self.step(ent)
                if owners:
                    prm = [sampling[b] for b in owners] if sampling else None
                    toks = self._pick(logits, prm, [len(prompts[b]) - 1 for b in owners]).cpu().tolist()
                    firsts.update(zip(owners, toks))
            t1 = time.perf_counter_ns()
            live = []
            for b in range(B):
                out[b].append(int(firsts[b]))
                if not (stop_on_eos and out[b][0] in self.cfg.eos_ids) and max_new_tokens > 1:
                    live.append(b)
            while live:
                rows = []
                for b in live:
                    seq = self.cache.get(keys[b])
                    self.cache.reserve(seq, seq.length + 1)
                    rows.append((seq.slot, seq.pages, seq.length, out[b][-1]))
                    seq.length += 1
                prm = [sampling[b] for b in live] if sampling else None
                toks = self._decode_rows(rows, prm, [len(prompts[b]) + len(out[b]) - 1 for b in live])
                nxt = []
                for b, t in zip(live, toks):
                    out[b].append(int(t))
                    if len(out[b]) < max_new_tokens and not (stop_on_eos and t in self.cfg.eos_ids):
                        nxt.append(b)
                live = nxt
            t2 = time.perf_counter_ns()
        finally:
            for k_ in keys:
                if k_ in self.cache:
                    self.cache.close(k_)
        res = []
        for b in range(B):
            toks, reason = out[b][:max_new_tokens], "length"
            if stop_on_eos and toks and toks[-1] in self.cfg.eos_ids:
                toks, reason = toks[:-1], "stop"
            res.append(GenResult(tokens=toks, prompt_eval_count=len(prompts[b]),
                                 prompt_eval_duration_ns=t1 - t0, eval_count=len(toks),
                                 eval_duration_ns=t2 - t1, total_duration_ns=t2 - t0,
                                 ttft_ns=t1 - t0, done_reason=reason))
        return res

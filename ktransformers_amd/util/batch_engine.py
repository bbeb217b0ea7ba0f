"""Step function and scheduler for batches of requests over a KHybridCache (models/custom_cache.py).

`BatchEngine.step(entries, end)` is the one place a batch of unequal requests meets the model: it admits new requests (a state
slot and pages from the cache's free lists), plans the step's ForwardBatch, runs the model's forward on the flattened tokens and
gives finished requests' pages and slot back.  A step runs only the tokens it brings — a whole prompt, a portion of one, or one
decoded token per request — from the cache and state earlier steps left.  `generate()` is the batched generation loop on top of
it (prompts of different lengths in one prefill step, then one token per live request per step; requests leave the batch when
they finish) with the sampling of util/generate.py."""
from __future__ import annotations

import torch

from ktransformers_amd.util.generate import sample_next_token


class _DecodeGraph:
    """One captured decode step (one token per request) for a batch of B requests: the step's metadata lives in ONE static int32
    device buffer whose slices are the ForwardBatch's tensors; a step fills a pinned host copy, sends it with one transfer and
    replays.  Valid while B, the page-list capacity, the key-range split and the cache's tensors stay what they were."""
    FIELDS = ("tokens", "positions", "tok_req", "cache_loc", "pos0", "slot", "q_indptr", "page_indptr", "page_indices")

    def __init__(self, engine, B: int, page_cap: int, nsplit: int, max_kv_len: int):
        from ktransformers_amd.models.custom_cache import ForwardBatch
        self.B, self.page_cap, self.nsplit = B, page_cap, nsplit
        sizes = dict(tokens=B, positions=B, tok_req=B, cache_loc=B, pos0=B, slot=B, q_indptr=B + 1, page_indptr=B + 1, page_indices=page_cap)
        self.offsets, at = {}, 0
        for k in self.FIELDS:
            self.offsets[k] = (at, sizes[k])
            at += (sizes[k] + 3) // 4 * 4                 # 16-byte aligned slices
        dev = engine.device
        self.host = torch.zeros(at, dtype=torch.int32, pin_memory=True)
        self.meta = torch.zeros(at, dtype=torch.int32, device=dev)
        v = {k: self.meta[o:o + n] for k, (o, n) in self.offsets.items()}
        self.tokens = v["tokens"]
        self.batch = ForwardBatch(T=B, B=B, max_q_len=1, max_kv_len=max_kv_len, nsplit=nsplit,
                                  **{k: v[k] for k in self.FIELDS if k != "tokens"})
        self.graph, self.logits = None, None

    def fill(self, d: dict, tokens) -> None:
        h = self.host
        for k in self.FIELDS:
            o, n = self.offsets[k]
            vals = tokens if k == "tokens" else d[k]
            h[o:o + len(vals)] = torch.tensor(vals, dtype=torch.int32)
        self.meta.copy_(h, non_blocking=True)

    def capture(self, engine) -> None:
        cache, model, dev = engine.cache, engine.model, engine.device
        # the warm-up runs advance the recurrent state of the batch's slots: put it back afterwards (appending the same key rows
        # again changes nothing)
        keep = [(t, t.clone()) for t in cache.state_tensors()]
        stream = torch.cuda.Stream(device=dev)
        stream.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(stream):
            for _ in range(2):
                model(self.tokens, None, cache, batch=self.batch)
        torch.cuda.current_stream(dev).wait_stream(stream)
        torch.cuda.synchronize(dev)
        for t, saved in keep:
            t.copy_(saved)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=stream):
            self.logits = model(self.tokens, None, cache, batch=self.batch)
        torch.cuda.synchronize(dev)


class BatchEngine:
    def __init__(self, model, cache, use_graph: bool = False):
        """use_graph: steps that bring exactly one token for every request (decode steps) replay a captured HIP graph."""
        self.model, self.cache = model, cache
        self.device = cache.device
        self.use_graph = use_graph
        self._graphs: dict = {}
        self._graph_generation = cache.generation

    def _decode_graph_step(self, plan, tokens, rows):
        d = self.cache.plan_lists(plan)
        if self._graph_generation != self.cache.generation:          # the cache re-allocated its tensors
            self._graphs.clear()
            self._graph_generation = self.cache.generation
        B = d["B"]
        page_cap = (len(d["page_indices"]) + 63) // 64 * 64
        kv_bucket = (d["max_kv_len"] + 1023) // 1024 * 1024
        nsplit = max(1, min(1024 // B, kv_bucket // 128))
        key = (B, page_cap, nsplit)
        g = self._graphs.get(key)
        fresh = g is None
        if fresh:
            g = self._graphs[key] = _DecodeGraph(self, B, page_cap, nsplit, kv_bucket)
        g.fill(d, tokens)
        if fresh:
            g.capture(self)
        g.graph.replay()
        return g.logits[torch.tensor(rows, dtype=torch.long, device=self.device)] if rows else None

    @torch.no_grad()
    def step(self, entries, end=()):
        """entries: [{"id": request id, "tokens": [ids...], "want": [indices into tokens]}]; end: ids finished after this step.
        Returns fp32 logits [sum(len(want)), vocab] in the order of the entries and their `want` (None when nothing is wanted)."""
        plan, tokens, rows, base = [], [], [], 0
        for e in entries:
            if e["id"] not in self.cache.requests:
                self.cache.admit(e["id"])
            n = len(e["tokens"])
            if n == 0:
                raise ValueError(f"request {e['id']!r}: a step must bring at least one token")
            plan.append((e["id"], n))
            tokens.extend(e["tokens"])
            for w in e.get("want", ()):
                if not 0 <= w < n:
                    raise IndexError(f"request {e['id']!r}: wanted place {w} outside its {n} tokens")
                rows.append(base + w)
            base += n
        logits = None
        if plan and self.use_graph and all(n == 1 for _, n in plan) and all(self.cache.seq_len(r) > 0 for r, _ in plan):
            logits = self._decode_graph_step(plan, tokens, rows)
        elif plan:
            batch = self.cache.plan(plan)
            ids = torch.tensor(tokens, dtype=torch.int32, device=self.device)
            if rows:
                logits = self.model(ids, None, self.cache, batch=batch, logits_rows=torch.tensor(rows, dtype=torch.int32, device=self.device))
            else:   # the step still has to advance cache and state; only the last row is sent through the head
                self.model(ids, None, self.cache, batch=batch, logits_rows=torch.tensor([base - 1], dtype=torch.int32, device=self.device))
        for rid in end:
            if rid in self.cache.requests:
                self.cache.release(rid)
        return logits

    @torch.no_grad()
    def generate(self, prompts: dict, max_new_tokens: int = 16, do_sample: bool = False, temperature: float = 1.0, top_k: int = 0,
                 top_p: float = 1.0, generator: torch.Generator | None = None, eos_token_id=None, chunk_size: int | None = None) -> dict:
        """prompts: {request id: [token ids]} -> {request id: [generated ids]}.  One prefill step for all prompts (or portions of
        `chunk_size` tokens), then one token per live request per step.  Greedy unless do_sample."""
        live = list(prompts)
        out = {rid: [] for rid in live}
        done_len = {rid: 0 for rid in live}
        logits = None
        while True:   # prefill, in portions when asked
            entries = []
            for rid in live:
                rest = prompts[rid][done_len[rid]:]
                if rest:
                    part = rest if chunk_size is None else rest[:chunk_size]
                    done_len[rid] += len(part)
                    last = done_len[rid] == len(prompts[rid])
                    entries.append({"id": rid, "tokens": part, "want": [len(part) - 1] if last else []})
            if not entries:
                break
            lg = self.step(entries)
            k = 0
            for e in entries:
                if e["want"]:
                    logits = {} if logits is None else logits
                    logits[e["id"]] = lg[k]
                    k += 1
        for _ in range(max_new_tokens):
            nxt = {rid: int(sample_next_token(logits[rid], do_sample, temperature, top_k, top_p, generator)) for rid in live}
            for rid in live:
                out[rid].append(nxt[rid])
            ended = [rid for rid in live if len(out[rid]) >= max_new_tokens or (eos_token_id is not None and nxt[rid] == eos_token_id)]
            live = [rid for rid in live if rid not in ended]
            for rid in ended:
                self.cache.release(rid)
            if not live:
                break
            lg = self.step([{"id": rid, "tokens": [nxt[rid]], "want": [0]} for rid in live])
            logits = {rid: lg[i] for i, rid in enumerate(live)}
        return out

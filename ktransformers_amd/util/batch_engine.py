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


class BatchEngine:
    def __init__(self, model, cache):
        self.model, self.cache = model, cache
        self.device = cache.device

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
        if plan:
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

"""The ragged-step engine: requests, the scheduler that cuts them into steps, the step function, sampling.

A STEP is a list of entries (request, its next tokens, which of them want logits).  `Engine.run_step` is the one step function: it
asks the CacheManager for the pages and the slot of each entry, builds the RaggedBatch, runs the model once over all tokens of the step
and returns the wanted logits.  Everything else drives it:
  * `Engine.step()` -- the generation scheduler: every running request that has a sampled token contributes that token (decode), and
    waiting / partly prefilled requests contribute the next portion of their prompt, up to `max_step_tokens` tokens per step and
    `max_seqs` live requests, admitted in arrival order while pages are free; the last prompt token's logits and every decode token's
    logits are sampled.
  * `trace.replay` feeds steps that somebody else cut.
Sampling (greedy, temperature, top-k, top-p, seeded) runs on the library's logit kernels (ops.argmax_advance / softmax_rows / topk_rows);
the draw itself is host-side from a counter-based generator per request.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np
import torch

from . import seqops
from ._lib import ZLError
from .cache import CacheManager


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0          # 0: greedy
    top_k: int = 0                    # 0: the whole vocabulary
    top_p: float = 1.0
    seed: int = 0
    eos_id: Optional[int] = None


@dataclass
class Request:
    rid: str
    prompt: List[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    done_prompt: int = 0              # prompt tokens already run
    pending: Optional[int] = None     # the sampled token that the next step feeds
    output: List[int] = field(default_factory=list)
    finished: bool = False
    admitted: bool = False


@dataclass
class Entry:
    rid: str
    tokens: List[int]
    want: List[int] = field(default_factory=list)     # indices into tokens


class Engine:
    def __init__(self, model, max_tokens, max_seqs=4, max_step_tokens=512):
        if not getattr(model, "ragged", False):
            raise ZLError("this engine drives models that run ragged steps")
        self.model = model
        self.cache = model.bind_cache(CacheManager(max_tokens, max_seqs, model.device, page_size=model.page_size))
        self.max_seqs, self.max_step_tokens = max_seqs, max_step_tokens
        self.waiting: List[Request] = []
        self.running: Dict[str, Request] = {}
        self.finished: Dict[str, Request] = {}

    # ---- the step function --------------------------------------------------------------------------------------------------------
    def run_step(self, entries: List[Entry]):
        """Run one step; returns fp32 logits (sum of len(want), vocab) on the device in the order of the entries, or None."""
        if not entries:
            return None
        seen = set()
        for e in entries:
            if e.rid in seen or not e.tokens:
                raise ZLError("a step holds every request at most once, with at least one token")
            seen.add(e.rid)
            if any(w < 0 or w >= len(e.tokens) for w in e.want):
                raise ZLError("a wanted place lies outside the entry's tokens")
            have = self.cache.length(e.rid) if e.rid in self.cache.seqs else 0
            if have + len(e.tokens) > self.model.max_positions:
                raise ZLError(f"request {e.rid}: more positions than the model has ({self.model.max_positions})")
        for e in entries:
            if e.rid not in self.cache.seqs:
                self.cache.admit(e.rid)
        seqs, flat, rows, base = [], [], [], 0
        for e in entries:
            pos0, slot, pages = self.cache.extend(e.rid, len(e.tokens))
            seqs.append((len(e.tokens), pos0, slot, list(pages)))
            flat += e.tokens
            rows += [base + w for w in e.want]
            base += len(e.tokens)
        dev = self.model.device
        batch = seqops.RaggedBatch(seqs, self.cache.page_size, dev)
        ids = torch.tensor(flat + rows, dtype=torch.int32).to(dev)
        tokens, want = ids[:len(flat)], (ids[len(flat):] if rows else None)
        return self.model.forward(tokens, batch, want)

    def release(self, rid):
        if rid in self.cache.seqs:
            self.cache.release(rid)

    # ---- generation ---------------------------------------------------------------------------------------------------------------
    def add_request(self, rid, prompt, params: Optional[SamplingParams] = None):
        if not prompt:
            raise ZLError("a request needs a prompt of at least one token")
        if rid in self.running or rid in self.finished or any(r.rid == rid for r in self.waiting):
            raise ZLError(f"request id {rid} is in use")
        r = Request(rid, list(prompt), params or SamplingParams())
        r._rng = np.random.Generator(np.random.Philox(key=r.params.seed))
        self.waiting.append(r)
        return r

    def has_work(self):
        return bool(self.waiting or self.running)

    def schedule(self):
        """the entries of the next step: decode tokens first, then prompt portions in arrival order within the token and page budgets"""
        entries, budget = [], self.max_step_tokens
        free_pages = len(self.cache.free_pages)
        for r in self.running.values():
            need = 0 if self.cache.length(r.rid) % self.cache.page_size else 1
            if r.pending is not None and budget > 0 and need <= free_pages:
                entries.append(Entry(r.rid, [r.pending], [0]))
                budget -= 1
                free_pages -= need
        for r in list(self.running.values()) + self.waiting:
            if budget <= 0:
                break
            if r.pending is not None or r.done_prompt >= len(r.prompt):
                continue
            if not r.admitted and len(self.running) + sum(1 for e in entries if e.rid not in self.running) >= self.max_seqs:
                break
            have = self.cache.length(r.rid) if r.rid in self.cache.seqs else 0
            held = (have + self.cache.page_size - 1) // self.cache.page_size
            room = (held + max(free_pages, 0)) * self.cache.page_size - have
            n = min(budget, len(r.prompt) - r.done_prompt, room)
            if n <= 0:
                break
            free_pages -= (have + n + self.cache.page_size - 1) // self.cache.page_size - held
            toks = r.prompt[r.done_prompt:r.done_prompt + n]
            last = r.done_prompt + n == len(r.prompt)
            entries.append(Entry(r.rid, toks, [n - 1] if last else []))
            budget -= n
        return entries

    def step(self):
        """one scheduled step; returns {request id: new token} for the requests that sampled one"""
        entries = self.schedule()
        if not entries:
            if self.has_work():
                raise ZLError("nothing can be scheduled: the cache is too small for the live requests")
            return {}
        by_id = {r.rid: r for r in self.waiting}
        by_id.update(self.running)
        for e in entries:
            r = by_id[e.rid]
            if not r.admitted:
                r.admitted = True
                self.waiting.remove(r)
                self.running[r.rid] = r
        logits = self.run_step(entries)
        out, row = {}, 0
        sampled = [by_id[e.rid] for e in entries if e.want]
        picks = self.sample(logits, sampled) if sampled else []
        for e in entries:
            r = by_id[e.rid]
            if r.pending is not None:
                r.pending = None
            else:
                r.done_prompt += len(e.tokens)
            if e.want:
                tok = picks[row]
                row += 1
                r.output.append(tok)
                out[r.rid] = tok
                if len(r.output) >= r.params.max_new_tokens or tok == r.params.eos_id or \
                        self.cache.length(r.rid) + 1 > self.model.max_positions:
                    r.finished = True
                    self.release(r.rid)
                    del self.running[r.rid]
                    self.finished[r.rid] = r
                else:
                    r.pending = tok
        return out

    def sample(self, logits, reqs):
        """one token per row of logits (fp32, device) under each request's parameters"""
        from . import ops
        n = logits.shape[0]
        picks = [None] * n
        if any(r.params.temperature <= 0 for r in reqs):
            greedy = torch.empty(n, dtype=torch.int32, device=logits.device)
            ops.argmax_advance(logits, tokens=greedy)
            g = greedy.cpu().tolist()
            for i, r in enumerate(reqs):
                if r.params.temperature <= 0:
                    picks[i] = int(g[i])
        for i, r in enumerate(reqs):
            if picks[i] is not None:
                continue
            p = r.params
            probs = ops.softmax_rows(logits[i:i + 1].contiguous(), temperature=p.temperature)
            k = p.top_k if 0 < p.top_k < probs.shape[1] else probs.shape[1]
            if k <= 64:
                vals, idx = ops.topk_rows(probs, k)
                vals, idx = vals[0].double().cpu().numpy(), idx[0].cpu().numpy()
            else:                                   # (the top-k kernel reads a row once per candidate: small k only)
                pr = probs[0].double().cpu().numpy()
                idx = np.argsort(-pr, kind="stable")[:k]
                vals = pr[idx]
            if p.top_p < 1.0:
                keep = int(np.searchsorted(np.cumsum(vals), p.top_p * vals.sum(), side="left")) + 1
                vals, idx = vals[:keep], idx[:keep]
            u = r._rng.random() * vals.sum()
            picks[i] = int(idx[min(int(np.searchsorted(np.cumsum(vals), u, side="right")), len(idx) - 1)])
        return picks

    def generate(self, prompts, params: Optional[SamplingParams] = None):
        """run a list of prompts to the end through the scheduler; returns the generated tokens of each, in order"""
        reqs = [self.add_request(f"g{len(self.finished) + len(self.running) + len(self.waiting)}", p, params) for p in prompts]
        while self.has_work():
            self.step()
        return [r.output for r in reqs]

"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.

Differences from the reference's scheduler
(/root/reference/src/torchlet/v10_triton_paged_gqa/scheduler.py:97-167), on purpose:

* one mixed batch per step instead of a prefill batch and a decode batch: every running
  request that is decoding gives one token, and what is left of the step's token budget
  goes to prompt portions, oldest request first;
* a prompt longer than the budget is fed in portions over several steps; only the portion
  that reaches the end of the sequence asks for logits;
* when pages run out, the reference parks a running request with its pages and fails
  everything if nobody can move (scheduler.py:106-109,162-165).  Here the **youngest**
  running request is preempted instead: its pages and slot are given back and it returns
  to the front of the waiting queue, to be recomputed from ``prompt + generated so far``
  when pages are free again.  The oldest running request therefore always makes progress,
  and a request that alone can never fit the pool is refused when it is added.

The rules for applying a sampled token are the reference's (scheduler.py:255-266): a stop
token ends the request and is not kept; otherwise the token is kept and the request ends
when it has ``max_new_tokens``.  The last kept token is never fed to the model, hence the
``- 1`` in the length check (scheduler.py:84-95).

The scheduler decides with the cache manager's host-side bookkeeping only, so it is
tested without a GPU.
"""
from __future__ import annotations

from dataclasses import dataclass

from ..cache.manager import CacheManager
from .request import Request, RequestState


@dataclass
class Scheduled:
    request: Request
    start: int          # position of the first token fed in this step
    count: int          # tokens fed in this step
    samples: bool       # the step reaches the end of the sequence: a token is sampled from its last logits


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_tokens_per_step: int, max_positions: int):
        if max_tokens_per_step <= 0:
            raise ValueError("max_tokens_per_step must be positive")
        self.cache = cache
        self.max_tokens_per_step = max_tokens_per_step
        self.max_positions = max_positions
        self.waiting: list[Request] = []
        self.running: list[Request] = []      # in order of admission: oldest first
        self.finished: list[Request] = []
        self.num_preemptions = 0

    # ------------------------------------------------------------------ intake
    def validate(self, req: Request) -> None:
        if req.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive")
        if not req.prompt_tokens:
            raise ValueError("a request needs at least one prompt token")
        if req.temperature < 0:
            raise ValueError("temperature must not be negative")
        need = len(req.prompt_tokens) + req.max_new_tokens - 1
        if need > self.max_positions:
            raise ValueError(f"request {req.req_id} requires {need} cache positions, "
                             f"but max_position_embeddings is {self.max_positions}")
        for pages, capacity in zip(self.cache.pages_for(need), self.cache.capacity()):
            if pages > capacity:
                raise ValueError(f"request {req.req_id} needs {pages} cache pages for {need} tokens; the pool has {capacity}")

    def add_request(self, req: Request) -> None:
        self.validate(req)
        req.state = RequestState.WAITING
        self.waiting.append(req)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ------------------------------------------------------------------ deciding a step
    def _try_reserve(self, req: Request, count: int) -> bool:
        return self.cache.reserve(req.req_id, req.computed_tokens + count)

    def _preempt(self, req: Request) -> None:
        self.cache.release(req.req_id)
        self.running.remove(req)
        req.computed_tokens = 0
        req.state = RequestState.WAITING
        req.preemptions += 1
        self.num_preemptions += 1
        self.waiting.insert(0, req)

    def schedule(self) -> list[Scheduled]:
        budget = self.max_tokens_per_step
        chosen: list[Scheduled] = []
        preempted = False
        # 1. running requests, oldest first; decoding ones need one token, others a portion
        for req in list(self.running):
            if req not in self.running:        # preempted by an older request in this very loop
                continue
            if budget == 0:
                break
            count = min(req.sequence_length - req.computed_tokens, budget)
            while not self._try_reserve(req, count):
                preempted = True
                youngest = self.running[-1]
                if youngest is req:
                    # nothing younger to take pages from: it waits itself
                    self._preempt(req)
                    count = 0
                    break
                budget += sum(c.count for c in chosen if c.request is youngest)
                chosen = [c for c in chosen if c.request is not youngest]
                self._preempt(youngest)
            if count:
                chosen.append(Scheduled(req, req.computed_tokens, count,
                                        req.computed_tokens + count == req.sequence_length))
                budget -= count
        # 2. waiting requests, first come first served, while slots, pages and budget last
        # (not in a step that had to preempt: what was just freed is for the running requests)
        while not preempted and self.waiting and budget > 0 and self.cache.free_slots() > 0:
            req = self.waiting[0]
            count = min(req.sequence_length, budget)
            self.cache.add_request(req.req_id)
            if not self._try_reserve(req, count):
                self.cache.release(req.req_id)
                break
            self.waiting.pop(0)
            req.state = RequestState.RUNNING
            self.running.append(req)
            chosen.append(Scheduled(req, 0, count, count == req.sequence_length))
            budget -= count
        if not chosen and self.has_work():
            raise RuntimeError("cache pool exhausted; no request can make progress")
        return chosen

    def schedule_ahead(self, prev: list[Scheduled]) -> list[Scheduled]:
        """The step after ``prev``, decided before the tokens of ``prev`` are known, or nothing where
        it cannot be foreseen.  It can when ``prev`` gave every running request one decoded token and
        nobody waits: the next step then gives each of them one more, except those that end with the
        token of ``prev`` for having ``max_new_tokens``.  A request that the token of ``prev`` ends
        as a stop token is in this step for nothing; the caller drops its place when it learns so.
        Pages are taken for all or for none."""
        if self.waiting or not prev or len(prev) != len(self.running) or len(prev) > self.max_tokens_per_step:
            return []
        if any(c.count != 1 or not c.samples or c.request.state is not RequestState.RUNNING for c in prev):
            return []
        going = [c.request for c in prev if len(c.request.output_tokens) + 1 < c.request.max_new_tokens]
        if not going:
            return []
        need = [0] * len(self.cache.groups)
        for r in going:
            for g, m in enumerate(self.cache.pages_missing(r.req_id, r.computed_tokens + 2)):
                need[g] += m
        if any(n > f for n, f in zip(need, self.cache.free_pages())):
            return []
        for r in going:
            self.cache.reserve(r.req_id, r.computed_tokens + 2)
        return [Scheduled(r, r.computed_tokens + 1, 1, True) for r in going]

    # ------------------------------------------------------------------ applying results
    def process_output(self, chosen: list[Scheduled], sampled: list[int]) -> list[Request]:
        """``sampled``: one token per entry of ``chosen`` with ``samples`` set, in order.
        Returns the requests that finished; their pages and slots are already given back."""
        it = iter(sampled)
        done: list[Request] = []
        for c in chosen:
            req = c.request
            req.computed_tokens += c.count
            if not c.samples:
                continue
            tok = int(next(it))
            if tok in req.stop_token_ids:
                req.finish_reason = "stop"
            else:
                req.output_tokens.append(tok)
                if len(req.output_tokens) >= req.max_new_tokens:
                    req.finish_reason = "length"
            if req.finish_reason is not None:
                req.state = RequestState.FINISHED
                done.append(req)
        for req in done:
            self.running.remove(req)
            self.cache.release(req.req_id)
        self.finished.extend(done)
        return done

    def drain_finished(self) -> list[Request]:
        out, self.finished = self.finished, []
        return out

    def fail_all(self, error: Exception) -> list[Request]:
        """Every request that is not finished ends with ``error``; the cache is reset
        (after scheduler.py:294-332 of the reference)."""
        failed = []
        for req in self.running + self.waiting:
            req.error = error
            req.finish_reason = "error"
            req.state = RequestState.FINISHED
            failed.append(req)
        out = self.finished + failed
        self.running, self.waiting, self.finished = [], [], []
        self.cache.reset()
        return out

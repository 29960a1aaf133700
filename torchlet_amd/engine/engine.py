"""The engine: scheduler above, step function below, sampler beside
(after /root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:101-135,204-217).

``step()`` asks the scheduler what to run, feeds that to the step function as one batch,
samples a token for every request whose portion reached the end of its sequence, and
hands the tokens back to the scheduler, which finishes and frees.  It is synchronous for its
caller; the asynchronous ``generate`` of the Python entry point wraps it.  Inside, a decode step may
be enqueued one step ahead of the tokens the host has read (see ``Engine``).
"""
from __future__ import annotations

from concurrent.futures import CancelledError

from ..sampling.sampler import Sampler
from .batch import StepEntry
from .request import Request
from .runner import ModelRunner
from .scheduler import Scheduler


class _Launched:
    """A step that is enqueued: what it ran, the draw of its tokens, and the requests that turned
    out to be in it for nothing (ended by the step before it, which was still unread when this
    one was enqueued)."""

    def __init__(self, chosen, drawn):
        self.chosen = chosen
        self.drawn = drawn
        self.void: set = set()


class Engine:
    """``lookahead``: while the host waits for the tokens of a step in which every running request
    decoded one token, the next such step is already enqueued; it takes its tokens from where the
    sampling kernel left them on the GPU, so the GPU does not idle while the host reads tokens,
    books them and prepares the next step.  Tokens, their order and what each request generates
    are the same with and without it; a request that ends on a stop token is found out one step
    late and costs one token's worth of work for nothing."""

    def __init__(self, runner: ModelRunner, *, max_tokens_per_step: int = 2048, seed: int = 0, lookahead: bool = True):
        self.runner = runner
        self.scheduler = Scheduler(runner.cache, max_tokens_per_step=max_tokens_per_step,
                                   max_positions=runner.max_positions)
        self.sampler = Sampler(seed)
        self.steps = 0
        self.lookahead = lookahead
        self.steps_ahead = 0              # steps that were enqueued before their tokens were known
        self._ahead: _Launched | None = None

    def validate(self, req: Request) -> None:
        """Raise ``ValueError`` for a request that could never run (the scheduler's rules, and token ids
        outside the vocabulary); nothing is kept of it."""
        bad = [t for t in req.prompt_tokens if not 0 <= t < self.runner.vocab_size]
        if bad:
            raise ValueError(f"request {req.req_id}: token id {bad[0]} outside the vocabulary of {self.runner.vocab_size}")
        self.scheduler.validate(req)

    def add_request(self, req: Request) -> None:
        self.validate(req)
        self.scheduler.add_request(req)

    def add_requests(self, reqs: list[Request]) -> None:
        """All of them or none: every request is checked before the first one is queued, so a call that
        fails leaves nothing waiting."""
        for r in reqs:
            self.validate(r)
        for r in reqs:
            self.scheduler.add_request(r)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def _launch(self, chosen, after: _Launched | None = None) -> _Launched:
        """Enqueue the step ``chosen`` and the draw of its tokens; with ``after``, every request
        takes its token from the draw of that step, on the GPU."""
        if after is None:
            entries = [StepEntry(c.request.req_id, c.request.tokens(c.start, c.count), [c.count - 1] if c.samples else [])
                       for c in chosen]
            logits = self.runner.step(entries)
            ahead = 0
        else:
            place = {r: i for i, r in enumerate(c.request for c in after.chosen if c.samples)}
            entries = [StepEntry(c.request.req_id, [0], [0]) for c in chosen]
            logits = self.runner.step(entries, device_tokens=(after.drawn.device, [place[c.request] for c in chosen]))
            ahead = 1              # the token of `after` is not in output_tokens yet
        sampling = [c.request for c in chosen if c.samples]
        drawn = None
        if sampling:
            drawn = self.sampler.launch(logits, [r.temperature for r in sampling], [r.seed for r in sampling],
                                        [len(r.output_tokens) + ahead for r in sampling])
        return _Launched(chosen, drawn)

    def step(self) -> list[Request]:
        """Finish one step; returns the requests that finished in it."""
        launched, self._ahead = self._ahead, None
        if launched is None:
            launched = self._launch(self.scheduler.schedule())
        if self.lookahead:
            nxt = self.scheduler.schedule_ahead([c for c in launched.chosen if c.request not in launched.void])
            if nxt:
                self._ahead = self._launch(nxt, after=launched)
                self.steps_ahead += 1
        tokens = launched.drawn.tokens() if launched.drawn is not None else []
        chosen = launched.chosen
        if launched.void:           # their places in the step and their tokens count for nothing
            kept = [c.request not in launched.void for c in chosen if c.samples]
            tokens = [t for t, k in zip(tokens, kept) if k]
            chosen = [c for c in chosen if c.request not in launched.void]
        self.steps += 1
        done = self.scheduler.process_output(chosen, tokens)
        if self._ahead is not None:
            self._ahead.void.update(r for r in done if any(c.request is r for c in self._ahead.chosen))
            if all(c.request in self._ahead.void for c in self._ahead.chosen):
                self._ahead = None
        return done

    def fail_all(self, error: Exception) -> list[Request]:
        """Every unfinished request ends with ``error``; a step enqueued ahead is forgotten."""
        self._ahead = None
        return self.scheduler.fail_all(error)

    def shutdown(self) -> list[Request]:
        """Give up every request that is not finished (they end with a cancellation error) and take
        back all pages, as the reference's engine does when it is shut down (engine.py:81-99 of
        the reference); the engine can be used again afterwards."""
        return self.fail_all(CancelledError("the engine was shut down"))

    def run_until_done(self) -> list[Request]:
        """Step until no request is waiting or running; on an error every unfinished request
        fails with it (engine.py:213-217 of the reference) and the error is raised."""
        done: list[Request] = []
        try:
            while self.has_work():
                done.extend(self.step())
        except Exception as exc:
            self.fail_all(exc)
            raise
        self.scheduler.drain_finished()
        return done

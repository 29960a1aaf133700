"""The engine: scheduler above, step function below, sampler beside
(after /root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:101-135,204-217).

``step()`` asks the scheduler what to run, feeds that to the step function as one batch,
samples a token for every request whose portion reached the end of its sequence, and
hands the tokens back to the scheduler, which finishes and frees.  It is synchronous; the
asynchronous ``generate`` of the Python entry point wraps it.
"""
from __future__ import annotations

from concurrent.futures import CancelledError

from ..sampling.sampler import Sampler
from .batch import StepEntry
from .request import Request
from .runner import ModelRunner
from .scheduler import Scheduler


class Engine:
    def __init__(self, runner: ModelRunner, *, max_tokens_per_step: int = 2048, seed: int = 0):
        self.runner = runner
        self.scheduler = Scheduler(runner.cache, max_tokens_per_step=max_tokens_per_step,
                                   max_positions=runner.max_positions)
        self.sampler = Sampler(seed)
        self.steps = 0

    def add_request(self, req: Request) -> None:
        bad = [t for t in req.prompt_tokens if not 0 <= t < self.runner.vocab_size]
        if bad:
            raise ValueError(f"request {req.req_id}: token id {bad[0]} outside the vocabulary of {self.runner.vocab_size}")
        self.scheduler.add_request(req)

    def has_work(self) -> bool:
        return self.scheduler.has_work()

    def step(self) -> list[Request]:
        """Run one step; returns the requests that finished in it."""
        chosen = self.scheduler.schedule()
        entries = [StepEntry(c.request.req_id, c.request.tokens(c.start, c.count), [c.count - 1] if c.samples else [])
                   for c in chosen]
        logits = self.runner.step(entries)
        sampling = [c.request for c in chosen if c.samples]
        tokens: list[int] = []
        if sampling:
            tokens = self.sampler.sample(logits, [r.temperature for r in sampling], [r.seed for r in sampling],
                                         [len(r.output_tokens) for r in sampling])
        self.steps += 1
        return self.scheduler.process_output(chosen, tokens)

    def shutdown(self) -> list[Request]:
        """Give up every request that is not finished (they end with a cancellation error) and take
        back all pages, as the reference's engine does when it is shut down (engine.py:81-99 of
        the reference); the engine can be used again afterwards."""
        return self.scheduler.fail_all(CancelledError("the engine was shut down"))

    def run_until_done(self) -> list[Request]:
        """Step until no request is waiting or running; on an error every unfinished request
        fails with it (engine.py:213-217 of the reference) and the error is raised."""
        done: list[Request] = []
        try:
            while self.has_work():
                done.extend(self.step())
        except Exception as exc:
            self.scheduler.fail_all(exc)
            raise
        self.scheduler.drain_finished()
        return done

"""Ways of cutting the same requests into steps, and the check of a replay against the
plain implementation.  A *step* is ``{"step": i, "entries": [{"id", "tokens", "want"}], "end": [...]}``
as ``bin/trace_run`` reads it."""
import random

import numpy as np
import torch

import plain_qwen2

FP32_TOL = dict(atol=4e-6, rtol=2e-5)     # ~10x the 32-bit rounding of the plain implementation itself (3.7e-7)
BF16_TOL = dict(atol=1e-2, rtol=1e-2)     # ~3x what the design's bfloat16 roundings add on these models (3.3e-3)


def make_requests(vocab: int, lengths, seed: int) -> dict[str, list[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _round_up(n, m):
    return -(-n // m) * m


def whole(requests):
    """Each request alone and whole: one step, every logit wanted."""
    return [dict(entries=[dict(id=r, tokens=t, want=list(range(len(t))))], end=[r]) for r, t in requests.items()]


def tail_singles(requests, tail=32):
    """Most of a request in one step, then its last ``tail`` tokens one by one."""
    steps = []
    for r, t in requests.items():
        head = max(1, len(t) - tail)
        steps.append(dict(entries=[dict(id=r, tokens=t[:head], want=list(range(head)))], end=[]))
        for i in range(head, len(t)):
            steps.append(dict(entries=[dict(id=r, tokens=[t[i]], want=[0])], end=[r] if i == len(t) - 1 else []))
        if head == len(t):
            steps[-1]["end"] = [r]
    return steps


def portions(requests, sizes=(7, 16, 2, 5, 3, 33, 2, 9, 17, 2, 64)):
    """Portions of changing size, down to two tokens, across page edges at odd offsets."""
    steps = []
    for k, (r, t) in enumerate(requests.items()):
        i, j = 0, k
        while i < len(t):
            n = min(sizes[j % len(sizes)], len(t) - i)
            if len(t) - i - n == 1:      # never leave a lone last token: portions are of two or more
                n += 1
            steps.append(dict(entries=[dict(id=r, tokens=t[i:i + n], want=list(range(n)))], end=[r] if i + n == len(t) else []))
            i += n
            j += 1
    return steps


def mixed(requests, seed=0, max_live=4, prompt_fraction=0.6):
    """Up to ``max_live`` live requests; portions of some beside single tokens of others; a
    request is sometimes left out of a step; later requests arrive as earlier ones end."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            r, _ = waiting.pop(0)
            live[r] = 0
        entries, end = [], []
        for r in list(live):
            t, done = requests[r], live[r]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                  # left out of this step
            prompt = max(2, int(len(t) * prompt_fraction))
            if done < prompt:
                n = min(rng.choice([2, 3, 5, 8, 13, 21]), prompt - done)
                if prompt - done - n == 1:
                    n += 1
            else:
                n = 1
            n = min(n, len(t) - done)
            entries.append(dict(id=r, tokens=t[done:done + n], want=list(range(n))))
            live[r] = done + n
            if live[r] == len(t):
                end.append(r)
                del live[r]
        if entries:
            steps.append(dict(entries=entries, end=end))
    return steps


def number(steps, first=0):
    return [dict(step=first + i, **s) for i, s in enumerate(steps)]


def max_tokens_needed(steps, unit=64) -> int:
    """Most tokens live requests hold at any time, each rounded up to a multiple of ``unit``."""
    held: dict[str, int] = {}
    worst = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        worst = max(worst, sum(_round_up(n, unit) for n in held.values()))
        for r in s["end"]:
            held.pop(r, None)
    return worst


def expected_logits(folder, requests):
    cfg, weights = plain_qwen2.load_folder(folder, torch.float64)
    return {r: plain_qwen2.forward(cfg, weights, t) for r, t in requests.items()}


def bounds_from_plain(cfg, tensors, requests):
    """The plain implementation as its own yardstick, on the device of ``tensors``:
    ``(expected, noise, noise16, rms16)``.  ``expected``: float64 logits of every request (on the host);
    ``noise``: how far the plain implementation's own 32-bit evaluation lies from them at most (rounding
    that depends on the order of summation only); ``noise16`` and ``rms16``: how far, at most and in the
    root mean square, it moves when evaluated in 64-bit but with every tensor that separate kernels hand
    to each other through memory rounded to bfloat16."""
    w64 = {k: v.double() for k, v in tensors.items()}
    expected = {r: plain_qwen2.forward(cfg, w64, t).cpu() for r, t in requests.items()}
    rounded = lambda t: t.to(torch.bfloat16).double()
    moved = {r: plain_qwen2.forward(cfg, w64, t, stored=rounded).cpu() - expected[r] for r, t in requests.items()}
    del w64
    w32 = {k: v.float() for k, v in tensors.items()}
    noise = max(float((plain_qwen2.forward(cfg, w32, t).cpu().double() - expected[r]).abs().max()) for r, t in requests.items())
    del w32
    noise16 = max(float(m.abs().max()) for m in moved.values())
    rms16 = float(torch.cat([m.flatten() for m in moved.values()]).pow(2).mean().sqrt())
    return expected, noise, noise16, rms16


def _rows(steps, outputs, expected, what=""):
    """Every wanted row of a replay beside the plain implementation's logits of its request
    at its absolute position: ``(got, ref, place)``."""
    pos: dict[str, int] = {}
    for s in steps:
        rows = outputs.get(s["step"])
        k = 0
        for e in s["entries"]:
            base = pos.get(e["id"], 0)
            for w in e["want"]:
                got = torch.from_numpy(np.asarray(rows[k], dtype=np.float32)).double()
                yield got, expected[e["id"]][base + w], (f"step {s['step']} request {e['id']} position {base + w} "
                                                        f"(portion starts at {base}, place {w} of {len(e['tokens'])})")
                k += 1
            pos[e["id"]] = base + len(e["tokens"])
        assert rows is None or k == len(rows), f"{what}: step {s['step']} returned {len(rows)} rows, {k} wanted"
        for r in s["end"]:
            pos.pop(r, None)


def check(steps, outputs, expected, tol, what=""):
    """``outputs[step]``: array ``[wanted, vocab]``.  Every row is compared with the plain
    implementation's logits of its request at its absolute position; the first mismatch
    is reported with its place."""
    for got, ref, place in _rows(steps, outputs, expected, what):
        if not torch.allclose(got, ref, **tol):
            raise AssertionError(f"{what}: {place}: max abs error {float((got - ref).abs().max()):.3e}")


def rms_error(steps, outputs, expected) -> float:
    """Root mean square of the error over every wanted logit of a replay."""
    total, count = 0.0, 0
    for got, ref, _ in _rows(steps, outputs, expected):
        total += float((got - ref).pow(2).sum())
        count += ref.numel()
    return (total / max(count, 1)) ** 0.5


def check_steps_ahead_on_a_random_workload(model, page_size, seed, use_graphs=False):
    """A random workload (arrivals at random steps, lengths, temperatures, stop tokens, a pool so small
    that requests are preempted) through the whole engine, with and without steps enqueued ahead of
    their tokens: every request generates the same tokens and ends for the same reason, no page is
    lost, and every pool ends full.  Returns the engine of the run with steps ahead."""
    from torchlet_amd.engine.config import EngineConfig
    from torchlet_amd.engine.loading import make_engine
    from torchlet_amd.engine.request import Request

    rnd = random.Random(seed)
    vocab = model.spec.vocab_size
    n = rnd.randrange(3, 7)
    lengths = [rnd.randrange(1, 40) for _ in range(n)]
    prompts = list(make_requests(vocab, lengths, seed=seed).values())
    news = [rnd.randrange(1, 20) for _ in range(n)]
    temps = [rnd.choice([0.0, 0.0, 0.7, 1.3]) for _ in range(n)]
    arrive = sorted(rnd.randrange(0, 25) for _ in range(n))
    stop = frozenset(rnd.sample(range(vocab), 24))
    pages = rnd.choice([6, 8, 30]) * 16 // page_size          # few of them force preemptions
    budget = rnd.choice([8, 24, 64])
    slots = rnd.choice([2, 4])
    dtype = "float32" if model.dtype == torch.float32 else "bfloat16"

    def run(lookahead):
        e = make_engine(model, EngineConfig(page_size=page_size, num_pages=pages, max_slots=slots, max_tokens_per_step=budget,
                                            dtype=dtype, use_graphs=use_graphs, lookahead=lookahead, seed=3))
        reqs = [Request(prompt_tokens=p, seed=i, max_new_tokens=m, temperature=t, stop_token_ids=stop)
                for i, (p, m, t) in enumerate(zip(prompts, news, temps))]
        step = 0
        while step <= max(arrive) or e.has_work():
            for i, a in enumerate(arrive):
                if a == step:
                    e.add_request(reqs[i])
            if e.has_work():
                e.step()
            e.runner.cache.check()
            step += 1
        assert e.runner.cache.live_requests() == [] and e._ahead is None
        assert e.runner.cache.free_pages() == e.runner.cache.capacity()
        return e, [(r.output_tokens, r.finish_reason) for r in reqs]

    e0, plain = run(False)
    e1, ahead = run(True)
    assert ahead == plain, f"seed {seed}: steps enqueued ahead changed what was generated"
    assert all(reason in ("stop", "length") for _, reason in plain)
    assert e0.steps_ahead == 0
    return e1

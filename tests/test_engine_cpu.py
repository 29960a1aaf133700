"""The engine's host logic on the CPU: step function over the cache manager, scheduler
and sampler, with the HIP entry points replaced by the stand-ins of ``emulated_ops.py``.
The kernels themselves are tested on the GPU (``-m gpu``)."""
import json

import pytest
import torch

import plain_qwen2
import scenarios
import tiny_models
from torchlet_amd.cache.manager import OutOfPages
from torchlet_amd.engine.batch import StepEntry
from torchlet_amd.engine.engine import Engine
from torchlet_amd.engine.loading import load_model, make_runner
from torchlet_amd.engine.request import Request
from torchlet_amd.sampling.sampler import draw_key


def runner_for(folder, name, dtype="float32", pages=64, slots=4):
    _, model = load_model(folder, dtype, device="cpu")
    return make_runner(model, page_size=tiny_models.PAGE_SIZES[name], num_pages=pages, max_requests=slots)


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("mode", ["whole", "portions", "mixed"])
def test_step_function_equals_plain_under_every_split(cpu_ops, model_folders, name, mode):
    cfg = json.loads((model_folders[name] / "config.json").read_text())
    reqs = scenarios.make_requests(cfg["vocab_size"], [37, 5, 70, 18, 33], seed=5)
    exp = scenarios.expected_logits(model_folders[name], reqs)
    steps = scenarios.number(getattr(scenarios, mode)(reqs))
    page = tiny_models.PAGE_SIZES[name]
    runner = runner_for(model_folders[name], name, pages=-(-scenarios.max_tokens_needed(steps) // page) + 1)
    out = {}
    for s in steps:
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            out[s["step"]] = logits.numpy()
        for r in s["end"]:
            runner.release(r)
        runner.cache.check()
    scenarios.check(steps, out, exp, scenarios.FP32_TOL, f"{name}/{mode}")
    assert runner.cache.live_requests() == []


def test_step_refuses_bad_input_and_a_failed_step_leaves_no_trace(cpu_ops, model_folders):
    runner = runner_for(model_folders["A"], "A", pages=3)          # 2 usable pages = 32 tokens
    with pytest.raises(ValueError, match="outside the vocabulary"):
        runner.step([StepEntry("a", [1, 256], [])])
    with pytest.raises(ValueError, match="twice"):
        runner.step([StepEntry("a", [1], []), StepEntry("a", [2], [])])
    with pytest.raises(ValueError, match="wanted place"):
        runner.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", list(range(20)), []), StepEntry("b", list(range(20)), [])])
    assert runner.cache.live_requests() == [] and runner.cache.free_pages() == [2]
    with pytest.raises(ValueError, match="max_position_embeddings"):
        runner_for(model_folders["A"], "A", pages=20).step([StepEntry("a", [1] * 129, [])])
    assert runner.step([StepEntry("a", [1, 2, 3], [])]) is None     # nothing wanted: no logits
    assert runner.step([StepEntry("a", [4], [0])]).shape == (1, 256)


def _generate(engine, prompts, **kw):
    reqs = [Request(prompt_tokens=p, seed=i, **kw) for i, p in enumerate(prompts)]
    for r in reqs:
        engine.add_request(r)
    engine.run_until_done()
    return reqs


def test_greedy_generation_equals_the_plain_loop(cpu_ops, model_folders):
    """Configuration A's workload: prompts of 5, 17 and 33 tokens, 8 greedy tokens each."""
    cfg, w = plain_qwen2.load_folder(model_folders["A"])
    prompts = list(scenarios.make_requests(cfg.vocab, [5, 17, 33], seed=2).values())
    engine = Engine(runner_for(model_folders["A"], "A"), max_tokens_per_step=24)
    reqs = _generate(engine, prompts, max_new_tokens=8)
    for r, p in zip(reqs, prompts):
        assert r.output_tokens == plain_qwen2.greedy(cfg, w, p, 8)
    assert engine.runner.cache.live_requests() == []


def test_temperature_sampling_is_the_same_alone_batched_and_after_preemption(cpu_ops, model_folders):
    """Configuration B's workload: prompts of 1, 9, 40 and 64 tokens, temperature 0.8 with a
    fixed sampler seed, 12 new tokens, arrivals at steps 0, 0, 3 and 5."""
    cfg = json.loads((model_folders["B"] / "config.json").read_text())
    prompts = list(scenarios.make_requests(cfg["vocab_size"], [1, 9, 40, 64], seed=3).values())
    kw = dict(max_new_tokens=12, temperature=0.8)
    alone = []
    for i, p in enumerate(prompts):
        e = Engine(runner_for(model_folders["B"], "B"), max_tokens_per_step=256, seed=42)
        r = Request(prompt_tokens=p, seed=i, **kw)
        e.add_request(r)
        e.run_until_done()
        alone.append(r.output_tokens)
    assert len({tuple(a) for a in alone}) == 4 and all(len(a) == 12 for a in alone)

    def staggered(pages, budget):
        e = Engine(runner_for(model_folders["B"], "B", pages=pages), max_tokens_per_step=budget, seed=42)
        reqs = [Request(prompt_tokens=p, seed=i, **kw) for i, p in enumerate(prompts)]
        arrivals = {0: [0, 1], 3: [2], 5: [3]}
        step = 0
        while step < 6 or e.has_work():
            for i in arrivals.get(step, []):
                e.add_request(reqs[i])
            if e.has_work():
                e.step()
            step += 1
            e.runner.cache.check()
        return e, reqs

    e, reqs = staggered(pages=64, budget=16)                    # portions of at most 16 beside decode tokens
    assert [r.output_tokens for r in reqs] == alone
    e, reqs = staggered(pages=16, budget=32)                    # 15 pages of 8 = 120 tokens for 4 requests that want 150
    assert e.scheduler.num_preemptions > 0
    assert [r.output_tokens for r in reqs] == alone
    assert e.runner.cache.free_pages() == [15]
    other = Engine(runner_for(model_folders["B"], "B"), max_tokens_per_step=256, seed=43)
    r = Request(prompt_tokens=prompts[1], seed=1, **kw)
    other.add_request(r)
    other.run_until_done()
    assert r.output_tokens != alone[1]                          # another sampler seed, other draws


def test_a_step_enqueued_ahead_of_its_tokens_changes_nothing_that_is_generated(cpu_ops, model_folders):
    """Decode steps that take their tokens from the sampler's output before the host has read them:
    same tokens as without, for requests that end by length at different times, that end on a stop
    token (found out one step late: the place in the step already enqueued counts for nothing), that
    sample with a temperature, and with a request that arrives in between."""
    cfg = json.loads((model_folders["B"] / "config.json").read_text())
    prompts = list(scenarios.make_requests(cfg["vocab_size"], [3, 9, 20, 14], seed=7).values())

    def run(lookahead, stop=frozenset(), late=True):
        e = Engine(runner_for(model_folders["B"], "B"), max_tokens_per_step=64, seed=9, lookahead=lookahead)
        reqs = [Request(prompt_tokens=p, seed=i, max_new_tokens=n, temperature=t, stop_token_ids=stop)
                for i, (p, n, t) in enumerate(zip(prompts, (5, 17, 11, 9), (0.0, 0.9, 0.0, 0.7)))]
        for r in reqs[:3]:
            e.add_request(r)
        step = 0
        while e.has_work() or step < 8:
            if step == 7 and late:
                e.add_request(reqs[3])
            if e.has_work():
                e.step()
            e.runner.cache.check()
            step += 1
        assert e.runner.cache.live_requests() == [] and e._ahead is None
        return e, [(r.output_tokens, r.finish_reason) for r in reqs[:4 if late else 3]]

    e0, plain = run(False)
    e1, ahead = run(True)
    assert ahead == plain and e0.steps_ahead == 0 and e1.steps_ahead >= 8
    assert [len(t) for t, _ in plain] == [5, 17, 11, 9]
    # a stop token: one that the second request generates in the middle of its run
    stop = frozenset({plain[1][0][6]})
    e0, plain_s = run(False, stop)
    e1, ahead_s = run(True, stop)
    assert ahead_s == plain_s and plain_s[1][1] == "stop" and len(plain_s[1][0]) <= 6 and e1.steps_ahead > 0


@pytest.mark.parametrize("name", ["A", "C"])          # C: a window on the later layers, two cache groups
@pytest.mark.parametrize("seed", range(4))
def test_steps_ahead_under_random_arrivals_stop_tokens_and_few_pages(cpu_ops, model_folders, name, seed):
    """Random workloads (arrivals at random steps, lengths, temperatures, stop tokens, a pool so small
    that requests are preempted): with and without steps enqueued ahead, every request generates
    the same tokens and ends for the same reason; no page is lost.  (The same runs on the GPU, with
    decode steps replayed as graphs, in test_generate_gpu.py.)"""
    _, model = load_model(model_folders[name], "float32", device="cpu")
    scenarios.check_steps_ahead_on_a_random_workload(model, tiny_models.PAGE_SIZES[name], seed)


def test_max_model_len_bounds_the_step_function(cpu_ops, model_folders):
    _, model = load_model(model_folders["A"], "float32", device="cpu")
    runner = make_runner(model, page_size=16, num_pages=20, max_requests=2, max_model_len=30)
    assert runner.step([StepEntry("a", [1] * 30, [29])].copy()).shape == (1, 256)
    with pytest.raises(ValueError, match="max_model_len"):
        runner.step([StepEntry("a", [1], [0])])


def test_draw_keys_differ_in_every_argument():
    keys = {draw_key(s, r, i) for s in (0, 1, 2 ** 40) for r in (0, 1, 2 ** 33) for i in range(4)}
    assert len(keys) == 36 and all(-2 ** 31 <= k < 2 ** 31 for k in keys)


def test_errors_fail_every_unfinished_request(cpu_ops, model_folders, monkeypatch):
    engine = Engine(runner_for(model_folders["A"], "A"), max_tokens_per_step=64)
    reqs = [Request(prompt_tokens=[1, 2, 3], max_new_tokens=4), Request(prompt_tokens=[4, 5], max_new_tokens=4)]
    for r in reqs:
        engine.add_request(r)
    engine.step()
    monkeypatch.setattr(engine.runner, "step", lambda entries: (_ for _ in ()).throw(RuntimeError("device lost")))
    with pytest.raises(RuntimeError, match="device lost"):
        engine.run_until_done()
    assert all(isinstance(r.error, RuntimeError) and r.finish_reason == "error" for r in reqs)
    assert engine.runner.cache.live_requests() == [] and not engine.has_work()
    with pytest.raises(ValueError, match="outside the vocabulary"):
        engine.add_request(Request(prompt_tokens=[999]))


def test_toy_parts_and_a_layer_run_twice_on_the_host(cpu_ops):
    """The generality test of ``toy_parts.py`` (a routed feed-forward, a position encoding of its
    own, a layer that runs twice and reads its first run's cache) through the host logic."""
    import toy_parts
    toy_parts.run_toy_mix(torch.float32, torch.device("cpu"), lambda dtype, ref: dict(atol=2e-5, rtol=1e-4))


def test_shutdown_gives_up_unfinished_requests_and_frees_their_pages(cpu_ops, model_folders):
    from concurrent.futures import CancelledError
    runner = runner_for(model_folders["A"], "A", pages=12)
    engine = Engine(runner, max_tokens_per_step=16)
    done_early = Request(prompt_tokens=[1, 2, 3], max_new_tokens=1)
    long_one = Request(prompt_tokens=list(range(40)), max_new_tokens=30)
    waiting = Request(prompt_tokens=list(range(100)), max_new_tokens=5)
    for r in (done_early, long_one, waiting):
        engine.add_request(r)
    for _ in range(3):
        engine.step()
    assert done_early.finish_reason == "length" and long_one.finish_reason is None
    ended = engine.shutdown()
    assert {r.req_id for r in ended} >= {long_one.req_id, waiting.req_id}
    assert isinstance(long_one.error, CancelledError) and long_one.finish_reason == "error" and waiting.finish_reason == "error"
    assert done_early.error is None
    assert runner.cache.live_requests() == [] and not engine.has_work()
    runner.cache.check()
    again = Request(prompt_tokens=[5, 6], max_new_tokens=2)      # the engine goes on working
    engine.add_request(again)
    engine.run_until_done()
    assert len(again.output_tokens) == 2


def test_requests_are_added_all_or_none(cpu_ops, model_folders):
    """A call that brings one bad request leaves nothing waiting (``LLM.generate`` adds through this)."""
    engine = Engine(runner_for(model_folders["A"], "A"), max_tokens_per_step=24)
    good = Request(prompt_tokens=[1, 2, 3], max_new_tokens=4)
    for bad in (Request(prompt_tokens=[1] * 126, max_new_tokens=4),        # passes max_position_embeddings (128)
                Request(prompt_tokens=[1, 256], max_new_tokens=4),         # outside the vocabulary
                Request(prompt_tokens=[], max_new_tokens=4)):
        with pytest.raises(ValueError):
            engine.add_requests([good, bad])
        assert not engine.has_work()
    engine.add_requests([good])
    assert engine.has_work()
    engine.run_until_done()
    assert len(good.output_tokens) == 4 and engine.runner.cache.live_requests() == []


def test_chat_template_runs_in_a_sandbox():
    import jinja2

    from torchlet_amd.llm import render_chat_template

    ok = "{% for m in messages %}<|im_start|>{{ m['role'] }}\n{{ m['content'] }}<|im_end|>\n{% endfor %}" \
         "{% if add_generation_prompt %}<|im_start|>assistant\n{% endif %}"
    assert render_chat_template(ok, "hi") == "<|im_start|>user\nhi<|im_end|>\n<|im_start|>assistant\n"
    for evil in ("{{ messages.__class__.__mro__ }}", "{{ ''.__class__.__base__.__subclasses__() }}",
                 "{% set _ = messages.append(1) %}"):
        with pytest.raises(jinja2.exceptions.SecurityError):
            render_chat_template(evil, "hi")
    assert render_chat_template("{{ raise_exception.__globals__ }}", "hi") == ""      # a function's globals: not there
    with pytest.raises(jinja2.exceptions.SecurityError):
        render_chat_template("{{ raise_exception.__globals__['__builtins__'] }}", "hi")
    with pytest.raises(jinja2.exceptions.TemplateError, match="no system turn"):
        render_chat_template("{{ raise_exception('no system turn') }}", "hi")


def test_toy_attention_that_differs_in_one_stage_on_the_host(cpu_ops):
    """``toy_parts.run_toy_qk_norm`` (queries and keys normalised per head through the attention mixer's hook) on the host."""
    import toy_parts
    toy_parts.run_toy_qk_norm(torch.float32, torch.device("cpu"), lambda dtype, ref: dict(atol=2e-5, rtol=1e-4))


def test_toy_norm_of_another_kind_is_run_not_fused_on_the_host(cpu_ops):
    import toy_parts
    toy_parts.run_toy_norm(torch.float32, torch.device("cpu"))


def test_toy_mixer_whose_cache_planes_differ_on_the_host(cpu_ops):
    import toy_parts
    toy_parts.run_toy_latent(torch.float32, torch.device("cpu"))


def test_parts_of_the_keys_for_prompt_portions():
    """How the attention mixer deals the keys of 128-row tiles to work-groups: few tiles are split to fill the
    compute units; many tiles of equal length are split when that evens out the rounds of 512 work-groups."""
    from torchlet_amd.parts.attention import _prompt_splits
    assert _prompt_splits(160, 16384, uniform=True) == 4 and _prompt_splits(160, 16384, uniform=False) == 4
    assert _prompt_splits(160, 1100, uniform=True) == 2               # parts of at least 512 keys
    assert _prompt_splits(448, 2048, uniform=False) == 1              # a whole prompt: one round
    assert _prompt_splits(640, 16384, uniform=False) == 1             # tiles of a causal prompt differ in length: no rounds to even out
    assert _prompt_splits(640, 16384, uniform=True) == 4              # two rounds whole, five quarter rounds in four parts
    assert _prompt_splits(640, 1200, uniform=True) == 2
    assert _prompt_splits(1024, 16384, uniform=True) == 1             # two full rounds already
    assert _prompt_splits(1280, 16384, uniform=True) == 2             # 2.5 rounds: three whole, five half rounds in two parts
    assert _prompt_splits(512, 16384, uniform=True) == 1

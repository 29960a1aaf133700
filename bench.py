#!/usr/bin/python3
"""Benchmark of serving on one MI355X: decode throughput, prefill throughput, rooflines.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L] [--dtype bfloat16]
                    [--shape 7b|14b|32b] [--context N] [--new-tokens G] [--prefill-tokens T]
                    [--workload decode|serve] [--only decode|step|prefill] [--all]

The default run has the layer sizes of Qwen2.5-7B (28 layers, hidden 3584, 28 heads, 4 KV heads, head
size 128, intermediate 18944, vocabulary 152064) with random weights and goes through the whole engine
(scheduler, step function with decode steps replayed as HIP graphs and enqueued one ahead, sampler):
8 requests with 2048-token random prompts are prefilled by the engine and generate up to 256 tokens
each, greedily, with no stop token; after W untimed decode steps exactly K decode steps are timed.  It
prints ONE JSON line; ``value`` is decoded tokens per second.  Every figure of the line can be
recomputed from its own fields.  The same line carries

* ``roofline``: the bytes a decode step has to read (``bytes_per_step``: every weight it uses once,
  the embedding rows of the batch, and the cache of the live requests at their mean length over the timed
  steps) / its time, against the 8 TB/s of HBM3E (``frac``) and against the rate at which this GPU
  delivers memory to a kernel that only reads (``frac_measured``; ``measured`` holds that yardstick);
* ``step_function``: the same decode step driven directly (no scheduler): what the scheduler costs;
* ``prefill``: one 2048-token prompt in one step (tokens/s and ms as the mean of three timed runs, ``ms_best`` the
  fastest of them, flops, ``frac`` of the dense matrix-core peak of the dtype, ``frac_measured`` of the rate this
  repository's own large matrix product reaches);
* ``points``: decode tokens/s at batch 1 and batch 64 through the engine; ``points_detail`` gives each
  point's ms per step, bytes per step and fractions.

``--all`` adds the secondary workloads as ``extra`` (``--extra 14b,32b,fp32`` picks among them): Qwen2.5-14B sizes
served through the scheduler (32 requests, prompts 128-4096, 128 new tokens, 512 tokens a step); Qwen2.5-32B sizes
through the engine: one request whose 16384-token prompt the scheduler prefills in portions of 2048 tokens and that
then decodes 512 tokens greedily (``decode_32b_b1_ctx16384``, with the time of its prefill phase), and 16 requests
with 4096-token prompts (``decode_32b_b16_ctx4096``), each with the bare step function on synthetic caches as a
second figure (``step_function``), and the prefill of 16384 tokens as steps of the step function alone; and the same
32B sizes in true 32-bit, all 64 layers (``fp32_32b``: decode at batch 1 through the engine, prefill of 2048 tokens).
``--workload serve`` prints the serving run alone as a line of its own.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"bfloat16": 2500.0, "float32": 157.3}

QWEN25_7B = dict(
    architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584, num_hidden_layers=28,
    num_attention_heads=28, num_key_value_heads=4, intermediate_size=18944, max_position_embeddings=4096,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, use_sliding_window=False,
)
SHAPES = {
    "7b": ("Qwen2.5-7B", QWEN25_7B),
    "14b": ("Qwen2.5-14B", dict(QWEN25_7B, hidden_size=5120, num_hidden_layers=48, num_attention_heads=40,
                                 num_key_value_heads=8, intermediate_size=13824, rms_norm_eps=1e-5,
                                 max_position_embeddings=8192)),
    "32b": ("Qwen2.5-32B", dict(QWEN25_7B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=40,
                                 num_key_value_heads=8, intermediate_size=27648, rms_norm_eps=1e-5,
                                 max_position_embeddings=32768)),
}
CONTEXT = 2048
NEW_TOKENS = 256
PAGE = 16
PREFILL_BUDGET = 8192        # tokens a step of the engine may hold: four 2048-token prompts are prefilled at a time


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=224, help="timed decode steps")
    p.add_argument("--warmup", type=int, default=8, help="untimed decode steps before them")
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--shape", choices=list(SHAPES), default="7b", help="layer sizes")
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    p.add_argument("--context", type=int, default=CONTEXT, help="prompt tokens of each request in the decode runs")
    p.add_argument("--new-tokens", type=int, default=None, help="tokens each request may generate (decode: 256, serve: 128)")
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--workload", choices=["decode", "serve"], default="decode")
    p.add_argument("--requests", type=int, default=32)
    p.add_argument("--prompt-min", type=int, default=128)
    p.add_argument("--prompt-max", type=int, default=4096)
    p.add_argument("--portion", type=int, default=512, help="serve: token budget of a step")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points, the prefill and the yardsticks")
    p.add_argument("--only", choices=["decode", "step", "prefill"], default=None,
                   help="run one part only (for profiling): the engine's decode steps at --batch, the bare step function's, "
                        "or the prefill")
    p.add_argument("--all", action="store_true", help="add the secondary workloads (14B served, 32B prefill and decode, 32B in 32-bit)")
    p.add_argument("--extra", default=None, help="which secondary workloads, comma-separated: 14b, 32b, fp32 (implies --all)")
    return p.parse_args(argv)


def say(msg: str) -> None:
    """A line of progress on standard error (standard output carries the one JSON line)."""
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def build(shape: str, layers: int, dtype: str):
    import torch
    say(f"building {SHAPES[shape][0]} sizes, {layers} layers, {dtype}, random weights")
    from torchlet_amd.engine.loading import build_model
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import RandomTensors

    d = dict(SHAPES[shape][1], num_hidden_layers=layers)
    cfg = config_class(d["architectures"][0]).from_dict(d)
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    # every tensor drawn on the GPU as the model takes it: no second copy of the weights stands by
    # (the 32B sizes in 32-bit are 131 GB of the 288)
    model = build_model(cfg, dtype, tensors=RandomTensors(cfg, seed=2, dtype=store, device="cuda"))
    torch.cuda.empty_cache()
    return cfg, model


def decode_bytes(cfg, model, batch: int, context: float) -> float:
    """Bytes one decode step must read: every weight once (of the embedding only ``batch`` rows)
    and the keys and values of the live requests, ``context`` tokens each."""
    esize = 2 if str(model.dtype).endswith("bfloat16") else 4
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    per_layer = qkv * h + qkv + cfg.num_attention_heads * cfg.head_dim * h + 3 * h * i + 2 * h
    weights = (cfg.num_hidden_layers * per_layer + h + v * h + batch * h) * esize
    kv = batch * context * cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * esize
    return weights + kv


def prefill_flops(cfg, tokens: int) -> float:
    h, i, v = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    linear = cfg.num_hidden_layers * (qkv * h + cfg.num_attention_heads * cfg.head_dim * h + 3 * h * i)
    attn = cfg.num_hidden_layers * 2 * cfg.num_attention_heads * cfg.head_dim * tokens * tokens   # causal: half of 4*T^2
    return 2.0 * tokens * linear + attn + 2.0 * v * h


def random_prompts(vocab: int, count: int, length: int, seed: int = 0):
    import torch
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, vocab, (length,), generator=g).tolist() for _ in range(count)]


def engine_decode(cfg, model, batch: int, steps: int, warmup: int, context: int, new_tokens: int, budget: int = PREFILL_BUDGET) -> dict:
    """``batch`` requests with ``context``-token random prompts through the whole engine: the prompts are
    prefilled by the scheduler (portions under its token budget ``budget``), then every step decodes one token for
    each request.  The graphs of the decode steps are captured before the requests arrive; ``warmup`` decode steps
    are left untimed, ``steps`` are timed.  No stop token; nobody may finish before the timed steps are over."""
    import torch
    from torchlet_amd.engine.config import EngineConfig
    from torchlet_amd.engine.loading import make_engine
    from torchlet_amd.engine.request import Request

    say(f"engine: {batch} requests, {context}-token prompts, {warmup} + {steps} decode steps")
    pages = batch * (-(-(context + new_tokens) // PAGE)) + 1
    engine = make_engine(model, EngineConfig(page_size=PAGE, num_pages=pages, max_slots=batch, max_tokens_per_step=max(budget, batch),
                                             use_graphs=True, lookahead=True, seed=0))
    captured = engine.runner.warm_up(widths=[batch], max_len=context + new_tokens)     # ahead of need, as the Python entry point does
    reqs = [Request(prompt_tokens=p, max_new_tokens=new_tokens, temperature=0.0, stop_token_ids=frozenset())
            for p in random_prompts(cfg.vocab_size, batch, context)]
    engine.add_requests(reqs)
    finished = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    prefill_steps = engine.steps
    while any(not r.output_tokens for r in reqs):          # the prefill phase (with decode tokens of those already through)
        finished += engine.step()
    torch.cuda.synchronize()
    prefill_s = time.perf_counter() - t0
    prefill_steps = engine.steps - prefill_steps
    ahead = max(len(r.output_tokens) for r in reqs)
    if ahead + warmup + steps >= new_tokens:
        raise SystemExit(f"bench.py: {warmup} + {steps} decode steps after a prefill phase in which a request already generated "
                         f"{ahead} tokens do not fit {new_tokens} new tokens; lower --steps or raise --new-tokens")
    for _ in range(warmup):
        finished += engine.step()
    torch.cuda.synchronize()
    before = [len(r.output_tokens) for r in reqs]
    ctx0 = sum(r.computed_tokens for r in reqs) / batch
    t0 = time.perf_counter()
    for _ in range(steps):
        finished += engine.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(r.computed_tokens for r in reqs) / batch
    generated = sum(len(r.output_tokens) - b for r, b in zip(reqs, before))
    assert not finished and generated == batch * steps, (len(finished), generated)
    replays, ahead_steps = engine.runner.graph_replays, engine.steps_ahead
    engine.shutdown()
    del engine
    torch.cuda.empty_cache()
    ms = dt * 1e3 / steps
    mean_ctx = (ctx0 + ctx1) / 2.0 + 0.5      # keys a request's token attends to (its own included), averaged over the timed steps
    nbytes = decode_bytes(cfg, model, batch, mean_ctx)
    return {"batch": batch, "steps": steps, "ms_per_step": round(ms, 4), "tokens_per_s": round(batch * 1e3 / ms, 2),
            "mean_context": round(mean_ctx, 1), "bytes_per_step": int(nbytes), "graph_replays": replays, "steps_ahead": ahead_steps,
            "graphs_captured_ahead": captured, "prefill_phase_ms": round(prefill_s * 1e3, 2), "prefill_phase_steps": prefill_steps,
            "prefill_phase_tokens": batch * context}


def fill_context(runner, req_ids, context: int):
    """Give every request ``context`` cached tokens with random keys and values."""
    cache = runner.cache
    for r in req_ids:
        cache.add_request(r)
        if not cache.reserve(r, context):
            raise RuntimeError("cache pool too small for the benchmark")
        cache.commit(r, context)
    for g in cache.groups:
        for plane in g.tensors:
            plane.normal_(0.0, 0.5)


def step_function_decode(cfg, model, batch: int, steps: int, warmup: int, context: int) -> dict:
    """The decode step without the scheduler: the step function and the sampler driven directly, each step
    taking its tokens on the GPU from the sampling of the one before, on caches filled with random keys and
    values of ``context`` tokens (the time of a decode step does not depend on their values)."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    from torchlet_amd.sampling.sampler import Sampler

    say(f"step function: {batch} requests on {context}-token caches, {warmup} + {steps} decode steps")
    pages = batch * (-(-(context + steps + warmup + 2) // PAGE)) + 1
    runner = make_runner(model, page_size=PAGE, num_pages=pages, max_requests=batch, use_graphs=True)
    ids = [f"b{i}" for i in range(batch)]
    fill_context(runner, ids, context)
    sampler = Sampler(0)
    zeros = [0.0] * batch
    logits = runner.step([StepEntry(r, [1 + i], [0]) for i, r in enumerate(ids)])
    drawn = sampler.launch(logits, zeros, zeros, zeros)
    entries = [StepEntry(r, [0], [0]) for r in ids]
    generated = []

    def step():
        nonlocal drawn
        logits = runner.step(entries, device_tokens=(drawn.device, None))
        following = sampler.launch(logits, zeros, zeros, zeros)
        generated.append(drawn.tokens())
        drawn = following

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    assert len(generated) == warmup + steps and all(len(t) == batch for t in generated)
    del runner
    torch.cuda.empty_cache()
    mean_ctx = context + 1 + warmup + steps / 2.0
    return {"batch": batch, "steps": steps, "ms_per_step": round(ms, 4), "tokens_per_s": round(batch * 1e3 / ms, 2),
            "mean_context": round(mean_ctx, 1), "bytes_per_step": int(decode_bytes(cfg, model, batch, mean_ctx))}


def time_prefill(model, tokens: int, repeats: int = 3, context: int = 0):
    """(mean, best) ms of one step that brings ``tokens`` prompt tokens (after ``context`` tokens fed in 2048-token
    steps) over ``repeats`` runs after one that warms up."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner

    say(f"prefill: {tokens} tokens on {context} cached, {repeats} runs")
    runner = make_runner(model, page_size=PAGE, num_pages=-(-(context + tokens) // PAGE) + 2, max_requests=1)
    prompt = random_prompts(model.spec.vocab_size, 1, context + tokens)[0]
    times = []
    for i in range(repeats + 1):
        for a in range(0, context, 2048):
            runner.step([StepEntry("p", prompt[a:min(a + 2048, context)], [])])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("p", prompt[context:], [tokens - 1])])
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        runner.release("p")
        if i:                      # the first run warms up
            times.append(dt)
    del runner
    torch.cuda.empty_cache()
    return sum(times) / len(times), min(times)


def _best_ms(launch, rounds: int = 5, calls: int = 10) -> float:
    """ms of one call of ``launch``: ``calls`` of them back to back between two events (so that the host's
    part in a launch does not count), best of ``rounds`` after a warm-up round."""
    import torch
    best = float("inf")
    for i in range(rounds + 1):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(calls):
            launch()
        end.record()
        torch.cuda.synchronize()
        if i:
            best = min(best, start.elapsed_time(end) / calls)
    return best


def measure_stream_read_gbs() -> float:
    """GB/s at which a kernel that only reads gets 2 GiB from memory (far more than the caches hold)."""
    import torch
    from torchlet_amd.kernels import ops
    data = torch.empty(2 << 30, dtype=torch.uint8, device="cuda")
    data.random_(0, 255)
    ms = _best_ms(lambda: ops.stream_read(data))
    del data
    torch.cuda.empty_cache()
    return (2 << 30) / (ms * 1e-3) / 1e9


def measure_gemm_tflops(dtype) -> float:
    """TFLOP/s of this repository's own matrix product at 8192 x 8192 x 8192 (float32: 4096 cubed)."""
    import torch
    from torchlet_amd.kernels import ops
    n = 8192 if dtype == torch.bfloat16 else 4096
    x = torch.randn((n, n), device="cuda").to(dtype)
    w = torch.randn((n, n), device="cuda").to(dtype)
    out = torch.empty((n, n), dtype=dtype, device="cuda")
    ms = _best_ms(lambda: ops.linear(x, w, None, out), rounds=3, calls=4)
    del x, w, out
    torch.cuda.empty_cache()
    return 2.0 * n ** 3 / (ms * 1e-3) / 1e12


def serve(cfg, model, args) -> dict:
    """Requests through the whole engine: prompts of seeded random lengths, all arriving at
    once, cut into portions under the step's token budget beside the decode tokens of the
    requests that are further on; every request generates ``--new-tokens`` (no stop ids)."""
    import torch
    from torchlet_amd.engine.config import EngineConfig
    from torchlet_amd.engine.loading import make_engine
    from torchlet_amd.engine.request import Request

    g = torch.Generator().manual_seed(1)
    lengths = torch.randint(args.prompt_min, args.prompt_max + 1, (args.requests,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lengths]
    new_tokens = args.serve_new_tokens
    pages = sum(-(-(n + new_tokens) // PAGE) for n in lengths) + 1
    engine = make_engine(model, EngineConfig(page_size=PAGE, num_pages=pages, max_slots=args.requests, max_tokens_per_step=args.portion,
                                             dtype=args.dtype, use_graphs=True, seed=0))

    def run():
        say(f"serving {len(prompts)} requests, {sum(lengths)} prompt tokens, {new_tokens} new tokens each")
        engine.add_requests([Request(prompt_tokens=list(p), max_new_tokens=new_tokens) for p in prompts])
        steps0 = engine.steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = engine.run_until_done()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(done) == len(prompts) and all(len(r.output_tokens) == new_tokens for r in done)
        return dt, engine.steps - steps0

    run()                                   # warms up kernels and captures the decode graphs
    dt, steps = run()
    generated = args.requests * new_tokens
    del engine
    torch.cuda.empty_cache()
    return {
        "metric": f"served tokens/s, {SHAPES[args.shape][0]} shape, {args.requests} requests, prompts {args.prompt_min}-{args.prompt_max}, "
                  f"{new_tokens} new tokens each, at most {args.portion} tokens a step, one MI355X",
        "value": round((sum(lengths) + generated) / dt, 1), "unit": "tokens/s (prompt + generated)",
        "generated_tokens_per_s": round(generated / dt, 1), "prompt_tokens": sum(lengths), "generated_tokens": generated,
        "seconds": round(dt, 3), "engine_steps": steps, "ms_per_step": round(dt * 1e3 / steps, 3),
        "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "layers": cfg.num_hidden_layers,
        "data": "synthetic: seeded random weights, prompt lengths and token ids",
    }


def _with_roofline(r: dict) -> dict:
    gbs = r["bytes_per_step"] / (r["ms_per_step"] * 1e-3) / 1e9
    return dict(r, achieved_gbs=round(gbs, 1), frac=round(gbs / HBM_PEAK_GBS, 4))


def secondary_14b(args) -> dict:
    """14B sizes, all 48 layers, served: 32 requests, prompts 128-4096, 128 new tokens, 512 tokens a step."""
    import torch
    cfg, model = build("14b", SHAPES["14b"][1]["num_hidden_layers"], args.dtype)
    a = argparse.Namespace(**vars(args))
    a.shape, a.requests, a.prompt_min, a.prompt_max, a.serve_new_tokens, a.portion = "14b", 32, 128, 4096, 128, 512
    s = serve(cfg, model, a)
    del model
    torch.cuda.empty_cache()
    return {"serve_14b": {k: s[k] for k in ("value", "unit", "generated_tokens_per_s", "prompt_tokens", "generated_tokens", "seconds",
                                            "engine_steps", "ms_per_step", "layers")}}


def secondary_32b(args) -> dict:
    """32B sizes, all 64 layers, through the engine: one request with a 16384-token prompt (prefilled by the
    scheduler in portions of 2048 tokens) that decodes 512 tokens greedily, and 16 requests with 4096-token
    prompts; beside each the bare step function on synthetic caches, and the long prefill as steps of the step
    function alone."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    out = {}
    cfg, model = build("32b", SHAPES["32b"][1]["num_hidden_layers"], args.dtype)
    tokens = 16384
    runner = make_runner(model, page_size=PAGE, num_pages=-(-tokens // PAGE) + 2, max_requests=1)
    prompt = random_prompts(cfg.vocab_size, 1, tokens)[0]
    times = []
    for rep in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for a0 in range(0, tokens, 2048):
            runner.step([StepEntry("p", prompt[a0:a0 + 2048], [2047] if a0 + 2048 == tokens else [])])
        torch.cuda.synchronize()
        total = time.perf_counter() - t0
        runner.release("p")
        if rep:
            times.append(total)
    del runner
    torch.cuda.empty_cache()
    mean, best = sum(times) / len(times), min(times)
    flops = sum(prefill_flops_step(cfg, 2048, a0) for a0 in range(0, tokens, 2048))
    out["prefill_32b_16384"] = {"tokens": tokens, "steps_of": 2048, "ms": round(mean * 1e3, 2), "ms_best": round(best * 1e3, 2), "runs": len(times),
                                "value": round(tokens / mean, 1), "flops": flops,
                                "frac": round(flops / mean / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4), "layers": cfg.num_hidden_layers}
    # (name, requests, prompt tokens, new tokens, timed decode steps, token budget of a step)
    for name, batch, context, new_tokens, steps, budget in (("decode_32b_b1_ctx16384", 1, 16384, 512, 480, 2048),
                                                           ("decode_32b_b16_ctx4096", 16, 4096, 128, 96, 8192)):
        r = _with_roofline(engine_decode(cfg, model, batch, steps, 8, context, new_tokens, budget=budget))
        r["prefill_phase_flops"] = batch * sum(prefill_flops_step(cfg, min(2048, context - a0), a0) for a0 in range(0, context, 2048))
        r["prefill_phase_tokens_per_s"] = round(r["prefill_phase_tokens"] / (r["prefill_phase_ms"] * 1e-3), 1)
        r["step_function"] = _with_roofline(step_function_decode(cfg, model, batch, 32, 4, context))
        r["layers"], r["new_tokens"], r["token_budget"] = cfg.num_hidden_layers, new_tokens, budget
        out[name] = r
    del model
    torch.cuda.empty_cache()
    return out


def secondary_fp32_32b(args) -> dict:
    """32B sizes in true 32-bit, all 64 layers (131 GB of weights): decode at batch 1 through the engine after a
    2048-token prompt, and the prefill of 2048 tokens as one step."""
    import torch
    cfg, model = build("32b", SHAPES["32b"][1]["num_hidden_layers"], "float32")
    r = _with_roofline(engine_decode(cfg, model, 1, 32, 4, 2048, 64, budget=2048))
    pms, pbest = time_prefill(model, 2048, repeats=2)
    flops = prefill_flops(cfg, 2048)
    out = {"dtype": "fp32", "layers": cfg.num_hidden_layers, "weight_bytes": int(decode_bytes(cfg, model, 1, 0)),
           "decode_b1": r,
           "prefill": {"value": round(2048 * 1e3 / pms, 1), "tokens": 2048, "ms": round(pms, 2), "ms_best": round(pbest, 2), "runs": 2,
                       "flops": flops, "frac": round(flops / (pms * 1e-3) / (MFMA_PEAK_TFLOPS["float32"] * 1e12), 4)}}
    del model
    torch.cuda.empty_cache()
    return {"fp32_32b": out}


def secondary(args) -> dict:
    """The secondary workloads, each at its full layer count."""
    which = [w.strip() for w in (args.extra or "14b,32b,fp32").split(",") if w.strip()]
    parts = {"14b": secondary_14b, "32b": secondary_32b, "fp32": secondary_fp32_32b}
    unknown = [w for w in which if w not in parts]
    if unknown:
        raise SystemExit(f"bench.py: --extra knows 14b, 32b and fp32, not {', '.join(unknown)}")
    out = {}
    for w in which:
        out.update(parts[w](args))
    return out


def prefill_flops_step(cfg, tokens: int, context: int) -> float:
    """Flops of a step of ``tokens`` prompt tokens on top of ``context`` cached ones (no logits)."""
    h, i = cfg.hidden_size, cfg.intermediate_size
    qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
    linear = cfg.num_hidden_layers * (qkv * h + cfg.num_attention_heads * cfg.head_dim * h + 3 * h * i)
    keys = tokens * context + tokens * tokens / 2.0
    attn = cfg.num_hidden_layers * 4 * cfg.num_attention_heads * cfg.head_dim * keys
    return 2.0 * tokens * linear + attn


def main(argv=None) -> int:
    args = parse_args(argv)
    args.serve_new_tokens = args.new_tokens or 128
    args.new_tokens = args.new_tokens or NEW_TOKENS
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not built (this engine runs on a single MI355X)")
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X; no GPU is visible", file=sys.stderr)
        return 1
    name, sizes = SHAPES[args.shape]
    full_layers = sizes["num_hidden_layers"]
    layers = args.layers if args.layers is not None else full_layers
    cfg, model = build(args.shape, layers, args.dtype)
    ptokens = args.prefill_tokens
    peak_tflops = MFMA_PEAK_TFLOPS[args.dtype]

    def prefill_point(gemm_tflops=None):
        pms, pbest = time_prefill(model, ptokens)
        flops = prefill_flops(cfg, ptokens)
        point = {"value": round(ptokens * 1e3 / pms, 1), "tokens": ptokens, "ms": round(pms, 3), "ms_best": round(pbest, 3), "runs": 3,
                 "flops": flops, "frac": round(flops / (pms * 1e-3) / (peak_tflops * 1e12), 4)}
        if gemm_tflops:
            point["frac_measured"] = round(flops / (pms * 1e-3) / (gemm_tflops * 1e12), 4)
        return point

    if args.workload == "serve":
        print(json.dumps(serve(cfg, model, args)))
        return 0
    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_point(), "layers": layers}))
        return 0
    if args.only == "step":
        print(json.dumps({"step_function": step_function_decode(cfg, model, args.batch, min(args.steps, 64), args.warmup, args.context),
                          "layers": layers}))
        return 0
    if args.only == "decode":
        args.no_points = True
    head = engine_decode(cfg, model, args.batch, args.steps, args.warmup, args.context, args.new_tokens)
    ms = head["ms_per_step"]
    achieved = head["bytes_per_step"] / (ms * 1e-3) / 1e9
    result = {
        "metric": f"decode tokens/s, {name} shape, batch {args.batch}, {args.context}-token prompts, {args.new_tokens} new tokens, "
                  f"through the engine, one MI355X",
        "value": head["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": f"synthetic: seeded random weights and token ids; {args.context}-token random prompts prefilled by the engine, "
                f"greedy decoding with no stop token",
        "config": {
            "model": f"{name} shape (Qwen2ForCausalLM)", "layers": layers, "layers_full_model": full_layers,
            "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "new_tokens": args.new_tokens,
            "context_limit": cfg.max_position_embeddings, "page_size": PAGE, "prefill_tokens": ptokens,
            "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "bytes_per_step": head["bytes_per_step"],
                     "mean_context": head["mean_context"]},
        "engine": {"graph_replays": head["graph_replays"], "steps_ahead": head["steps_ahead"]},
    }
    if not args.no_points:
        stream_gbs = measure_stream_read_gbs()
        gemm_tflops = measure_gemm_tflops(model.dtype)
        result["measured"] = {"stream_read_gbs": round(stream_gbs, 1), "gemm_tflops": round(gemm_tflops, 1),
                              "how": "a kernel of this repository that only reads 2 GiB; its own 8192-cubed matrix product"}
        result["roofline"]["frac_measured"] = round(achieved / stream_gbs, 4)
        bare = step_function_decode(cfg, model, args.batch, 64, args.warmup, args.context)
        result["step_function"] = bare
        result["prefill"] = prefill_point(gemm_tflops)
        points, detail = {}, {}
        for b in (1, 64):
            r = engine_decode(cfg, model, b, max(8, args.steps // 2), max(2, args.warmup // 2), args.context, args.new_tokens)
            gbs = r["bytes_per_step"] / (r["ms_per_step"] * 1e-3) / 1e9
            points[f"decode_b{b}"] = r["tokens_per_s"]
            detail[f"decode_b{b}"] = {"ms_per_step": r["ms_per_step"], "steps": r["steps"], "bytes_per_step": r["bytes_per_step"],
                                      "mean_context": r["mean_context"], "achieved_gbs": round(gbs, 1),
                                      "frac": round(gbs / HBM_PEAK_GBS, 4), "frac_measured": round(gbs / stream_gbs, 4)}
        result["points"] = points
        result["points_detail"] = detail
    if args.all or args.extra:
        del model
        torch.cuda.empty_cache()
        result["extra"] = secondary(args)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())

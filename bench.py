#!/usr/bin/python3
"""Benchmark of the serving step on one MI355X: decode throughput, prefill throughput, rooflines.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bfloat16]
                    [--shape 7b|14b|32b] [--context N] [--prefill-tokens T] [--workload decode|serve]

The default run has the layer sizes of Qwen2.5-7B (28 layers, hidden 3584, 28 heads, 4 KV
heads, head size 128, intermediate 18944, vocabulary 152064) with random weights, a batch
of 8 requests that each hold a 2048-token context, and times K decode steps (one new token
per request and step, sampled greedily) through the engine's own step function and sampler.
It prints ONE JSON line; ``value`` is decoded tokens per second.  The same line carries

* ``prefill``: one 2048-token prompt in one step (tokens/s, ms, fraction of the dense
  matrix-core peak of the dtype: flops / time / peak),
* ``roofline``: bytes a decode step has to read (every weight it uses once, plus the cache
  of the live requests) / its time, against the 8 TB/s of HBM3E,
* ``points``: decode tokens/s at batch 1 and batch 64.

Caches of the decode runs are filled with random keys and values of 2048-token contexts
through the cache manager (the time of a decode step does not depend on their values).

Other layer sizes (``--shape 14b``, ``32b``), context lengths and prompt lengths measure the same
step at further sizes.  ``--workload serve`` runs requests through the whole engine instead
(scheduler, prompt portions under a token budget beside decode tokens, sampler): ``--requests``
prompts of random lengths in ``[--prompt-min, --prompt-max]``, ``--new-tokens`` each, at most
``--portion`` tokens per step, and prints a line of its own.
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
PAGE = 16


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--shape", choices=list(SHAPES), default="7b", help="layer sizes")
    p.add_argument("--layers", type=int, default=None, help="fewer layers than the model has (named in config)")
    p.add_argument("--context", type=int, default=CONTEXT, help="cached tokens of each request in the decode runs")
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--workload", choices=["decode", "serve"], default="decode")
    p.add_argument("--requests", type=int, default=32)
    p.add_argument("--prompt-min", type=int, default=128)
    p.add_argument("--prompt-max", type=int, default=4096)
    p.add_argument("--new-tokens", type=int, default=128)
    p.add_argument("--portion", type=int, default=512, help="serve: token budget of a step")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    p.add_argument("--only", choices=["decode", "prefill"], default=None,
                   help="run one part only (for profiling): the decode steps at --batch, or the 2048-token prefill")
    return p.parse_args(argv)


def build(shape: str, layers: int, dtype: str):
    import torch
    from torchlet_amd.engine.loading import build_model
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import random_tensors

    d = dict(SHAPES[shape][1], num_hidden_layers=layers)
    cfg = config_class(d["architectures"][0]).from_dict(d)
    store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    tensors = random_tensors(cfg, seed=2, dtype=store, device="cuda")
    model = build_model(cfg, dtype, tensors=tensors)
    del tensors
    torch.cuda.empty_cache()
    return cfg, model


def decode_bytes(cfg, model, batch: int, context: float) -> float:
    """Bytes one decode step must read: every weight once (the embedding only ``batch`` rows
    of it) and the keys and values of the live requests."""
    esize = 2 if model.dtype.__str__().endswith("bfloat16") else 4
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


def fill_context(runner, req_ids, context: int):
    """Give every request ``context`` cached tokens with random keys and values."""
    import torch
    cache = runner.cache
    for r in req_ids:
        cache.add_request(r)
        if not cache.reserve(r, context):
            raise RuntimeError("cache pool too small for the benchmark")
        cache.commit(r, context)
    for g in cache.groups:
        for plane in g.tensors:
            plane.normal_(0.0, 0.5)


def time_decode(model, batch: int, steps: int, warmup: int, context: int = CONTEXT):
    """ms per decode step at ``batch`` requests of ``context`` cached tokens each."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    from torchlet_amd.sampling.sampler import Sampler

    pages = batch * (-(-(context + steps + warmup + 2) // PAGE)) + 1
    runner = make_runner(model, page_size=PAGE, num_pages=pages, max_requests=batch, use_graphs=True)
    ids = [f"b{i}" for i in range(batch)]
    fill_context(runner, ids, context)
    sampler = Sampler(0)
    zeros = [0.0] * batch
    # As the engine runs decode steps: a step takes its tokens on the GPU from the sampling of the step
    # before it and is enqueued while the host still waits for those tokens; every token is read.
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
    return ms


def time_prefill(model, tokens: int, repeats: int = 3):
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner

    runner = make_runner(model, page_size=PAGE, num_pages=-(-tokens // PAGE) + 2, max_requests=1)
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, model.spec.vocab_size, (tokens,), generator=g).tolist()
    best = float("inf")
    for i in range(repeats + 1):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.step([StepEntry("p", prompt, [tokens - 1])])
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        runner.release("p")
        if i:                      # the first run warms up
            best = min(best, dt)
    del runner
    torch.cuda.empty_cache()
    return best


def serve(cfg, model, args) -> dict:
    """Requests through the whole engine: prompts of seeded random lengths, all arriving at
    once, cut into portions under the step's token budget beside the decode tokens of the
    requests that are further on; every request generates ``--new-tokens`` (no stop ids)."""
    import torch
    from torchlet_amd.engine.engine import Engine
    from torchlet_amd.engine.loading import make_runner
    from torchlet_amd.engine.request import Request

    g = torch.Generator().manual_seed(1)
    lengths = torch.randint(args.prompt_min, args.prompt_max + 1, (args.requests,), generator=g).tolist()
    prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist() for n in lengths]
    pages = sum(-(-(n + args.new_tokens) // PAGE) for n in lengths) + 1
    runner = make_runner(model, page_size=PAGE, num_pages=pages, max_requests=args.requests, use_graphs=True)
    engine = Engine(runner, max_tokens_per_step=args.portion, seed=0)

    def run():
        for p in prompts:
            engine.add_request(Request(prompt_tokens=list(p), max_new_tokens=args.new_tokens))
        steps0 = engine.steps
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        done = engine.run_until_done()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert len(done) == len(prompts) and all(len(r.output_tokens) == args.new_tokens for r in done)
        return dt, engine.steps - steps0

    run()                                   # warms up kernels and captures the decode graphs
    dt, steps = run()
    generated = args.requests * args.new_tokens
    return {
        "metric": f"served tokens/s, {SHAPES[args.shape][0]} shape, {args.requests} requests, prompts {args.prompt_min}-{args.prompt_max}, "
                  f"{args.new_tokens} new tokens each, at most {args.portion} tokens a step, one MI355X",
        "value": round((sum(lengths) + generated) / dt, 1), "unit": "tokens/s (prompt + generated)",
        "generated_tokens_per_s": round(generated / dt, 1), "prompt_tokens": sum(lengths), "generated_tokens": generated,
        "seconds": round(dt, 3), "engine_steps": steps, "ms_per_step": round(dt * 1e3 / steps, 3),
        "n_gpus": 1, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "layers": cfg.num_hidden_layers,
        "data": "synthetic: seeded random weights, prompt lengths and token ids",
    }


def main(argv=None) -> int:
    args = parse_args(argv)
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

    def prefill_point():
        pms = time_prefill(model, ptokens)
        flops = prefill_flops(cfg, ptokens)
        return {"value": round(ptokens * 1e3 / pms, 1), "tokens": ptokens, "ms": round(pms, 3),
                "frac": round(flops / (pms * 1e-3) / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4)}

    if args.workload == "serve":
        print(json.dumps(serve(cfg, model, args)))
        return 0
    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_point(), "layers": layers}))
        return 0
    if args.only == "decode":
        args.no_points = True
    ms = time_decode(model, args.batch, args.steps, args.warmup, args.context)
    mean_ctx = args.context + args.warmup + args.steps / 2.0
    nbytes = decode_bytes(cfg, model, args.batch, mean_ctx)
    achieved = nbytes / (ms * 1e-3) / 1e9
    result = {
        "metric": f"decode tokens/s, {name} shape, batch {args.batch}, {args.context}-token contexts, one MI355X",
        "value": round(args.batch * 1e3 / ms, 2),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": f"synthetic: seeded random weights and token ids; decode caches hold random keys/values of {args.context}-token contexts",
        "config": {
            "model": f"{name} shape (Qwen2ForCausalLM)", "layers": layers, "layers_full_model": full_layers,
            "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": args.context, "context_limit": cfg.max_position_embeddings,
            "page_size": PAGE, "prefill_tokens": ptokens, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        result["prefill"] = prefill_point()
        points = {}
        for b in (1, 64):
            pm = time_decode(model, b, max(8, args.steps // 2), max(2, args.warmup // 2), args.context)
            points[f"decode_b{b}"] = round(b * 1e3 / pm, 2)
        result["points"] = points
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())

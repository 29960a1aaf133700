#!/usr/bin/python3
"""Benchmark of the serving step on one MI355X: decode throughput, prefill throughput, rooflines.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--dtype bfloat16]

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
FULL_LAYERS = QWEN25_7B["num_hidden_layers"]
CONTEXT = 2048
PAGE = 16


def parse_args(argv=None):
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--layers", type=int, default=FULL_LAYERS, help="fewer layers than the model has (named in config)")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    p.add_argument("--only", choices=["decode", "prefill"], default=None,
                   help="run one part only (for profiling): the decode steps at --batch, or the 2048-token prefill")
    return p.parse_args(argv)


def build(layers: int, dtype: str):
    import torch
    from torchlet_amd.engine.loading import build_model
    from torchlet_amd.registry import config_class
    from torchlet_amd.weights.random_init import random_tensors

    d = dict(QWEN25_7B, num_hidden_layers=layers)
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
        g.tensor.normal_(0.0, 0.5)


def time_decode(model, batch: int, steps: int, warmup: int):
    """ms per decode step at ``batch`` requests of ``CONTEXT`` cached tokens each."""
    import torch
    from torchlet_amd.engine.batch import StepEntry
    from torchlet_amd.engine.loading import make_runner
    from torchlet_amd.sampling.sampler import Sampler

    pages = batch * (-(-(CONTEXT + steps + warmup + 1) // PAGE)) + 1
    runner = make_runner(model, page_size=PAGE, num_pages=pages, max_requests=batch, use_graphs=True)
    ids = [f"b{i}" for i in range(batch)]
    fill_context(runner, ids, CONTEXT)
    sampler = Sampler(0)
    tokens = [1 + i for i in range(batch)]
    zeros = [0.0] * batch

    def step():
        nonlocal tokens
        logits = runner.step([StepEntry(r, [t], [0]) for r, t in zip(ids, tokens)])
        tokens = sampler.sample(logits, zeros, zeros, zeros)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
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


def main(argv=None) -> int:
    args = parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not built (this engine runs on a single MI355X)")
        return 2
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X; no GPU is visible", file=sys.stderr)
        return 1
    cfg, model = build(args.layers, args.dtype)
    if args.only == "prefill":
        pms = time_prefill(model, 2048)
        flops = prefill_flops(cfg, 2048)
        print(json.dumps({"prefill": {"value": round(2048 * 1e3 / pms, 1), "tokens": 2048, "ms": round(pms, 3),
                                      "frac": round(flops / (pms * 1e-3) / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4)},
                          "layers": args.layers}))
        return 0
    if args.only == "decode":
        args.no_points = True
    ms = time_decode(model, args.batch, args.steps, args.warmup)
    mean_ctx = CONTEXT + args.warmup + args.steps / 2.0
    nbytes = decode_bytes(cfg, model, args.batch, mean_ctx)
    achieved = nbytes / (ms * 1e-3) / 1e9
    result = {
        "metric": f"decode tokens/s, Qwen2.5-7B shape, batch {args.batch}, 2048-token contexts, one MI355X",
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
        "data": "synthetic: seeded random weights and token ids; decode caches hold random keys/values of 2048-token contexts",
        "config": {
            "model": "Qwen2.5-7B shape (Qwen2ForCausalLM)", "layers": args.layers, "layers_full_model": FULL_LAYERS,
            "hidden_size": cfg.hidden_size, "num_attention_heads": cfg.num_attention_heads,
            "num_key_value_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
            "global_batch": args.batch, "seq_len": CONTEXT, "context_limit": cfg.max_position_embeddings,
            "page_size": PAGE, "prefill_tokens": 2048, "parallelism": "single GPU",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        pms = time_prefill(model, 2048)
        flops = prefill_flops(cfg, 2048)
        result["prefill"] = {"value": round(2048 * 1e3 / pms, 1), "tokens": 2048, "ms": round(pms, 3),
                             "frac": round(flops / (pms * 1e-3) / (MFMA_PEAK_TFLOPS[args.dtype] * 1e12), 4)}
        points = {}
        for b in (1, 64):
            pm = time_decode(model, b, max(8, args.steps // 2), max(2, args.warmup // 2))
            points[f"decode_b{b}"] = round(b * 1e3 / pm, 2)
        result["points"] = points
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())

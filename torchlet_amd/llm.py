"""The Python entry point and the command line.

In the manner of the reference's ``LLM`` (/root/reference/src/torchlet/
v10_triton_paged_gqa/llm.py:20-110): ``LLM(model_id, max_decode_slots=4, kv_block_size=16,
max_num_blocks=None)`` and ``generate(inputs, max_new_tokens=128)``, with the same names and
meanings: ``max_decode_slots`` is the most requests live at a time, ``kv_block_size`` the
tokens per cache page, ``max_num_blocks`` the pages of the pool including the sentinel
(default ``max_decode_slots * ceil(max_position_embeddings / kv_block_size) + 1``,
engine.py:40-47 of the reference, capped by free GPU memory).  ``model_id`` is a local
model folder (nothing is downloaded).  Additions: ``dtype`` (default: the folder's own, its ``torch_dtype`` or the
element type it stores, as the reference runs a checkpoint in the dtype it is stored in, utils.py:18-38;
``bfloat16`` or ``float32`` converts at load), ``max_num_batched_tokens`` (the
step's token budget), ``max_model_len`` (sequences no longer than this: a smaller default pool), ``seed``,
``use_graphs`` (decode-only steps replay a captured HIP graph); or all of them at once as an
:class:`~torchlet_amd.engine.config.EngineConfig` (``engine_config=``).  ``generate`` also takes ``temperature``,
``seed`` and ``stop_token_ids``, and accepts prompts as lists of token ids, which bypass the tokenizer.

Strings are wrapped as a single user turn and run through the tokenizer's chat template
with the generation prompt (llm.py:87-96); the stop ids are the tokenizer's end-of-sequence
id and ``<|im_end|>`` (llm.py:40-44); output text skips special tokens (engine.py:194-196).
The tokenizer is read from the folder's ``tokenizer.json`` with the ``tokenizers`` library.

    python -m torchlet_amd --model DIR --prompt "hello" --max-new-tokens 64
    python -m torchlet_amd --model DIR --prompt-ids 1,2,3 --temperature 0.8 --seed 1
    python -m torchlet_amd init --config config.json --seed 0 --out DIR     # random weights
    python -m torchlet_amd replay --model DIR --dtype float32 --out DIR --max-tokens N < steps.jsonl    # = bin/trace_run
"""
from __future__ import annotations

import argparse
import asyncio
import json
import sys
from pathlib import Path

from .engine.config import EngineConfig
from .engine.loading import load_model, make_engine, require_gpu
from .engine.request import Request
from .logger import backend_info, logger, weights_info


class LLM:
    def __init__(self, model_id: str, max_decode_slots: int = 4, kv_block_size: int = 16,
                 max_num_blocks: int | None = None, *, dtype: str | None = None,
                 max_num_batched_tokens: int = 2048, max_model_len: int | None = None, seed: int = 0,
                 use_graphs: bool = True, lookahead: bool = True, engine_config: EngineConfig | None = None):
        self.device = require_gpu()
        if kv_block_size <= 0:
            raise ValueError("kv_block_size must be positive")
        if max_decode_slots <= 0:
            raise ValueError("max_decode_slots must be positive")
        self.engine_config = engine_config or EngineConfig(
            page_size=kv_block_size, num_pages=max_num_blocks, max_slots=max_decode_slots,
            max_tokens_per_step=max_num_batched_tokens, max_model_len=max_model_len, dtype=None if dtype is None else str(dtype).replace("torch.", ""),
            use_graphs=use_graphs, lookahead=lookahead, seed=seed)
        self.model_dir = Path(model_id)
        if logger.isEnabledFor(20):                         # INFO: the start-up reports of the reference's LLM (llm.py:28-36)
            from .weights.loader import SafetensorsFolder
            logger.info("backend:\n%s", backend_info())
            logger.info("tensors of %s:\n%s", self.model_dir, weights_info(SafetensorsFolder(self.model_dir)))
        self.config, self.model = load_model(self.model_dir, self.engine_config.dtype, self.device)
        self.engine = make_engine(self.model, self.engine_config)
        self.runner = self.engine.runner
        self.engine_config = self.runner.config            # with the dtype and the number of pages filled in
        self.graphs_captured = self.runner.warm_up()       # ahead of need: no serving step stops to capture one
        logger.info("model: %s, %d runs of %d layers, %s; engine: %s; cache: %s pages free per group, %d bytes a page",
                    self.config.architecture, len(self.model.spec.order), len(self.model.spec.layers), self.model.dtype,
                    self.engine_config, self.runner.cache.free_pages(), self.runner.cache.bytes_per_page())
        self.tokenizer = _load_tokenizer(self.model_dir)
        self.stop_ids = self._stop_ids()
        self._next_seed = 0

    def _stop_ids(self) -> frozenset:
        ids = set()
        eos = getattr(self.config, "eos_token_id", -1)
        if isinstance(eos, int) and eos >= 0:
            ids.add(eos)
        if self.tokenizer is not None:
            ids |= self.tokenizer.stop_ids()
        return frozenset(ids)

    def _requests(self, inputs, max_new_tokens, temperature, seed, stop_token_ids) -> list[Request]:
        stop = self.stop_ids if stop_token_ids is None else frozenset(stop_token_ids)
        reqs = []
        for i, item in enumerate(inputs):
            if isinstance(item, str):
                if self.tokenizer is None:
                    raise ValueError(f"{self.model_dir} has no tokenizer.json; give prompts as lists of token ids")
                text, ids = self.tokenizer.encode_chat(item)
            else:
                text, ids = "", [int(t) for t in item]
            if seed is None:
                s, self._next_seed = self._next_seed, self._next_seed + 1
            else:
                s = int(seed) + i
            reqs.append(Request(prompt_tokens=ids, max_new_tokens=max_new_tokens, temperature=float(temperature),
                                seed=s, stop_token_ids=stop, prompt=text))
        return reqs

    def generate(self, inputs, max_new_tokens: int = 128, *, temperature: float = 0.0, seed: int | None = None,
                 stop_token_ids=None):
        """Generate for every input; strings give strings, token-id lists give token-id lists."""
        if not inputs:
            return []
        if max_new_tokens <= 0:
            return ["" if isinstance(x, str) else [] for x in inputs]
        reqs = self._requests(inputs, max_new_tokens, temperature, seed, stop_token_ids)
        self.engine.add_requests(reqs)          # all or none: a bad request leaves nothing queued
        self.engine.run_until_done()
        return self._outputs(inputs, reqs)

    async def generate_async(self, inputs, max_new_tokens: int = 128, **kw):
        """Coroutine form, as the reference's ``generate`` is from its fourth version on:
        requests of concurrent callers share the engine's steps (continuous batching)."""
        if not inputs:
            return []
        if max_new_tokens <= 0:
            return ["" if isinstance(x, str) else [] for x in inputs]
        reqs = self._requests(inputs, max_new_tokens, kw.get("temperature", 0.0), kw.get("seed"), kw.get("stop_token_ids"))
        self.engine.add_requests(reqs)
        while any(r.finish_reason is None for r in reqs):
            try:
                self.engine.step()
            except Exception as exc:
                self.engine.fail_all(exc)
                raise
            await asyncio.sleep(0)
        self.engine.scheduler.drain_finished()
        return self._outputs(inputs, reqs)

    def _outputs(self, inputs, reqs):
        out = []
        for item, r in zip(inputs, reqs):
            if r.error is not None:
                raise r.error
            if isinstance(item, str):
                r.output = self.tokenizer.decode(r.output_tokens)
                out.append(r.output)
            else:
                out.append(list(r.output_tokens))
        return out


class _Tokenizer:
    """``tokenizer.json`` through the ``tokenizers`` library, plus the folder's chat template."""

    def __init__(self, folder: Path):
        from tokenizers import Tokenizer
        self.tok = Tokenizer.from_file(str(folder / "tokenizer.json"))
        cfg_path = folder / "tokenizer_config.json"
        self.cfg = json.loads(cfg_path.read_text()) if cfg_path.exists() else {}
        self.template = self.cfg.get("chat_template")

    def _token_text(self, key):
        v = self.cfg.get(key)
        return v.get("content") if isinstance(v, dict) else v

    def stop_ids(self) -> set:
        ids = set()
        for text in (self._token_text("eos_token"), "<|im_end|>"):
            if text:
                i = self.tok.token_to_id(text)
                if i is not None:
                    ids.add(i)
        return ids

    def encode_chat(self, user_text: str):
        text = render_chat_template(self.template, user_text, self._token_text("bos_token") or "",
                                    self._token_text("eos_token") or "") if self.template else user_text
        return text, self.tok.encode(text, add_special_tokens=False).ids

    def decode(self, ids) -> str:
        return self.tok.decode(list(ids), skip_special_tokens=True)


def render_chat_template(template: str, user_text: str, bos_token: str = "", eos_token: str = "") -> str:
    """One user turn with the generation prompt through a model folder's chat template.  The template
    is text from the model folder and is not trusted: it runs in jinja2's immutable sandbox, where
    reaching for ``__class__``, ``__globals__`` and the like, or changing a passed object, raises
    ``jinja2.exceptions.SecurityError`` (the reference goes through ``apply_chat_template``, llm.py:87-96,
    which renders in the same kind of sandbox)."""
    import jinja2
    from jinja2.sandbox import ImmutableSandboxedEnvironment

    def raise_exception(message):
        raise jinja2.exceptions.TemplateError(message)

    env = ImmutableSandboxedEnvironment(trim_blocks=True, lstrip_blocks=True)
    env.globals["raise_exception"] = raise_exception
    return env.from_string(template).render(messages=[{"role": "user", "content": user_text}], add_generation_prompt=True,
                                            bos_token=bos_token, eos_token=eos_token)


def _load_tokenizer(folder: Path):
    return _Tokenizer(folder) if (folder / "tokenizer.json").exists() else None


# ------------------------------------------------------------------------ command line

def _parser():
    p = argparse.ArgumentParser(prog="python -m torchlet_amd", description="Qwen2.5 inference on one MI355X")
    sub = p.add_subparsers(dest="command")
    g = sub.add_parser("generate", help="generate from prompts (the default command)")
    for q in (p, g):
        q.add_argument("--model", help="model folder: config.json, *.safetensors, optionally tokenizer.json")
        q.add_argument("--prompt", action="append", default=[], help="a prompt string (repeatable)")
        q.add_argument("--prompt-ids", action="append", default=[], help="a prompt as comma-separated token ids (repeatable)")
        q.add_argument("--max-new-tokens", type=int, default=128)
        q.add_argument("--temperature", type=float, default=0.0, help="0: greedy")
        q.add_argument("--seed", type=int, default=0, help="sampler seed")
        q.add_argument("--dtype", default=None, choices=["bfloat16", "float32"], help="compute dtype (default: the model folder's own)")
        q.add_argument("--max-decode-slots", type=int, default=4)
        q.add_argument("--kv-block-size", type=int, default=16)
        q.add_argument("--max-num-blocks", type=int, default=None)
        q.add_argument("--max-num-batched-tokens", type=int, default=2048)
        q.add_argument("--max-model-len", type=int, default=None, help="sequences no longer than this (default: the model's limit)")
        q.add_argument("--verbose", action="store_true", help="report the backend, the folder's tensors and the engine's sizes at start-up")
    sub.add_parser("replay", add_help=False, help="feed given token ids step by step and write logits (the options of bin/trace_run)")
    i = sub.add_parser("init", help="write a model folder with random weights from a configuration and a seed")
    i.add_argument("--config", required=True, help="a config.json")
    i.add_argument("--seed", type=int, default=0)
    i.add_argument("--out", required=True)
    i.add_argument("--store-dtype", default="bfloat16", choices=["bfloat16", "float32"])
    return p


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "replay":              # the trace replay program's own options (bin/trace_run is the same program)
        from .engine import trace
        return trace.main(argv[1:])
    args = _parser().parse_args(argv)
    if args.command == "init":
        from .engine.loading import parse_dtype
        from .registry import config_class
        from .weights.random_init import write_model_folder
        d = json.loads(Path(args.config).read_text())
        cfg = config_class(d["architectures"][0]).from_dict(d)
        folder = write_model_folder(cfg, args.seed, args.out, parse_dtype(args.store_dtype))
        print(folder)
        return 0
    if not args.model:
        print("--model is required", file=sys.stderr)
        return 2
    if args.verbose:
        import logging

        from .logger import get_logger
        get_logger(level=logging.INFO)
    prompts = list(args.prompt) + [[int(t) for t in s.split(",") if t.strip()] for s in args.prompt_ids]
    if not prompts:
        print("give at least one --prompt or --prompt-ids", file=sys.stderr)
        return 2
    llm = LLM(args.model, max_decode_slots=args.max_decode_slots, kv_block_size=args.kv_block_size,
              max_num_blocks=args.max_num_blocks, dtype=args.dtype,
              max_num_batched_tokens=args.max_num_batched_tokens, max_model_len=args.max_model_len, seed=args.seed)
    outputs = llm.generate(prompts, max_new_tokens=args.max_new_tokens, temperature=args.temperature, seed=0)
    for prompt, out in zip(prompts, outputs):
        print(json.dumps({"prompt": prompt, "output": out}))
    return 0


if __name__ == "__main__":
    sys.exit(main())

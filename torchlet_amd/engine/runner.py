"""The step function: a batch of ``(request, its next tokens)`` in, logits out.

It runs only the tokens it is given, as one batch, on top of what earlier steps left in
the cache, and returns the logits at the wanted places.  Pages are reserved before the
model runs and the new lengths are committed after it; a step that cannot get its pages
raises :class:`~torchlet_amd.cache.manager.OutOfPages` and leaves the cache as it was.
"""
from __future__ import annotations

import numpy as np
import torch

from ..cache.manager import CacheManager, OutOfPages
from .batch import StaticDecodeContext, StepContext, StepEntry


def _next_pow2(n: int) -> int:
    return 1 << max(0, (n - 1).bit_length())


class _DecodeGraph:
    """The forward pass over a :class:`StaticDecodeContext`, captured as a HIP graph."""

    def __init__(self, ctx: StaticDecodeContext):
        self.ctx = ctx
        self.graph: torch.cuda.CUDAGraph | None = None
        self.logits: torch.Tensor | None = None


class ModelRunner:
    """``use_graphs``: decode-only steps (one new token for every request) run from static
    buffers under a captured HIP graph, one graph per (batch width, context length) bucket,
    as the reference replays its decode step as a CUDA graph
    (/root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:137-185).  :meth:`warm_up` captures
    the graphs an engine can reach before it serves; a bucket that was not captured ahead runs its first
    step eagerly from the static buffers and is captured then.  Capture records without
    running, so results are only ever read after an eager run or a replay (the reference
    reads its output buffer right after capture, engine.py:165-176)."""

    def __init__(self, model, cache: CacheManager, use_graphs: bool = False, max_graph_width: int = 256,
                 max_model_len: int | None = None):
        self.model = model
        self.cache = cache
        self.device = model.device
        self.caches = [cache.layer_cache(i) for i in range(len(model.spec.order))]
        self.tile_sizes = model.tile_token_sizes()
        self.max_positions = model.spec.max_positions if max_model_len is None else min(max_model_len, model.spec.max_positions)
        self.vocab_size = model.spec.vocab_size
        self.use_graphs = use_graphs and torch.device(self.device).type == "cuda" and model.graph_safe()
        self.max_graph_width = max_graph_width
        self._graphs: dict[tuple[int, int], _DecodeGraph] = {}
        self._graph_pool = None
        self.graph_replays = 0

    def step(self, entries: list[StepEntry], device_tokens: tuple | None = None) -> torch.Tensor | None:
        """Logits ``[number of wanted places, vocab]`` (float32, on the GPU), in the order
        of the entries and of their ``want`` lists; ``None`` if nothing is wanted.

        ``device_tokens = (tokens, places)``: every entry brings one token, and entry ``i`` takes it
        from ``tokens[places[i]]`` (an int32 tensor on the GPU, ``places`` a list or ``None`` for
        ``0, 1, 2, ...``) instead of from its own list, whose one element only stands in.  The step
        is then enqueued without the host knowing the tokens: a step can follow the sampling of the
        one before it while the host still waits for those tokens."""
        if not entries:
            return None
        cache = self.cache
        added = []
        try:
            return self._step(entries, added, device_tokens)
        except Exception:
            for req_id in added:            # a failed step leaves no trace of requests it introduced
                if cache.has(req_id) and cache.length(req_id) == 0:
                    cache.release(req_id)
            raise

    def _step(self, entries: list[StepEntry], added: list, device_tokens: tuple | None = None) -> torch.Tensor | None:
        cache = self.cache
        taken = None
        if device_tokens is not None:
            source, places = device_tokens
            if any(len(e.tokens) != 1 for e in entries):
                raise ValueError("tokens taken from the GPU: every request brings exactly one")
            if places is None or list(places) == list(range(len(entries))):
                taken = source[: len(entries)]
            else:
                taken = source[torch.as_tensor(list(places), dtype=torch.int64).to(source.device)]
            if taken.numel() != len(entries):
                raise ValueError(f"{len(entries)} requests, but {taken.numel()} tokens on the GPU")
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if not e.tokens:
                raise ValueError(f"request {e.req_id!r} brings no tokens")
            bad = [t for t in e.tokens if not 0 <= t < self.vocab_size]
            if bad:
                raise ValueError(f"request {e.req_id!r}: token id {bad[0]} outside the vocabulary of {self.vocab_size}")
            if any(not 0 <= w < len(e.tokens) for w in e.want):
                raise ValueError(f"request {e.req_id!r}: wanted place outside its {len(e.tokens)} tokens")
            if not cache.has(e.req_id):
                cache.add_request(e.req_id)
                added.append(e.req_id)
            if cache.length(e.req_id) + len(e.tokens) > self.max_positions:
                raise ValueError(f"request {e.req_id!r} would pass max_position_embeddings or the engine's max_model_len ({self.max_positions})")
        ctx_lens = [cache.length(e.req_id) for e in entries]
        new_lens = [len(e.tokens) for e in entries]
        # all-or-nothing over the whole step: check first, then take
        need = [0] * len(cache.groups)
        for e, c, n in zip(entries, ctx_lens, new_lens):
            for g, m in enumerate(cache.pages_missing(e.req_id, c + n)):
                need[g] += m
        free = cache.free_pages()
        if any(n > f for n, f in zip(need, free)):
            raise OutOfPages(f"step needs {need} pages per group, {free} are free")
        for e, c, n in zip(entries, ctx_lens, new_lens):
            if not cache.reserve(e.req_id, c + n):      # cannot happen after the check above
                raise OutOfPages(f"request {e.req_id!r}: reservation failed")

        req_ids = [e.req_id for e in entries]
        blocks = -(-max(c + n for c, n in zip(ctx_lens, new_lens)) // cache.page_size)
        if (self.use_graphs and max(new_lens) == 1 and len(entries) <= self.max_graph_width
                and all(e.want == [0] for e in entries)):
            logits = self._graph_step(entries, req_ids, ctx_lens, blocks, taken)
            for e, c in zip(entries, ctx_lens):
                cache.commit(e.req_id, c + 1)
            return logits
        token_ids, want_rows, base = [], [], 0
        for e in entries:
            token_ids.extend(e.tokens)
            want_rows.extend(base + w for w in e.want)
            base += len(e.tokens)
        ctx = StepContext(
            new_lens=new_lens, ctx_lens=ctx_lens, slots=[cache.slot(r) for r in req_ids],
            token_ids=token_ids, want_rows=want_rows,
            block_tables=[cache.block_table(g, req_ids, blocks) for g in range(len(cache.groups))],
            tile_sizes=self.tile_sizes, device=self.device)
        if taken is not None:
            ctx.token_ids.copy_(taken)
        logits = self.model.forward(ctx, self.caches)
        for e, c, n in zip(entries, ctx_lens, new_lens):
            cache.commit(e.req_id, c + n)
        return logits

    def _bucket(self, blocks: int) -> int:
        """The context bucket (block-table width) of a graph step whose longest sequence has ``blocks`` pages."""
        most = -(-self.max_positions // self.cache.page_size)
        return min(most, max(_next_pow2(blocks), min(most, 256 // self.cache.page_size or 1)))

    def _decode_graph(self, key: tuple[int, int]) -> _DecodeGraph:
        dg = self._graphs.get(key)
        if dg is None:
            cache = self.cache
            dg = self._graphs[key] = _DecodeGraph(StaticDecodeContext(
                width=key[0], blocks=key[1], num_groups=len(cache.groups), tile_sizes=self.tile_sizes,
                page_size=cache.page_size, device=self.device, pad_slot=cache.pad_slot))
        return dg

    def _capture(self, dg: _DecodeGraph) -> None:
        """Record the forward pass over ``dg.ctx`` (recording runs nothing).  All graphs share one pool of
        memory: they replay one after the other on one stream, and what reads a graph's logits is enqueued
        before the next replay."""
        torch.cuda.synchronize()
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            dg.logits = self.model.forward(dg.ctx, self.caches)
        dg.graph = graph

    def warm_up(self, widths=None, max_len: int | None = None) -> int:
        """Capture, ahead of need, the graphs that decode steps can ask for, so that no serving step stops to
        capture one (the reference captures its one shape inside its first decode step,
        /root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:137-176): for every batch width (``widths``:
        numbers of requests, each rounded up to the width its steps run at; default: every width up to the cache's
        slots) every context bucket of sequences of up to ``max_len`` tokens (default: the engine's limit).  Each
        shape runs once eagerly on padding rows alone, which write to no page and to no request's state, and is
        then recorded.  Returns the number of graphs captured; nothing happens without ``use_graphs``."""
        if not self.use_graphs:
            return 0
        cache = self.cache
        if widths is None:
            top = min(_next_pow2(cache.max_requests), _next_pow2(self.max_graph_width))
            widths = [1 << i for i in range(top.bit_length())]
        widths = sorted({_next_pow2(int(w)) for w in widths if 0 < int(w) <= self.max_graph_width})
        max_len = self.max_positions if max_len is None else min(max_len, self.max_positions)
        most_blocks = _next_pow2(-(-max_len // cache.page_size))
        buckets = sorted({self._bucket(1 << i) for i in range(most_blocks.bit_length())})   # of 1, 2, 4, ... pages
        captured = 0
        for width in widths:
            for bucket in buckets:
                dg = self._decode_graph((width, bucket))
                if dg.graph is None:
                    dg.ctx.fill(token_ids=[], ctx_lens=[], slots=[],
                                block_tables=[np.zeros((0, bucket), dtype=np.int32) for _ in cache.groups])
                    self.model.forward(dg.ctx, self.caches)       # eager once: kernels loaded, buffers of this shape known
                    self._capture(dg)
                    captured += 1
        torch.cuda.synchronize()
        return captured

    def _graph_step(self, entries, req_ids, ctx_lens, blocks, taken=None) -> torch.Tensor:
        cache = self.cache
        width = _next_pow2(len(entries))
        bucket = self._bucket(blocks)
        dg = self._decode_graph((width, bucket))
        dg.ctx.fill(token_ids=[e.tokens[0] for e in entries], ctx_lens=ctx_lens,
                    slots=[cache.slot(r) for r in req_ids],
                    block_tables=[cache.block_table(g, req_ids, bucket) for g in range(len(cache.groups))])
        if taken is not None:
            dg.ctx.token_ids[: len(entries)].copy_(taken)             # after the copy of the step's other numbers
        if dg.graph is None:                                          # a shape that was not captured ahead
            logits = self.model.forward(dg.ctx, self.caches)          # eager: this step's result
            result = logits[: len(entries)].clone()
            self._capture(dg)
            return result
        dg.graph.replay()
        self.graph_replays += 1
        return dg.logits[: len(entries)]

    def release(self, req_id) -> None:
        if self.cache.has(req_id):
            self.cache.release(req_id)

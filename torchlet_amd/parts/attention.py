"""Grouped-query attention over a paged key/value cache.

Formulas (/root/reference/src/torchlet/v10_triton_paged_gqa/layer/gqa.py:112-146 and
kernel/gqa.py:58-111): ``q = h Wq^T + bq`` and likewise k, v; heads are split head-major
(feature ``= head * head_dim + d``); q and k are position-encoded; the encoded k and the
raw v of every new token are stored in the cache; query head ``i`` reads KV head
``i // (heads / kv_heads)``; scores are scaled by ``head_dim ** -0.5`` (or the specification's ``scale``), masked causally
(and to the last ``window`` keys if the layer has a window), soft-maxed in 32-bit, and
the weighted values go through ``o_proj`` (no bias).

The three projections are stacked into one ``[(heads + 2 kv_heads) * head_dim, hidden]``
matrix at load time, so one matrix product reads ``h`` once.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import KEEP_COMPUTE, KEEP_STORED, MIXERS, POSITION_ENCODINGS, LazyNorm, Mixer, PagedNeed, WeightSpec

# The plans below deal work-groups to the GPU's compute units; their number comes from the device
# (``ops.compute_units()``), the thresholds in keys and tokens were measured on an MI355X (256 units).
_MIN_KEYS_PER_SPLIT = 256
_MIN_KEYS_PER_SPLIT_32BIT = 64
_PORTION_MIN_TOKENS = 16     # requests that bring at least this many tokens go to a prompt-portion kernel: the
                             # 128-row one where it is built (head size 64 or 128, pages of 8, 16, 32, ...
                             # tokens; measured on MI355X at 28/4 heads of 128: 2048 new tokens 222 -> 110 us,
                             # 8192 new tokens 2.9 -> 0.84 ms), else the 64-row one ...
_PORTION_MIN_CONTEXT = 4096  # ... which pays only in steps whose longest sequence has at least this many tokens
# The 128-row kernel: two work-groups fit a compute unit; the keys of a step's tiles are dealt out to make two rounds
# of them (measured: 14B serving 16.2k -> 16.5k tokens/s against one round), but only in steps whose tiles alone
# cannot give every compute unit one (a whole prompt of 2048 tokens has 456: split in two it took 85 + 19 us of
# merge against 90 us)
_PROMPT_MIN_KEYS_PER_SPLIT = 512
_PROMPT_MAX_SPLITS = 4


def _prompt_splits(groups: int, keys: int, uniform: bool, units: int = ops.MEASURED_COMPUTE_UNITS) -> int:
    """Into how many parts the 128-row kernel deals the keys of every tile: ``groups`` work-groups without a split,
    ``keys`` the longest sequence; ``uniform``: every tile sees about as many keys (portions deep into their
    prompts), so the work-groups come in rounds of equal length; ``units``: the GPU's compute units."""
    most = max(1, min(_PROMPT_MAX_SPLITS, keys // _PROMPT_MIN_KEYS_PER_SPLIT))
    round_ = 2 * units                  # work-groups of the 128-row kernel that run at once
    if groups <= units:
        return max(1, min(most, 2 * round_ // max(groups, 1)))
    if not uniform or groups <= round_:
        return 1
    # rounds of work-groups (two to a compute unit; 512 on the MI355X), the last one as long as the others however few are in it:
    # 640 tiles of a 2048-token step of 40 heads take two rounds whole and five quarter rounds in four parts
    # (measured at 32B sizes, 2048 tokens after 0 to 14336 cached ones: 545 -> 442 us a layer, and 24 us of merge)
    cost = lambda n: -(-groups * n // round_) / n * (1.0 if n == 1 else 1.08)
    return min(range(1, most + 1), key=cost)


@MIXERS.register("gqa_attention")
class GQAttention(Mixer):
    graph_safe = True       # nothing in forward() depends on host-side values of the step; a subclass whose stage or
                            # `transform_qk` hook reads values of the step on the host must set it back to False

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.num_heads % spec.num_kv_heads:
            raise ConfigError(f"attention: {spec.num_heads} heads are not a multiple of {spec.num_kv_heads} KV heads")
        if spec.head_dim % 2 or not 2 <= spec.head_dim <= 256:
            raise ConfigError(f"attention kernels are built for even head sizes from 2 to 256, not {spec.head_dim}")
        if spec.window is not None and spec.window < 1:
            raise ConfigError(f"attention: a window must hold at least one key, got {spec.window}")
        self.hidden = spec.hidden
        self.heads = spec.num_heads
        self.kv_heads = spec.num_kv_heads
        self.head_dim = spec.head_dim
        self.window = spec.window
        self.scale = float(spec.head_dim) ** -0.5 if spec.scale is None else float(spec.scale)
        self.q_width = self.heads * self.head_dim
        self.kv_width = self.kv_heads * self.head_dim
        self.qkv_bias = spec.qkv_bias
        self.position = POSITION_ENCODINGS.build(spec.position, dtype, device) if spec.position is not None else None
        self.compute_units = ops.compute_units()       # of the GPU it runs on: how far the keys of a request are dealt out
        self.tile_tokens = ops.attention_tile_tokens(self.heads, self.kv_heads)
        self.portion_tile_tokens = ops.prefill_attention_tile_tokens(self.heads, self.kv_heads)
        self.prompt_tile_tokens = ops.prompt_attention_tile_tokens(self.heads, self.kv_heads)
        self.pair_layout = False      # set when the weights are loaded
        self.w_qkv: torch.Tensor | None = None
        self.b_qkv: torch.Tensor | None = None
        self.w_o: torch.Tensor | None = None

    # -- declarations -------------------------------------------------------------
    def paged_need(self):
        return PagedNeed(num_heads=self.kv_heads, head_dim=self.head_dim, window=self.window, planes=2)

    def kernel_libraries(self):
        return [ops.attention_library(self.head_dim)]

    def parts(self):
        yield self
        if self.position is not None:
            yield from self.position.parts()

    def weight_specs(self):
        specs = {
            "q_proj.weight": WeightSpec((self.q_width, self.hidden)),
            "k_proj.weight": WeightSpec((self.kv_width, self.hidden)),
            "v_proj.weight": WeightSpec((self.kv_width, self.hidden)),
            "o_proj.weight": WeightSpec((self.hidden, self.q_width)),
        }
        if self.qkv_bias:
            specs["q_proj.bias"] = WeightSpec((self.q_width,), keep=KEEP_STORED)
            specs["k_proj.bias"] = WeightSpec((self.kv_width,), keep=KEEP_STORED)
            specs["v_proj.bias"] = WeightSpec((self.kv_width,), keep=KEEP_STORED)
        return specs

    def load_weights(self, tensors):
        # The bfloat16 engine keeps the rows of the query and key projections in the pair layout, in
        # which the rotary encoding turns neighbouring dimensions: the projection of a decode step
        # then rotates in its own epilogue.  Keys lie in the cache in that order too; scores are
        # sums over a head's dimensions and do not notice.
        # (not with a `transform_qk` hook: it sees the heads' dimensions in the checkpoint's order)
        self.pair_layout = (self.dtype == torch.bfloat16 and self.position is not None
                            and self.position.fused_inv_freq() is not None and self.transform_qk is None)
        rows = {"q": ops.pair_layout_rows(self.heads, self.head_dim), "k": ops.pair_layout_rows(self.kv_heads, self.head_dim)}
        order = lambda n, t: t[rows[n]] if self.pair_layout and n in rows else t
        self.w_qkv = self._place(torch.cat([order(n, tensors[f"{n}_proj.weight"]) for n in "qkv"], dim=0), KEEP_COMPUTE)
        if self.qkv_bias:
            biases = [order(n, tensors[f"{n}_proj.bias"]) for n in "qkv"]
            if len({b.dtype for b in biases}) > 1:
                biases = [b.to(torch.float32) for b in biases]
            self.b_qkv = self._place(torch.cat(biases), KEEP_STORED)
        self.w_o = self._place(tensors["o_proj.weight"], KEEP_COMPUTE)

    # -- the step -----------------------------------------------------------------
    def _splits(self, ctx, tiles: int, longest: int | None = None) -> tuple[int, int]:
        """(parts of every request's keys, waves of a work-group) for the 16-row kernel: work-groups of eight waves
        while one per tile and head group leaves compute units idle, with as many parts as give each unit one
        work-group; from there on work-groups of four waves, two to a unit, and no parts beyond that."""
        group = self.heads // self.kv_heads
        chunks = -(-group // ops.ATTENTION_ROWS)
        base = max(1, tiles * self.kv_heads * chunks)
        units = self.compute_units
        waves = 8 if base <= units and self.dtype == torch.bfloat16 else 4      # (the 32-bit kernel has work-groups of four)
        by_fill = -(-(units if waves == 8 else 2 * units) // base)      # four waves: enough work-groups to fill the units twice
        longest = ctx.max_total_len if longest is None else longest
        longest = longest if self.window is None else min(longest, self.window + ctx.max_new_tokens)
        # (the 32-bit engine's kernel walks its keys 32 at a time through shared memory, one work-group of four waves
        # on a part: parts of 64 keys keep the compute units busy where 256 left most of them idle)
        by_keys = max(1, longest // (_MIN_KEYS_PER_SPLIT if self.dtype == torch.bfloat16 else _MIN_KEYS_PER_SPLIT_32BIT))
        return max(1, min(by_fill, by_keys, 64)), waves

    takes_lazy_norm = True

    # The step has three stages, each a method of its own, so that a mixer that differs from this one in one
    # stage overrides that stage and keeps the others: projection of q, k, v with position encoding and cache
    # write (`project`), attention of the queries over the cache (`attend`), output projection (`output`).
    # A mixer that only needs to do something to the projected queries and keys before they are encoded and
    # stored (a norm per head, say) defines `transform_qk`; the kernels that fuse projection, rotation and
    # cache write are then left out, since they would rotate what has not been transformed yet.
    transform_qk = None      # or: def transform_qk(self, q3, k3, ctx) -> None, in place on [T, heads, head_dim] views (k3 may be None)

    def forward(self, h, ctx, cache):
        qkv = self.project(h, ctx, cache)
        out = self.attend(qkv[:, : self.q_width], ctx, cache)
        return self.output(out)

    def _cache_views(self, ctx, cache):
        # the cache hands out two planes of [pages, kv_heads, page, head_dim]; this mixer keeps the
        # values of a page transposed, [kv_heads, head_dim, page], as its kernels read them
        k_plane, v_plane = cache.planes
        v_plane = v_plane.view(v_plane.shape[0], self.kv_heads, self.head_dim, cache.page_size)
        return k_plane, v_plane, ctx.block_tables[cache.group]

    def project(self, h, ctx, cache):
        """``[T, q_width (+ 2 kv_width)]``: position-encoded queries in the first ``q_width`` columns; the encoded
        keys and the values of the step's tokens are in their pages when this returns (if the run owns its cache)."""
        lazy = h if isinstance(h, LazyNorm) else None      # one row whose norm the projection's kernel can make itself
        device = lazy.residual.device if lazy is not None else h.device
        T = 1 if lazy is not None else h.shape[0]
        writes = cache.writable
        width = self.q_width + (2 * self.kv_width if writes else 0)
        w = self.w_qkv if writes else self.w_qkv[: self.q_width]
        b = self.b_qkv if (self.b_qkv is None or writes) else self.b_qkv[: self.q_width]
        qkv = torch.empty((T, width), dtype=self.dtype, device=device)
        k_plane, v_plane, table = self._cache_views(ctx, cache)
        kv_heads = self.kv_heads if writes else 0
        inv_freq = self.position.fused_inv_freq() if self.position is not None else None
        cache_args = (ctx.token_req, table, k_plane, v_plane, cache.page_size) if writes else (None, None, None, None, 0)
        plain = self.transform_qk is not None               # nothing fused: the hook sits between projection and rotation
        fused = False
        if lazy is not None:
            rms = lazy.rmsnorm()          # the fused kernel makes a root-mean-square norm and no other
            if self.pair_layout and not plain and rms is not None:
                residual_out = torch.empty_like(lazy.residual)
                fused = ops.linear_rope_cache_write_normed(lazy.residual, lazy.pending, rms[0], rms[1],
                                                           residual_out, w, b, qkv, self.heads, self.kv_heads, self.head_dim,
                                                           ctx.positions, inv_freq, *cache_args)
                if fused:
                    lazy.done(residual_out)
            if not fused:
                h = lazy.value()
        fused = fused or (self.pair_layout and not plain and
                          ops.linear_rope_cache_write(h, w, b, qkv, self.heads, self.kv_heads, self.head_dim,
                                                      ctx.positions, inv_freq, *cache_args))
        if not fused and not plain and self.dtype == torch.bfloat16 and (inv_freq is not None or self.position is None) \
                and ops.linear_partials_pay(T, width, self.hidden):
            # few rows against a narrow matrix: K split over work-groups; the rotation kernel adds the slabs up
            ops.rope_cache_write(qkv, self.heads, kv_heads, self.head_dim, self.heads + kv_heads, ctx.positions, inv_freq,
                                 *cache_args, pairs=self.pair_layout, parts=ops.linear_partials(h, w), bias=b)
        elif not fused:
            ops.linear(h, w, b, qkv)
            q3 = qkv[:, : self.q_width].unflatten(1, (self.heads, self.head_dim))
            k3 = qkv[:, self.q_width: self.q_width + self.kv_width].unflatten(1, (self.kv_heads, self.head_dim)) if writes else None
            if plain:
                self.transform_qk(q3, k3, ctx)
            if self.position is not None and inv_freq is None:
                self.position.apply(q3, k3, ctx.positions)
            if inv_freq is not None or writes:
                ops.rope_cache_write(qkv, self.heads, kv_heads, self.head_dim, self.heads + kv_heads, ctx.positions, inv_freq,
                                     *cache_args, pairs=self.pair_layout)
        return qkv

    def attend(self, q, ctx, cache):
        """Causal (and windowed) attention of the step's queries ``q [T, q_width]`` (a row-strided view) over their
        requests' cached keys and values: ``[T, q_width]``."""
        T = q.shape[0]
        k_plane, v_plane, table = self._cache_views(ctx, cache)
        out = torch.empty((T, self.q_width), dtype=self.dtype, device=q.device)
        common = (self.heads, self.kv_heads, self.head_dim, cache.page_size, self.window or 0, self.scale)
        rows128 = (ops.prompt_attention_fits(self.dtype, self.head_dim, cache.page_size, -(-ctx.max_total_len // cache.page_size), self.scale)
                   and ctx.max_new_tokens >= _PORTION_MIN_TOKENS)
        portions = (self.dtype == torch.bfloat16 and self.head_dim <= ops.PREFILL_ATTENTION_MAX_HEAD_DIM
                    and self.head_dim % 16 == 0 and cache.page_size % 4 == 0 and ctx.max_new_tokens >= _PORTION_MIN_TOKENS
                    and ctx.max_total_len >= _PORTION_MIN_CONTEXT)
        if rows128 or portions:
            # prompt portions: tiles of 128 (or 64) rows with keys and values through shared memory; the
            # other requests of the step (decode tokens, short portions): 16-row tiles, keys split over waves
            tq = self.prompt_tile_tokens if rows128 else self.portion_tile_tokens
            kernel = ops.paged_attention_prompt if rows128 else ops.paged_attention_prefill
            short, long = ctx.tiles_by_length(self.tile_tokens, tq, _PORTION_MIN_TOKENS)
            extra = {}
            if rows128:
                # few tiles against long sequences (a portion of a few hundred tokens deep into a prompt):
                # each tile's keys are dealt to several work-groups, so that the compute units have work
                groups = long[2] * self.kv_heads * -(-(self.heads // self.kv_heads) // ops.PROMPT_ATTENTION_ROWS)
                keys = ctx.max_total_len if self.window is None else min(ctx.max_total_len, self.window + tq)
                splits = _prompt_splits(groups, keys, uniform=long[5] >= 2 * ctx.max_new_tokens, units=self.compute_units)
                extra = dict(max_total_len=ctx.max_total_len, splits=splits, merge_tokens=(long[3], long[4]))
            kernel(q, out, k_plane, v_plane, table, ctx.req_indptr, ctx.ctx_lens, long[0], long[1], long[2], tq, *common, **extra)
            if short[2]:     # split over their keys; the merge of the parts is kept to the rows of these requests
                splits, waves = self._splits(ctx, short[2], short[5])
                ops.paged_attention(q, out, k_plane, v_plane, table, ctx.req_indptr, ctx.ctx_lens,
                                    short[0], short[1], short[2], self.tile_tokens, *common,
                                    splits, merge_tokens=(short[3], short[4]), waves=waves)
        else:
            tile_req, tile_tok0, tiles = ctx.tiles(self.tile_tokens)
            if ctx.decode_only and tiles == T:      # one token per request: no tile list to look up
                tile_req = tile_tok0 = None
            splits, waves = self._splits(ctx, tiles)
            ops.paged_attention(q, out, k_plane, v_plane, table, ctx.req_indptr, ctx.ctx_lens,
                                tile_req, tile_tok0, tiles, self.tile_tokens, *common, splits, waves=waves)
        return out

    def output(self, out):
        """The output projection (no bias) of the mixed heads ``[T, q_width]``: ``[T, hidden]``, or float32 slabs of
        partial sums ``[P, T, hidden]`` that the next norm adds up."""
        T = out.shape[0]
        if self.dtype == torch.bfloat16 and ops.linear_partials_pay(T, self.hidden, self.q_width):
            # few rows against a narrow matrix: K split over work-groups; the next norm adds the slabs up
            return ops.linear_partials(out, self.w_o)
        y = torch.empty((T, self.hidden), dtype=self.dtype, device=out.device)
        ops.linear(out, self.w_o, None, y)
        return y

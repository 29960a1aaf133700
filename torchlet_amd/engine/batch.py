"""One step's batch: what the host hands to the model, and how it reaches the GPU.

A step is a list of ``(request, its next tokens, wanted places)``.  Each request adds
``n >= 1`` tokens at the positions ``length .. length + n - 1`` after what it already
holds in the cache; ``n == 1`` is a decoded token, ``n > 1`` a portion of a prompt, and
both kinds share one batch (the reference's two kinds of batches,
/root/reference/src/torchlet/v10_triton_paged_gqa/scheduler.py:182-253, are one here).

All integer metadata of a step is packed into one int32 buffer and copied to the GPU
once; the fields of :class:`StepContext` are views into that copy.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


@dataclass
class StepEntry:
    req_id: object
    tokens: list[int]
    want: list[int] = field(default_factory=list)   # places among `tokens` whose logits are wanted


class StepContext:
    """Device-side description of a step, shared by every layer.

    ``token_ids, positions, token_req`` are ``[T]``; ``req_indptr`` ``[R+1]``; ``ctx_lens``
    (tokens cached before the step) and ``slots`` ``[R]``; ``want_rows`` flat token indices;
    ``block_tables[g]`` ``[R, blocks]`` for cache group ``g``.  All int32.
    """

    def __init__(self, *, new_lens, ctx_lens, slots, token_ids, want_rows, block_tables, tile_sizes, device):
        R = len(new_lens)
        new_lens = np.asarray(new_lens, dtype=np.int32)
        ctx_np = np.asarray(ctx_lens, dtype=np.int32)
        indptr = np.zeros(R + 1, dtype=np.int32)
        np.cumsum(new_lens, out=indptr[1:])
        T = int(indptr[-1])
        token_req = np.repeat(np.arange(R, dtype=np.int32), new_lens)
        positions = (np.arange(T, dtype=np.int32) - indptr[:-1][token_req] + ctx_np[token_req]).astype(np.int32)
        self.num_tokens = T
        self.num_requests = R
        self.num_wanted = len(want_rows)
        self.max_total_len = int((ctx_np + new_lens).max()) if R else 0
        self.max_new_tokens = int(new_lens.max()) if R else 0
        self.decode_only = bool(R and self.max_new_tokens == 1)
        self.device = device
        self._host_new_lens = new_lens
        self._host_ctx_lens = ctx_np
        self._tiles: dict[int, tuple] = {}

        fields = {
            "token_ids": np.asarray(token_ids, dtype=np.int32),
            "positions": positions,
            "token_req": token_req,
            "req_indptr": indptr,
            "ctx_lens": ctx_np,
            "slots": np.asarray(slots, dtype=np.int32),
            "want_rows": np.asarray(want_rows, dtype=np.int32),
        }
        for g, bt in enumerate(block_tables):
            fields[f"bt{g}"] = np.ascontiguousarray(bt, dtype=np.int32).reshape(-1)
        host_tiles = {}
        for tq in sorted(tile_sizes):
            tr, t0 = self._build_tiles(tq)
            host_tiles[tq] = len(tr)
            fields[f"tile_req{tq}"] = tr
            fields[f"tile_tok0{tq}"] = t0
        views = self._upload(fields)
        self.token_ids = views["token_ids"]
        self.positions = views["positions"]
        self.token_req = views["token_req"]
        self.req_indptr = views["req_indptr"]
        self.ctx_lens = views["ctx_lens"]
        self.slots = views["slots"]
        self.want_rows = views["want_rows"] if self.num_wanted else None
        self.block_tables = [views[f"bt{g}"].view(R, -1) for g in range(len(block_tables))]
        for tq, n in host_tiles.items():
            self._tiles[tq] = (views[f"tile_req{tq}"], views[f"tile_tok0{tq}"], n)

    def _build_tiles(self, tq: int, select=None):
        """Tiles of up to ``tq`` consecutive new tokens of one request (of the requests where
        ``select`` is true, if given)."""
        counts = -(-self._host_new_lens // tq)
        if select is not None:
            counts = np.where(select, counts, 0)
        tile_req = np.repeat(np.arange(self.num_requests, dtype=np.int32), counts)
        first = np.zeros(self.num_requests + 1, dtype=np.int64)
        np.cumsum(counts, out=first[1:])
        tile_tok0 = ((np.arange(int(first[-1])) - first[:-1][tile_req]) * tq).astype(np.int32)
        return tile_req, tile_tok0

    def _upload(self, fields: dict[str, np.ndarray]) -> dict[str, torch.Tensor]:
        # every field starts at a multiple of 4 ints (16 bytes)
        offsets, total = {}, 0
        for k, a in fields.items():
            offsets[k] = total
            total += -(-max(a.size, 1) // 4) * 4
        buf = np.zeros(total, dtype=np.int32)
        for k, a in fields.items():
            buf[offsets[k]: offsets[k] + a.size] = a
        dev = torch.from_numpy(buf).to(self.device)
        return {k: dev[offsets[k]: offsets[k] + a.size] for k, a in fields.items()}

    def tiles(self, tq: int):
        """``(tile_req, tile_tok0, number of tiles)`` for tiles of ``tq`` tokens."""
        t = self._tiles.get(tq)
        if t is None:
            tr, t0 = self._build_tiles(tq)
            v = self._upload({"r": tr, "t": t0})
            t = self._tiles[tq] = (v["r"], v["t"], len(tr))
        return t

    def tiles_by_length(self, tq_short: int, tq_long: int, threshold: int):
        """Two tile lists: requests that bring fewer than ``threshold`` tokens in tiles of
        ``tq_short`` tokens, the others in tiles of ``tq_long``.  The first list comes with the
        indices of its requests' tokens and the largest sequence length among them, the second
        with its requests' tokens and the smallest sequence length among them:
        ``((tile_req, tile_tok0, tiles, tokens, number of tokens, longest),
        (tile_req, tile_tok0, tiles, tokens, number of tokens, shortest))``."""
        key = (tq_short, tq_long, threshold)
        t = self._tiles.get(key)
        if t is None:
            long = self._host_new_lens >= threshold
            sr, s0 = self._build_tiles(tq_short, ~long)
            lr, l0 = self._build_tiles(tq_long, long)
            starts = np.zeros(self.num_requests + 1, dtype=np.int64)
            np.cumsum(self._host_new_lens, out=starts[1:])
            short_tokens = np.concatenate([np.arange(starts[r], starts[r + 1]) for r in np.nonzero(~long)[0]] or
                                          [np.zeros(0, dtype=np.int64)]).astype(np.int32)
            long_tokens = np.concatenate([np.arange(starts[r], starts[r + 1]) for r in np.nonzero(long)[0]] or
                                         [np.zeros(0, dtype=np.int64)]).astype(np.int32)
            totals = self._host_new_lens + self._host_ctx_lens
            longest = int(totals[~long].max()) if (~long).any() else 0
            shortest = int(totals[long].min()) if long.any() else 0
            v = self._upload({"sr": sr, "s0": s0, "lr": lr, "l0": l0, "st": short_tokens, "lt": long_tokens})
            t = self._tiles[key] = ((v["sr"], v["s0"], len(sr), v["st"], len(short_tokens), longest),
                                    (v["lr"], v["l0"], len(lr), v["lt"], len(long_tokens), shortest))
        return t


class StaticDecodeContext:
    """A step context of fixed shape for decode-only steps: ``width`` requests with one new
    token each and block tables of ``blocks`` entries, living in one static device buffer
    that is refilled before every step (one copy from pinned host memory).  Because no
    address or launch size changes between steps, the model's forward pass over it can be
    captured once as a HIP graph and replayed.  Unused rows are padded with requests of
    length zero whose block tables point at the sentinel page (the cache-write kernels drop what
    would go to that page, so nothing writes it) and whose slot is ``pad_slot``, a state row that
    belongs to no request.
    """

    def __init__(self, *, width: int, blocks: int, num_groups: int, tile_sizes, page_size: int, device, pad_slot: int = 0):
        S = width
        self.pad_slot = pad_slot
        self.width = S
        self.blocks = blocks
        self.num_tokens = S
        self.num_requests = S
        self.num_wanted = S
        self.max_total_len = blocks * page_size       # an upper bound: fixes the attention's split count
        self.max_new_tokens = 1
        self.decode_only = True
        self.device = device
        sizes = {"token_ids": S, "positions": S, "ctx_lens": S, "slots": S, "token_req": S, "req_indptr": S + 1,
                 "want_rows": S, "tile_req": S, "tile_tok0": S}
        for g in range(num_groups):
            sizes[f"bt{g}"] = S * blocks
        self._offsets, total = {}, 0
        for k, n in sizes.items():
            self._offsets[k] = (total, n)
            total += -(-n // 4) * 4
        self._host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self._np = self._host.numpy()
        self._dev = torch.zeros(total, dtype=torch.int32, device=device)
        ar = np.arange(S + 1, dtype=np.int32)
        self._set("token_req", ar[:S])
        self._set("req_indptr", ar)
        self._set("want_rows", ar[:S])
        self._set("tile_req", ar[:S])
        v = {k: self._dev[o: o + n] for k, (o, n) in self._offsets.items()}
        self.token_ids, self.positions, self.ctx_lens, self.slots = v["token_ids"], v["positions"], v["ctx_lens"], v["slots"]
        self.token_req, self.req_indptr, self.want_rows = v["token_req"], v["req_indptr"], v["want_rows"]
        self.block_tables = [v[f"bt{g}"].view(S, blocks) for g in range(num_groups)]
        self._tile = (v["tile_req"], v["tile_tok0"], S)
        self._dev.copy_(self._host)
        self._copied = torch.cuda.Event() if torch.device(device).type == "cuda" else None

    def _set(self, key: str, values) -> None:
        o, n = self._offsets[key]
        self._np[o: o + n] = 0
        self._np[o: o + len(values)] = values

    def tiles(self, tq: int):
        return self._tile                 # one token per request: a tile per request whatever its height

    def fill(self, *, token_ids, ctx_lens, slots, block_tables) -> None:
        """New tokens, lengths and block-table rows of the live requests (``<= width``)."""
        if self._copied is not None:
            self._copied.synchronize()        # the previous copy has read the pinned buffer
        self._set("token_ids", token_ids)
        self._set("positions", ctx_lens)
        self._set("ctx_lens", ctx_lens)
        self._set("slots", list(slots) + [self.pad_slot] * (self.width - len(slots)))
        for g, bt in enumerate(block_tables):
            o, n = self._offsets[f"bt{g}"]
            dst = self._np[o: o + n].reshape(self.width, self.blocks)
            dst[:] = 0
            dst[: bt.shape[0], : bt.shape[1]] = bt
        self._dev.copy_(self._host, non_blocking=True)
        if self._copied is not None:
            self._copied.record()

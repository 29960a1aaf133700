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

    def _build_tiles(self, tq: int):
        """Tiles of up to ``tq`` consecutive new tokens of one request."""
        counts = -(-self._host_new_lens // tq)
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

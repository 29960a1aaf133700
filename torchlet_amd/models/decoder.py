"""A decoder built from a :class:`~torchlet_amd.config.base.ModelSpec`.

embedding (times ``embed_scale``) -> the runs of the layer order -> final norm on the wanted rows
(times ``logit_scale``) -> LM head (plus its bias, if the specification says it has one)
(/root/reference/src/torchlet/v10_triton_paged_gqa/model/qwen2_5.py:55-87, where the factors are 1 and
there is no bias).  The class
knows nothing of any architecture: which parts a layer has, their sizes, the names of
their tensors and the order of the runs all come from the specification.
"""
from __future__ import annotations

import torch

from ..config.base import ModelSpec
from ..kernels import ops
from ..parts import BLOCKS, NORMS, Stream, WeightSpec
from ..parts.base import KEEP_COMPUTE, KEEP_STORED, place


class DecoderModel:
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"compute dtype must be float32 or bfloat16, got {dtype}")
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.blocks = [BLOCKS.build(b, dtype, self.device) for b in spec.layers]
        self.final_norm = NORMS.build(spec.final_norm, dtype, self.device)
        self.embed: torch.Tensor | None = None
        self.head: torch.Tensor | None = None
        self.head_bias: torch.Tensor | None = None

    # ------------------------------------------------------------------ weights
    def weight_specs(self) -> dict[str, WeightSpec]:
        s = self.spec
        specs = {f"{s.embed_name}.weight": WeightSpec((s.vocab_size, s.hidden))}
        for i, block in enumerate(self.blocks):
            for k, v in block.weight_specs().items():
                specs[f"{s.layers_prefix}.{i}.{k}"] = v
        for k, v in self.final_norm.weight_specs().items():
            specs[f"{s.final_norm_name}.{k}"] = v
        # a tied head is the embedding matrix; a checkpoint may still carry a copy of it
        specs[f"{s.head_name}.weight"] = WeightSpec((s.vocab_size, s.hidden), optional=s.tie_head)
        if s.head_bias:
            specs[f"{s.head_name}.bias"] = WeightSpec((s.vocab_size,), keep=KEEP_STORED)
        return specs

    def load_weights(self, tensors: dict[str, torch.Tensor]) -> None:
        s = self.spec
        self.embed = place(tensors[f"{s.embed_name}.weight"], KEEP_COMPUTE, self.dtype, self.device)
        names = list(tensors)      # `tensors` may read from disk on access: touch each name once
        for i, block in enumerate(self.blocks):
            prefix = f"{s.layers_prefix}.{i}."
            block.load_weights({k[len(prefix):]: tensors[k] for k in names if k.startswith(prefix)})
        prefix = s.final_norm_name + "."
        self.final_norm.load_weights({k[len(prefix):]: tensors[k] for k in names if k.startswith(prefix)})
        if s.tie_head:
            self.head = self.embed
        else:
            self.head = place(tensors[f"{s.head_name}.weight"], KEEP_COMPUTE, self.dtype, self.device)
        if s.head_bias:
            self.head_bias = place(tensors[f"{s.head_name}.bias"], KEEP_STORED, self.dtype, self.device)

    # ------------------------------------------------------------------ cache needs
    def cache_plan(self):
        """Per run of the order: ``(paged need, state need, cache_of)``."""
        plan = []
        for e in self.spec.order:
            mixer = self.blocks[e.layer].mixer
            plan.append((mixer.paged_need(), mixer.state_need(), e.cache_of))
        return plan

    def tile_token_sizes(self) -> set[int]:
        return {b.mixer.tile_tokens for b in self.blocks if hasattr(b.mixer, "tile_tokens")}

    def parts(self):
        """Every part of the model: each block with what is inside it, and the final norm."""
        for b in self.blocks:
            yield from b.parts()
        yield from self.final_norm.parts()

    def graph_safe(self) -> bool:
        """Every part of every block (and the final norm) says that it runs from device-side values only,
        so a decode step can be captured once as a graph and replayed."""
        return all(getattr(p, "graph_safe", False) for p in self.parts())

    def kernel_libraries(self) -> list[str]:
        libs = ["elementwise", "gemm", "sampling"]
        for b in self.blocks:
            if hasattr(b.mixer, "kernel_libraries"):
                libs += b.mixer.kernel_libraries()
        return list(dict.fromkeys(libs))

    # ------------------------------------------------------------------ the step
    def forward(self, ctx, caches) -> torch.Tensor | None:
        """Run the tokens of ``ctx`` through every run of the order; ``caches[i]`` is the
        cache view of run ``i``.  Returns float32 logits ``[wanted rows, vocab]`` (``None``
        when no row is wanted)."""
        T = ctx.num_tokens
        residual = torch.empty((T, self.spec.hidden), dtype=torch.float32, device=self.device)
        ops.embedding(ctx.token_ids, self.embed, residual, self.spec.embed_scale)
        stream = Stream(residual)
        for i, e in enumerate(self.spec.order):
            stream = self.blocks[e.layer].forward(stream, ctx, caches[i])
        if ctx.want_rows is None or ctx.num_wanted == 0:
            return None
        h = self.final_norm.forward(stream, rows=ctx.want_rows, gain=self.spec.logit_scale)
        logits = torch.empty((ctx.num_wanted, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        ops.linear(h, self.head, self.head_bias, logits)
        return logits

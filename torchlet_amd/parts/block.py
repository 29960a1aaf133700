"""Pre-norm residual block: ``x += mixer(norm1(x)); x += ffn(norm2(x))``
(/root/reference/src/torchlet/v10_triton_paged_gqa/layer/transformer_block.py:37-40).

The additions are deferred: a branch's output is left ``pending`` on the stream and the
next norm (the block's second one, the next block's first one, or the model's final one)
adds it in 32-bit while it normalises.
"""
from __future__ import annotations

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, Stream


@BLOCKS.register("prenorm_residual")
class PreNormBlock(Block):
    graph_safe = True       # the arrangement itself; its four parts answer for themselves

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.mixer_norm = NORMS.build(spec.mixer_norm, dtype, device)
        self.mixer = MIXERS.build(spec.mixer, dtype, device)
        self.ffn_norm = NORMS.build(spec.ffn_norm, dtype, device)
        self.ffn = FEED_FORWARDS.build(spec.ffn, dtype, device)
        self._children = {
            spec.mixer_norm_name: self.mixer_norm,
            spec.mixer_name: self.mixer,
            spec.ffn_norm_name: self.ffn_norm,
            spec.ffn_name: self.ffn,
        }

    def parts(self):
        yield self
        for part in self._children.values():
            yield from part.parts()

    def weight_specs(self):
        return {f"{name}.{k}": v for name, part in self._children.items() for k, v in part.weight_specs().items()}

    def load_weights(self, tensors):
        for name, part in self._children.items():
            prefix = name + "."
            part.load_weights({k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)})

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        # a part that says it takes a norm that has not run yet (``takes_lazy_norm``) may get one, see LazyNorm
        h = (self.mixer_norm.lazy(stream) if getattr(self.mixer, "takes_lazy_norm", False) else None) or self.mixer_norm.forward(stream)
        stream.pending = self.mixer.forward(h, ctx, cache)
        h = (self.ffn_norm.lazy(stream) if getattr(self.ffn, "takes_lazy_norm", False) else None) or self.ffn_norm.forward(stream)
        stream.pending = self.ffn.forward(h, ctx)
        return stream

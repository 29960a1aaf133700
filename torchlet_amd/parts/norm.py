"""Root-mean-square norm, fused with the addition of the pending branch output.

``h = r * rsqrt(mean(r^2) + eps) * weight`` with ``r = residual + pending``; the epsilon
sits inside the root and the weight multiplies last, without a ``1 +`` offset
(/root/reference/src/torchlet/v10_triton_paged_gqa/kernel/rms_norm.py:13-19).  All of it
is computed in 32-bit; ``r`` is stored back as the new 32-bit residual.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import KEEP_STORED, NORMS, LazyNorm, Norm, Stream, WeightSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.dim = spec.dim
        self.eps = float(spec.eps)
        self.weight: torch.Tensor | None = None

    def weight_specs(self):
        return {"weight": WeightSpec((self.dim,), keep=KEEP_STORED, init="one_plus_normal")}

    def load_weights(self, tensors):
        self.weight = self._place(tensors["weight"], KEEP_STORED)

    def forward(self, stream: Stream, rows: torch.Tensor | None = None, gain: float = 1.0) -> torch.Tensor:
        n = stream.residual.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=self.dtype, device=stream.residual.device)
        ops.add_rmsnorm(stream.residual, stream.pending, self.weight, self.eps, out, rows, gain)
        if rows is None:
            stream.pending = None
        return out

    def lazy(self, stream: Stream) -> LazyNorm | None:
        # one row in bfloat16: the kernels that read the norm's output can make it while their weights arrive
        if self.dtype == torch.bfloat16 and stream.residual.shape[0] == 1 and stream.residual.is_cuda:
            return LazyNorm(self, stream, "rmsnorm", weight=self.weight, eps=self.eps)
        return None

"""Dense SwiGLU feed-forward: ``down(silu(gate(h)) * up(h))``, no biases
(/root/reference/src/torchlet/v10_triton_paged_gqa/layer/ffn_swiglu.py:22-59).

``gate_proj`` and ``up_proj`` are stacked into one ``[2I, H]`` matrix at load time so that
one matrix product reads ``h`` once; the gate is applied to the two halves of its result.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, WeightSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = spec.hidden
        self.inter = spec.intermediate
        self.gate_up: torch.Tensor | None = None
        self.down: torch.Tensor | None = None

    def weight_specs(self):
        return {
            "gate_proj.weight": WeightSpec((self.inter, self.hidden)),
            "up_proj.weight": WeightSpec((self.inter, self.hidden)),
            "down_proj.weight": WeightSpec((self.hidden, self.inter)),
        }

    def load_weights(self, tensors):
        self.gate_up = self._place(torch.cat((tensors["gate_proj.weight"], tensors["up_proj.weight"]), dim=0), "matrix")
        self.down = self._place(tensors["down_proj.weight"], "matrix")

    def forward(self, h, ctx):
        T = h.shape[0]
        gu = torch.empty((T, 2 * self.inter), dtype=self.dtype, device=h.device)
        ops.linear(h, self.gate_up, None, gu)
        z = torch.empty((T, self.inter), dtype=self.dtype, device=h.device)
        ops.swiglu(gu, z)
        y = torch.empty((T, self.hidden), dtype=self.dtype, device=h.device)
        ops.linear(z, self.down, None, y)
        return y

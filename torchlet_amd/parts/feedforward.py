"""Dense SwiGLU feed-forward: ``down(silu(gate(h)) * up(h))``, no biases
(/root/reference/src/torchlet/v10_triton_paged_gqa/layer/ffn_swiglu.py:22-59).

``gate_proj`` and ``up_proj`` are put into one matrix at load time so that one matrix
product reads ``h`` once.  In bfloat16 (hidden a multiple of 8) the two are interleaved in
blocks of 32 rows and the gate ``silu(g) * u`` is applied to the 32-bit accumulators inside
the product's kernel, as the reference's fused kernel does (kernel/ffn_swiglu.py:139-160);
otherwise they are stacked ``[gate; up]`` and a separate kernel applies the gate.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, KEEP_COMPUTE, FeedForward, LazyNorm, WeightSpec


# The down product returns partial sums over slices of K where the kernel library finds that it
# pays (the matrix is narrow, so its output tiles alone are too few to keep the GPU busy; measured
# at 3584 x 18944: 64 rows 31 us in four parts against 90 us whole, 512 rows 82 against 147 us);
# the next norm adds the slabs up.


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

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
        self.fused_gate = self.dtype == torch.bfloat16 and self.hidden % 8 == 0
        if self.fused_gate:
            gate = self._place(tensors["gate_proj.weight"], KEEP_COMPUTE)
            up = self._place(tensors["up_proj.weight"], KEEP_COMPUTE)
            self.gate_up = ops.interleave_gate_up(gate, up)
        else:
            self.gate_up = self._place(torch.cat((tensors["gate_proj.weight"], tensors["up_proj.weight"]), dim=0), KEEP_COMPUTE)
        self.down = self._place(tensors["down_proj.weight"], KEEP_COMPUTE)

    takes_lazy_norm = True

    def forward(self, h, ctx):
        lazy = h if isinstance(h, LazyNorm) else None
        if lazy is not None:
            # one row: the gate/up kernel makes the norm itself while its first weights arrive
            rms = lazy.rmsnorm()          # the fused kernel makes a root-mean-square norm and no other
            if self.fused_gate and rms is not None:
                z = torch.empty((1, self.inter), dtype=self.dtype, device=lazy.residual.device)
                residual_out = torch.empty_like(lazy.residual)
                if ops.linear_swiglu_normed(lazy.residual, lazy.pending, rms[0], rms[1], residual_out,
                                            self.gate_up, z):
                    lazy.done(residual_out)
                    return self._down(z, 1)
            h = lazy.value()
        T = h.shape[0]
        z = torch.empty((T, self.inter), dtype=self.dtype, device=h.device)
        if self.fused_gate:
            ops.linear_swiglu(h, self.gate_up, z)
        else:
            gu = torch.empty((T, 2 * self.inter), dtype=self.dtype, device=h.device)
            ops.linear(h, self.gate_up, None, gu)
            ops.swiglu(gu, z)
        return self._down(z, T)

    def _down(self, z, T):
        if self.dtype == torch.bfloat16 and ops.linear_partials_pay(T, self.hidden, self.inter):
            # few rows, long K, narrow matrix: split K over work-groups; the next norm adds the slabs up
            return ops.linear_partials(z, self.down)
        y = torch.empty((T, self.hidden), dtype=self.dtype, device=z.device)
        ops.linear(z, self.down, None, y)
        return y

"""Rotary position encoding with the split-half pairing ``(j, j + head_dim/2)``.

``inv_freq[j] = 1 / theta**(2j / head_dim)`` is computed once in 32-bit exactly as the
reference builds its table (/root/reference/src/torchlet/v10_triton_paged_gqa/layer/rope.py:29-35);
the angle of a token is ``float32(position) * inv_freq[j]`` and the rotation
``y1 = x1*cos - x2*sin, y2 = x2*cos + x1*sin`` (kernel/rope.py:28-37) is done in 32-bit
inside the kernel, so no table of ``max_positions`` rows is kept.
"""
from __future__ import annotations

import torch

from ..config.base import ConfigError
from ..kernels import ops
from .base import POSITION_ENCODINGS, PositionEncoding


@POSITION_ENCODINGS.register("rope_split_half")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        if spec.head_dim % 2:
            raise ConfigError(f"rotary encoding needs an even head size, got {spec.head_dim}")
        self.head_dim = spec.head_dim
        self.max_positions = spec.max_positions
        j = torch.arange(0, spec.head_dim, 2, dtype=torch.float32)
        self.inv_freq = (1.0 / (float(spec.theta) ** (j / spec.head_dim))).to(device)

    def fused_inv_freq(self) -> torch.Tensor:
        """The attention mixer folds this encoding into its cache-write kernel."""
        return self.inv_freq

    def apply(self, q, k, positions):
        for x in (q, k):
            if x is None:
                continue
            T, heads, hd = x.shape
            flat = x.as_strided((T, heads * hd), (x.stride(0), 1))
            ops.rope_cache_write(flat, heads, 0, hd, heads, positions, self.inv_freq)

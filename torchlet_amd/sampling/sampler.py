"""Greedy and temperature sampling.

The reference samples greedily only: ``logits.argmax(dim=-1)``
(/root/reference/src/torchlet/v10_triton_paged_gqa/engine.py:187-188).  Here a request
with ``temperature == 0`` takes the arg max of the 32-bit logits (lowest index on ties);
with ``temperature > 0`` it draws from ``softmax(logits / temperature)`` by the Gumbel-max
rule inside the sampling kernel.  The randomness of a draw is a function of the sampler's
seed, the request's seed and the index of the token being generated, and of nothing else:
the same request yields the same tokens alone, in any batch, and after being preempted.
"""
from __future__ import annotations

import torch

from ..kernels import ops

_M32 = 0xFFFFFFFF


def mix32(x: int) -> int:
    """The 32-bit mixing function the sampling kernel uses (sampling.hip ``mix32``)."""
    x &= _M32
    x ^= x >> 16
    x = (x * 0x7FEB352D) & _M32
    x ^= x >> 15
    x = (x * 0x846CA68B) & _M32
    x ^= x >> 16
    return x


def draw_key(sampler_seed: int, request_seed: int, token_index: int) -> int:
    """32-bit key of one draw, as a signed int32 value."""
    k = mix32(sampler_seed & _M32)
    k = mix32(k ^ ((sampler_seed >> 32) & _M32))
    k = mix32(k ^ (request_seed & _M32))
    k = mix32(k ^ ((request_seed >> 32) & _M32) ^ 0x632BE5AB)
    k = mix32(k ^ (token_index & _M32))
    return k - (1 << 32) if k >= (1 << 31) else k


class Sampler:
    def __init__(self, seed: int = 0):
        self.seed = int(seed)

    def launch(self, logits: torch.Tensor, temperatures: list[float], request_seeds: list[int],
               token_indices: list[int]) -> "Drawn":
        """Start the draw of one token per row of ``logits [N, vocab]`` (float32, on the GPU) and the
        copy of the tokens to the host; nothing waits.  The tokens stay on the GPU as well
        (``Drawn.device``), where the next step can take them from before the host has seen them."""
        n = logits.shape[0]
        out = torch.empty(n, dtype=torch.int32, device=logits.device)
        if any(t > 0 for t in temperatures):
            temp = torch.tensor(temperatures, dtype=torch.float32).to(logits.device)
            keys = torch.tensor([draw_key(self.seed, s, i) for s, i in zip(request_seeds, token_indices)],
                                dtype=torch.int32).to(logits.device)
            ops.sample(logits, temp, keys, out)
        else:
            ops.sample(logits, None, None, out)
        return Drawn(out)

    def sample(self, logits: torch.Tensor, temperatures: list[float], request_seeds: list[int],
               token_indices: list[int]) -> list[int]:
        """One token per row of ``logits [N, vocab]`` (float32, on the GPU)."""
        return self.launch(logits, temperatures, request_seeds, token_indices).tokens()


class Drawn:
    """Tokens of one draw: on the GPU at once, on the host when :meth:`tokens` has waited for the copy."""

    def __init__(self, device_tokens: torch.Tensor):
        self.device = device_tokens
        self._host = None
        self._copied = None
        if device_tokens.is_cuda:
            self._host = torch.empty(device_tokens.shape, dtype=device_tokens.dtype, pin_memory=True)
            self._host.copy_(device_tokens, non_blocking=True)
            self._copied = torch.cuda.Event()
            self._copied.record()

    def tokens(self) -> list[int]:
        if self._copied is None:
            return self.device.tolist()
        self._copied.synchronize()
        return self._host.tolist()

"""Interfaces of the parts a layer is put together from, and their registries.

A part is built from its specification (plain sizes and constants), declares the
tensors it wants by relative name, receives them, and runs on the tokens of one
step.  No part sees a configuration, a layer index or the model it is in.

Five kinds of parts, each with a registry from the specification's ``kind`` to a class:

===================  =====================================================================
``Norm``             ``forward(stream) -> h``: folds the stream's pending branch output
                     into the 32-bit residual and returns the normalised activations.
``PositionEncoding`` ``apply(q, k, positions)``: in place on ``[T, heads, head_dim]`` views.
``Mixer``            ``forward(h, ctx, cache) -> [T, hidden]``: mixes tokens; declares the
                     cache it needs (pages per token and/or a fixed-size state per request).
``FeedForward``      ``forward(h, ctx) -> [T, hidden]``: stateless.
``Block``            ``forward(stream, ctx, cache) -> stream``: arranges the four above.
===================  =====================================================================
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

import torch

from ..config.base import ConfigError, PartSpec


# ------------------------------------------------------------------ weights of a part

# How a tensor is kept on the GPU, whatever its shape: a dtype policy.
KEEP_COMPUTE = "compute"     # the engine's compute dtype (matrix-product operands)
KEEP_STORED = "stored"       # as stored: bfloat16 stays bfloat16, 32-bit stays 32-bit; a 32-bit engine widens
KEEP_FLOAT32 = "float32"     # always 32-bit, also under a bfloat16 engine (a router, a gate, a decay)
KEEP_INT32 = "int32"         # integer tables
DTYPE_POLICIES = (KEEP_COMPUTE, KEEP_STORED, KEEP_FLOAT32, KEEP_INT32)

# The laws of the random-weights mode: name -> f(shape, generator, device, std) -> float32 (or int32) tensor.
# A part that needs another law (a log-decay, a positive-only scale) adds it here by name and declares it.
INIT_LAWS: dict[str, Callable] = {}


def register_init_law(name: str) -> Callable[[Callable], Callable]:
    def add(fn: Callable) -> Callable:
        INIT_LAWS[name] = fn
        return fn
    return add


@register_init_law("normal")
def _init_normal(shape, gen, device, std):
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std


@register_init_law("one_plus_normal")
def _init_one_plus_normal(shape, gen, device, std):
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std + 1.0


@register_init_law("random_table")
def _init_random_table(shape, gen, device, std):
    return torch.randint(0, 2 ** 15, shape, generator=gen, device=device, dtype=torch.int32)


@dataclass(frozen=True)
class WeightSpec:
    """One tensor a part wants from the checkpoint.

    ``keep``: the dtype policy, one of :data:`DTYPE_POLICIES`, independent of the tensor's shape:
    ``compute`` tensors take the engine's compute dtype (matrix-product operands), ``stored``
    tensors keep the dtype they are stored in (bfloat16 stays bfloat16, 32-bit stays 32-bit; a 32-bit
    engine widens them: norm weights, biases), ``float32`` tensors are 32-bit under every engine,
    ``int32`` tensors are integer tables.
    ``init``: the name of a law in :data:`INIT_LAWS` for the random-weights mode (``normal`` =
    N(0, std), ``one_plus_normal`` = 1 + N(0, std), ``random_table`` = integers).
    ``optional``: the checkpoint may leave it out (a tied head).
    """
    shape: tuple[int, ...]
    keep: str = KEEP_COMPUTE
    init: str = "normal"
    optional: bool = False

    def __post_init__(self):
        if self.keep not in DTYPE_POLICIES:
            raise ConfigError(f"a tensor's dtype policy is one of {', '.join(DTYPE_POLICIES)}, not {self.keep!r}")
        if self.init not in INIT_LAWS:
            raise ConfigError(f"no initialisation law {self.init!r}; known: {', '.join(sorted(INIT_LAWS))}")

    @property
    def integer(self) -> bool:
        return self.keep == KEEP_INT32


def place(t: torch.Tensor, keep: str, dtype: torch.dtype, device) -> torch.Tensor:
    """``t`` on ``device`` in the dtype that the policy ``keep`` gives it under an engine of ``dtype``."""
    if keep not in DTYPE_POLICIES:
        raise ConfigError(f"a tensor's dtype policy is one of {', '.join(DTYPE_POLICIES)}, not {keep!r}")
    if keep == KEEP_COMPUTE:
        return t.to(device=device, dtype=dtype).contiguous()
    if keep == KEEP_INT32:
        return t.to(device=device, dtype=torch.int32).contiguous()
    if keep == KEEP_FLOAT32 or dtype == torch.float32 or t.dtype not in (torch.bfloat16, torch.float32):
        t = t.to(torch.float32)
    return t.to(device).contiguous()


class Part:
    """Common protocol: declare tensors, receive them, say whether a step may be recorded.

    ``graph_safe``: nothing in the part's ``forward`` depends on host-side values of the step (no
    ``.item()``, ``.nonzero()``, shapes that follow the tokens), so a decode step through it can be
    captured once as a HIP graph and replayed.  ``False`` unless a part says otherwise; a model runs
    under graphs only if every part of every block says ``True``.  A subclass that overrides a stage or
    adds a hook that reads host values must set it back to ``False``."""

    graph_safe = False

    def __init__(self, spec: PartSpec, dtype: torch.dtype, device: torch.device):
        self.spec = spec
        self.dtype = dtype
        self.device = device

    def weight_specs(self) -> dict[str, WeightSpec]:
        return {}

    def load_weights(self, tensors: dict[str, torch.Tensor]) -> None:
        """``tensors``: the declared names (those present) -> CPU tensors as stored."""

    def parts(self):
        """This part and every part inside it (a block's four, a mixer's position encoding)."""
        yield self

    # helpers ---------------------------------------------------------------------
    def _place(self, t: torch.Tensor, keep: str) -> torch.Tensor:
        return place(t, keep, self.dtype, self.device)


# ------------------------------------------------------------------------ cache needs

@dataclass(frozen=True)
class PagedNeed:
    """Per-token cache: some planes of ``[heads, width]`` per token, kept for all tokens
    (``window=None``) or for the last ``window`` tokens.  ``planes`` is a count of planes of
    ``[num_heads, head_dim]`` each (keys and values are two), or a tuple of ``(heads, width)``, one per
    plane, for planes that differ (a compressed latent beside a small rotated part).  ``dtype``: the
    planes' element type; ``None`` is the model's.  Layers with equal needs share a group of pages."""
    num_heads: int
    head_dim: int
    window: int | None = None
    planes: int | tuple[tuple[int, int], ...] = 2
    dtype: torch.dtype | None = None

    @property
    def plane_shapes(self) -> tuple[tuple[int, int], ...]:
        """``(heads, width)`` of every plane."""
        if isinstance(self.planes, int):
            return ((self.num_heads, self.head_dim),) * self.planes
        return tuple((int(h), int(w)) for h, w in self.planes)


@dataclass(frozen=True)
class StateNeed:
    """Fixed-size per-request state: one tensor of ``shape`` per slot, zero when a
    request is admitted."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


# --------------------------------------------------------------------------- streams

class Stream:
    """The hidden state between parts: a 32-bit residual ``[T, hidden]`` and the output
    of the last branch that is still to be added to it (``pending``, or ``None``).
    The next norm adds ``pending`` in 32-bit while it normalises, which saves one pass
    over the residual per branch.  ``pending`` is ``[T, hidden]`` in the activation dtype, or
    float32 ``[P, T, hidden]``: P slabs of partial sums that the norm adds up as well."""

    __slots__ = ("residual", "pending")

    def __init__(self, residual: torch.Tensor, pending: torch.Tensor | None = None):
        self.residual = residual
        self.pending = pending


class LazyNorm:
    """A norm that has not run yet, handed to the part that reads its output: ``norm(residual + pending)`` of
    the stream.  It states which norm it is (``kind``, the norm's registry name) and carries that kind's
    constants (``rmsnorm``: ``weight`` and ``eps``), so that a consumer whose kernel can make a norm of that
    kind itself does so and calls :meth:`done` with the new residual it wrote; a consumer that does not know the
    kind, or whose shapes do not fit, calls :meth:`value`, which runs the norm the usual way (once).  The norm's
    own kernel is a launch and a trip to memory that a step of one token can do without."""

    def __init__(self, norm, stream: "Stream", kind: str, **constants):
        self.norm = norm
        self.stream = stream
        self.kind = kind
        self.constants = constants
        self._value = None

    def rmsnorm(self):
        """``(weight, eps)`` if this is a root-mean-square norm with one weight vector, else ``None``."""
        if self.kind != "rmsnorm":
            return None
        return self.constants["weight"], self.constants["eps"]

    @property
    def residual(self):
        return self.stream.residual

    @property
    def pending(self):
        return self.stream.pending

    def value(self) -> torch.Tensor:
        if self._value is None:
            self._value = self.norm.forward(self.stream)
        return self._value

    def done(self, residual_out: torch.Tensor) -> None:
        self.stream.residual = residual_out
        self.stream.pending = None


# ----------------------------------------------------------------------- part kinds

class Norm(Part):
    def forward(self, stream: Stream, rows: torch.Tensor | None = None, gain: float = 1.0) -> torch.Tensor:
        """Add ``stream.pending`` into ``stream.residual`` (both kept up to date) and
        return ``norm(residual) * gain`` in the activation dtype (the factor applied in 32-bit, before
        the one rounding of the result).  With ``rows`` (int32 indices) only those rows are read
        and returned, and the stream is left untouched."""
        raise NotImplementedError

    def lazy(self, stream: Stream) -> "LazyNorm | None":
        """A :class:`LazyNorm` of the stream where a consumer's kernel could make this norm itself (the
        norm says for which steps that is worth offering), else ``None``.  The :class:`LazyNorm` must name
        its kind and carry that kind's constants: consumers fuse only the kinds they know and run every
        other through :meth:`LazyNorm.value`."""
        return None


class PositionEncoding(Part):
    def apply(self, q: torch.Tensor, k: torch.Tensor | None, positions: torch.Tensor) -> None:
        """Encode ``positions [T]`` into ``q [T, heads, head_dim]`` and ``k`` in place
        (views with unit stride on the last axis)."""
        raise NotImplementedError

    def fused_inv_freq(self) -> torch.Tensor | None:
        """A declared capability: an encoding that is the split-half rotary form over the whole head,
        ``angle[j] = float32(position) * inv_freq[j]`` turning the pair ``(j, j + head_dim/2)``, returns its
        float32 ``inv_freq [head_dim/2]`` here, and a mixer may then fold the rotation into its own kernels
        (the projection's epilogue, the cache write) instead of calling :meth:`apply`.  ``None`` (the
        default): the encoding is applied through :meth:`apply` only."""
        return None


class Mixer(Part):
    def paged_need(self) -> PagedNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, h: torch.Tensor, ctx, cache) -> torch.Tensor:
        """``h [T, hidden]`` -> ``[T, hidden]``.  ``cache`` is this run's
        :class:`torchlet_amd.cache.manager.LayerCache` (or ``None`` when the mixer
        declared no need)."""
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, ctx) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    mixer: Mixer

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        raise NotImplementedError


# ------------------------------------------------------------------------ registries

class Registry:
    """``kind`` -> class, with a decorator to add to it and a clear error on a miss."""

    def __init__(self, what: str):
        self.what = what
        self._classes: dict[str, type] = {}

    def register(self, kind: str) -> Callable[[type], type]:
        def add(cls: type) -> type:
            self._classes[kind] = cls
            return cls
        return add

    def unregister(self, kind: str) -> None:
        self._classes.pop(kind, None)

    def names(self) -> list[str]:
        return sorted(self._classes)

    def build(self, spec: PartSpec, dtype: torch.dtype, device: torch.device):
        cls = self._classes.get(spec.kind)
        if cls is None:
            raise ConfigError(f"no {self.what} of kind {spec.kind!r}; known: {', '.join(self.names())}")
        return cls(spec, dtype, device)


NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
BLOCKS = Registry("block")

"""Typed model configurations and the part specifications they expand to.

A configuration class reads an architecture's own ``config.json`` keys, checks them
and expands into a :class:`ModelSpec`: plain data that names, layer by layer, which
mixer, feed-forward, norm and position encoding to build and with which sizes, and
the order in which the layers run.  Parts are built from these specifications only;
none of them sees a configuration or knows which model it is in.
"""
from __future__ import annotations

import dataclasses
import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A ``config.json`` that is incomplete, inconsistent or asks for what is not built."""


# ----------------------------------------------------------------------- part specs
# ``kind`` selects the class in the matching registry of ``torchlet_amd.parts``.

@dataclass(frozen=True)
class PartSpec:
    kind: ClassVar[str] = ""


@dataclass(frozen=True)
class RMSNormSpec(PartSpec):
    kind: ClassVar[str] = "rmsnorm"
    dim: int = 0
    eps: float = 1e-6


@dataclass(frozen=True)
class RotarySpec(PartSpec):
    """Split-half rotary position encoding over the whole head."""
    kind: ClassVar[str] = "rope_split_half"
    head_dim: int = 0
    theta: float = 1_000_000.0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec(PartSpec):
    """Grouped-query attention over a paged key/value cache."""
    kind: ClassVar[str] = "gqa_attention"
    hidden: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    qkv_bias: bool = True
    window: int | None = None          # None: every earlier key; W: the last W keys
    position: PartSpec | None = None   # position encoding applied to q and k
    scale: float | None = None         # factor on the scores before the softmax; None: head_dim ** -0.5


@dataclass(frozen=True)
class SwiGLUSpec(PartSpec):
    kind: ClassVar[str] = "swiglu"
    hidden: int = 0
    intermediate: int = 0


@dataclass(frozen=True)
class BlockSpec(PartSpec):
    """One layer: a mixer and a feed-forward, each behind its own norm.

    The ``*_name`` fields are the checkpoint's sub-module names of the four parts.
    """
    kind: ClassVar[str] = "prenorm_residual"
    mixer: PartSpec = None            # type: ignore[assignment]
    ffn: PartSpec = None              # type: ignore[assignment]
    mixer_norm: PartSpec = None       # type: ignore[assignment]
    ffn_norm: PartSpec = None         # type: ignore[assignment]
    mixer_name: str = "self_attn"
    ffn_name: str = "mlp"
    mixer_norm_name: str = "input_layernorm"
    ffn_norm_name: str = "post_attention_layernorm"


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order: which layer runs, and whose cache it uses.

    ``cache_of`` is ``None`` when this run owns a cache of its own (keyed by its place
    in the order), or the index of an earlier entry of the order whose cache this run
    reads without writing to it.
    """
    layer: int
    cache_of: int | None = None


@dataclass(frozen=True)
class ModelSpec:
    """Everything needed to build a decoder: parts, their names, and the run order."""
    vocab_size: int
    hidden: int
    layers: tuple[BlockSpec, ...]
    order: tuple[RunEntry, ...]
    final_norm: PartSpec
    tie_head: bool
    max_positions: int
    embed_name: str = "model.embed_tokens"
    layers_prefix: str = "model.layers"
    final_norm_name: str = "model.norm"
    head_name: str = "lm_head"
    embed_scale: float = 1.0       # factor on the embedding rows as they enter the residual stream
    logit_scale: float = 1.0       # factor on the logits (applied to the final norm's output, in 32-bit)
    head_bias: bool = False        # the output head has a bias vector ``<head_name>.bias``

    def __post_init__(self):
        for i, e in enumerate(self.order):
            if not 0 <= e.layer < len(self.layers):
                raise ConfigError(f"run order entry {i} names layer {e.layer}; there are {len(self.layers)} layers")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ConfigError(f"run order entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.order[e.cache_of].cache_of is not None:
                    raise ConfigError(f"run order entry {i} reads the cache of entry {e.cache_of}, which owns none")


# ------------------------------------------------------------------------- configs

@dataclass(frozen=True)
class ModelConfig:
    """Base of every architecture's typed configuration.

    Subclasses declare their ``config.json`` keys as dataclass fields (a field without
    a default is required), check them in :meth:`validate` and expand to parts in
    :meth:`to_spec`.
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, d: dict[str, Any]) -> "ModelConfig":
        d = cls.normalise(dict(d))
        kwargs = {}
        missing = []
        for f in fields(cls):
            if f.name in d and d[f.name] is not None:
                kwargs[f.name] = d[f.name]
            elif f.default is dataclasses.MISSING and f.default_factory is dataclasses.MISSING:
                missing.append(f.name)
        if missing:
            raise ConfigError(f"{cls.architecture}: config.json lacks required key(s): {', '.join(missing)}")
        try:
            cfg = cls(**kwargs)
        except TypeError as exc:  # wrong python type for a field
            raise ConfigError(f"{cls.architecture}: {exc}") from exc
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str | Path) -> "ModelConfig":
        path = Path(path)
        if path.is_dir():
            path = path / "config.json"
        return cls.from_dict(json.loads(path.read_text()))

    @classmethod
    def normalise(cls, d: dict[str, Any]) -> dict[str, Any]:
        """Hook: map alternative spellings of keys onto the fields (default: none)."""
        return d

    def validate(self) -> None:  # pragma: no cover - overridden
        pass

    def to_spec(self) -> ModelSpec:  # pragma: no cover - overridden
        raise NotImplementedError

    def to_dict(self) -> dict[str, Any]:
        """The ``config.json`` content of this configuration."""
        d = {f.name: getattr(self, f.name) for f in fields(self)}
        d["architectures"] = [self.architecture]
        return d

    def save(self, folder: str | Path) -> None:
        Path(folder).mkdir(parents=True, exist_ok=True)
        (Path(folder) / "config.json").write_text(json.dumps(self.to_dict(), indent=2) + "\n")


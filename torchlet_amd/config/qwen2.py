"""Configuration of the Qwen2 / Qwen2.5 dense decoder (``Qwen2ForCausalLM``).

Keys, meanings and defaults follow the reference's reader
(/root/reference/src/torchlet/v10_triton_paged_gqa/model/qwen2_5.py:8-36,75):
``num_key_value_heads`` defaults to the number of heads, ``rms_norm_eps`` to 1e-6,
``attention_bias`` to True, ``rope_theta`` is taken from ``rope_parameters`` when that
dictionary has it, else from the top level, else 1e6, ``tie_word_embeddings`` to False.

Keys the reference never reads but Qwen2 folders carry are read here too:
``head_dim`` (default ``hidden_size // num_attention_heads``), ``hidden_act`` (only
``silu`` is built), ``rope_scaling`` (must be absent or null) and the window keys:
with ``use_sliding_window`` the layers from ``max_window_layers`` on attend to the
last ``sliding_window`` keys only, the earlier layers to all of them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import (
    AttentionSpec,
    BlockSpec,
    ConfigError,
    ModelConfig,
    ModelSpec,
    RMSNormSpec,
    RotarySpec,
    RunEntry,
    SwiGLUSpec,
)


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    architecture: ClassVar[str] = "Qwen2ForCausalLM"

    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    intermediate_size: int
    max_position_embeddings: int
    num_key_value_heads: int = 0          # 0: same as num_attention_heads
    head_dim: int = 0                     # 0: hidden_size // num_attention_heads
    rms_norm_eps: float = 1e-6
    attention_bias: bool = True
    rope_theta: float = 1_000_000.0
    tie_word_embeddings: bool = False
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: int = 0               # 0: none given
    max_window_layers: int = -1           # -1: every layer attends to all keys
    torch_dtype: str = ""                 # "": the folder does not say; the engine then goes by what it stores
    bos_token_id: int = -1
    eos_token_id: int = -1

    @classmethod
    def normalise(cls, d: dict[str, Any]) -> dict[str, Any]:
        rope_parameters = d.get("rope_parameters")
        if isinstance(rope_parameters, dict) and "rope_theta" in rope_parameters:
            d["rope_theta"] = rope_parameters["rope_theta"]
        if d.get("rope_scaling") not in (None, {}):
            raise ConfigError("Qwen2ForCausalLM: rope_scaling is not built; it must be absent or null")
        if isinstance(d.get("eos_token_id"), (list, tuple)):
            d["eos_token_id"] = d["eos_token_id"][0] if d["eos_token_id"] else None
        if "dtype" in d and "torch_dtype" not in d:
            d["torch_dtype"] = d["dtype"]
        return d

    def __post_init__(self):
        if self.num_key_value_heads == 0:
            object.__setattr__(self, "num_key_value_heads", self.num_attention_heads)
        if self.head_dim == 0 and self.num_attention_heads > 0:
            object.__setattr__(self, "head_dim", self.hidden_size // self.num_attention_heads)
        if self.max_window_layers < 0:
            object.__setattr__(self, "max_window_layers", self.num_hidden_layers)
        object.__setattr__(self, "rope_theta", float(self.rope_theta))
        object.__setattr__(self, "rms_norm_eps", float(self.rms_norm_eps))

    @property
    def num_kv_groups(self) -> int:
        return self.num_attention_heads // self.num_key_value_heads

    def validate(self) -> None:
        a = self.architecture
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "intermediate_size", "max_position_embeddings", "num_key_value_heads", "head_dim"):
            v = getattr(self, name)
            if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
                raise ConfigError(f"{a}: {name} must be a positive integer, got {v!r}")
        if self.num_key_value_heads > self.num_attention_heads or self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"{a}: num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"{a}: head_dim must be even for the split-half rotation, got {self.head_dim}")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"{a}: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not self.rope_theta > 0:
            raise ConfigError(f"{a}: rope_theta must be positive, got {self.rope_theta}")
        if self.hidden_act != "silu":
            raise ConfigError(f"{a}: hidden_act {self.hidden_act!r} is not built; only 'silu'")
        if self.use_sliding_window:
            if self.sliding_window <= 0:
                raise ConfigError(f"{a}: use_sliding_window needs a positive sliding_window")
            if not 0 <= self.max_window_layers <= self.num_hidden_layers:
                raise ConfigError(f"{a}: max_window_layers must lie in [0, num_hidden_layers]")

    def window_of(self, layer: int) -> int | None:
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window
        return None

    def to_spec(self) -> ModelSpec:
        norm = RMSNormSpec(dim=self.hidden_size, eps=self.rms_norm_eps)
        rotary = RotarySpec(head_dim=self.head_dim, theta=self.rope_theta,
                            max_positions=self.max_position_embeddings)
        ffn = SwiGLUSpec(hidden=self.hidden_size, intermediate=self.intermediate_size)
        layers = tuple(
            BlockSpec(
                mixer=AttentionSpec(
                    hidden=self.hidden_size,
                    num_heads=self.num_attention_heads,
                    num_kv_heads=self.num_key_value_heads,
                    head_dim=self.head_dim,
                    qkv_bias=self.attention_bias,
                    window=self.window_of(i),
                    position=rotary,
                ),
                ffn=ffn,
                mixer_norm=norm,
                ffn_norm=norm,
            )
            for i in range(self.num_hidden_layers)
        )
        return ModelSpec(
            vocab_size=self.vocab_size,
            hidden=self.hidden_size,
            layers=layers,
            order=tuple(RunEntry(layer=i) for i in range(self.num_hidden_layers)),
            final_norm=norm,
            tie_head=self.tie_word_embeddings,
            max_positions=self.max_position_embeddings,
        )

    def to_dict(self) -> dict[str, Any]:
        d = super().to_dict()
        d["model_type"] = "qwen2"
        for key in ("bos_token_id", "eos_token_id"):
            if d[key] < 0:
                d[key] = None
        if not d["torch_dtype"]:
            d["torch_dtype"] = None
        if not self.use_sliding_window and self.sliding_window == 0:
            d["sliding_window"] = None
        return d

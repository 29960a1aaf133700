"""From a model folder to a model on the GPU and a step function over a cache."""
from __future__ import annotations

from pathlib import Path

import torch

from ..cache.manager import CacheManager
from ..config.base import ModelConfig
from ..kernels import ops
from ..models.decoder import DecoderModel
from ..registry import load_config
from ..weights.loader import folder_dtype, load_folder, load_into
from .config import EngineConfig
from .runner import ModelRunner

DTYPES = {
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}; choose bfloat16 or float32") from None


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise RuntimeError("torchlet_amd runs on an AMD GPU only and none is visible (torch.cuda.is_available() is False)")
    return torch.device("cuda", torch.cuda.current_device())


def build_model(config: ModelConfig, dtype, device=None, tensors=None, folder: str | Path | None = None) -> DecoderModel:
    """Build the configuration's model on the GPU and load ``tensors`` (a mapping) or the
    safetensors files of ``folder`` into it.  Compiles the kernels the model needs first."""
    dtype = parse_dtype(dtype)
    device = device if device is not None else require_gpu()
    model = DecoderModel(config.to_spec(), dtype, device)
    if torch.device(device).type == "cuda":
        ops.load(model.kernel_libraries())
    if tensors is not None:
        load_into(model, tensors)
    elif folder is not None:
        load_folder(model, folder)
    return model


def resolve_dtype(folder: str | Path, config: ModelConfig, dtype=None) -> str:
    """The engine's compute dtype for a model folder: ``dtype`` if the caller names one (the weights are
    converted at load), else what the folder says: its ``config.json``'s ``torch_dtype`` (for a configuration
    class that reads the key), else the element type of its first floating-point tensor.  The reference types
    its parameters and its cache after the checkpoint (/root/reference/src/torchlet/utils.py:18-38,
    v10_triton_paged_gqa/engine.py:58), so a folder stored in 32-bit gives a 32-bit engine."""
    if dtype is not None:
        return "float32" if parse_dtype(dtype) == torch.float32 else "bfloat16"
    return folder_dtype(folder, getattr(config, "torch_dtype", None) or None)


def load_model(folder: str | Path, dtype=None, device=None) -> tuple[ModelConfig, DecoderModel]:
    """``dtype=None``: the folder's own (see :func:`resolve_dtype`)."""
    config = load_config(folder)
    return config, build_model(config, resolve_dtype(folder, config, dtype), device, folder=folder)


def make_runner(model: DecoderModel, config: EngineConfig | None = None, *, page_size: int | None = None,
                num_pages: int | None = None, max_requests: int | None = None, use_graphs: bool | None = None,
                max_model_len: int | None = None, max_step_tokens: int | None = None) -> ModelRunner:
    """The step function over a cache of its own, from an :class:`EngineConfig` (the keywords override its
    fields; ``max_requests`` is its ``max_slots``).  Without ``num_pages`` the pool holds a sequence of the
    greatest length for every slot, as far as free memory goes.  ``max_step_tokens``: the caller's bound on
    the tokens of a step (a scheduler's budget), which sizes the pools of windowed groups; ``None`` for
    callers that step as they like."""
    from dataclasses import replace
    config = config or EngineConfig()
    given = dict(page_size=page_size, num_pages=num_pages, max_slots=max_requests, use_graphs=use_graphs, max_model_len=max_model_len)
    if config.dtype is None:             # not named: the dtype the model was built in
        given["dtype"] = "float32" if model.dtype == torch.float32 else "bfloat16"
    config = replace(config, **{k: v for k, v in given.items() if v is not None})
    if parse_dtype(config.dtype) != model.dtype:
        raise ValueError(f"the engine is configured for {config.dtype}, the model was built in {model.dtype}")
    plan = model.cache_plan()
    if config.num_pages is None:
        probe = CacheManager(plan, page_size=config.page_size, num_pages=2, max_requests=1, dtype=model.dtype, device=None,
                             max_step_tokens=max_step_tokens)
        free = torch.cuda.mem_get_info(model.device)[0] if torch.device(model.device).type == "cuda" else None
        config = config.resolve(model.spec.max_positions, probe.bytes_per_page(), free)
    cache = CacheManager(plan, page_size=config.page_size, num_pages=config.num_pages, max_requests=config.max_slots,
                         dtype=model.dtype, device=model.device, max_step_tokens=max_step_tokens)
    runner = ModelRunner(model, cache, use_graphs=config.use_graphs, max_model_len=config.max_model_len)
    runner.config = config
    return runner


def make_engine(model: DecoderModel, config: EngineConfig):
    """Scheduler, step function and sampler over a cache, all sized by ``config``."""
    from .engine import Engine
    runner = make_runner(model, config, max_step_tokens=config.max_tokens_per_step if config.bounded_steps else None)
    return Engine(runner, max_tokens_per_step=config.max_tokens_per_step, seed=config.seed, lookahead=config.lookahead)

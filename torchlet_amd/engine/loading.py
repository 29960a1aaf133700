"""From a model folder to a model on the GPU and a step function over a cache."""
from __future__ import annotations

from pathlib import Path

import torch

from ..cache.manager import CacheManager
from ..config.base import ModelConfig
from ..kernels import ops
from ..models.decoder import DecoderModel
from ..registry import load_config
from ..weights.loader import load_folder, load_into
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


def load_model(folder: str | Path, dtype="bfloat16", device=None) -> tuple[ModelConfig, DecoderModel]:
    config = load_config(folder)
    return config, build_model(config, dtype, device, folder=folder)


def make_runner(model: DecoderModel, *, page_size: int, num_pages: int, max_requests: int,
                use_graphs: bool = False) -> ModelRunner:
    cache = CacheManager(model.cache_plan(), page_size=page_size, num_pages=num_pages,
                         max_requests=max_requests, dtype=model.dtype, device=model.device)
    return ModelRunner(model, cache, use_graphs=use_graphs)

"""Random weights from a configuration and a seed.

Laws: matrices and biases ``N(0, 0.02)``, norm weights ``1 + N(0, 0.02)``; every tensor names its law
(:data:`~torchlet_amd.parts.base.INIT_LAWS`, to which a part may add one), drawn in 32-bit
from one ``torch.Generator(seed)`` in the order of the model's tensor declarations, then
rounded to the storage dtype (a tensor whose policy is 32-bit is stored in 32-bit).  :func:`write_model_folder` writes ``config.json`` and
``model.safetensors`` so that the engine and any other reader load identical values;
:func:`random_tensors` makes the same kind of tensors directly on a device (for
benchmark-size models, where a detour over a file would take minutes).
"""
from __future__ import annotations

from collections.abc import Mapping
from pathlib import Path

import torch
from safetensors.torch import save_file

from ..config.base import ModelConfig
from ..models.decoder import DecoderModel
from ..parts.base import INIT_LAWS, KEEP_FLOAT32

STD = 0.02


def _draw(spec, gen: torch.Generator, device) -> torch.Tensor:
    law = "random_table" if spec.integer and spec.init == "normal" else spec.init
    return INIT_LAWS[law](spec.shape, gen, device, STD)


def random_tensors(config: ModelConfig, seed: int, dtype: torch.dtype = torch.bfloat16, device="cpu") -> dict[str, torch.Tensor]:
    """``name -> tensor`` for every tensor the architecture's model declares (a tied head
    is left out, as in a checkpoint)."""
    model = DecoderModel(config.to_spec(), torch.float32, "cpu")
    gen = torch.Generator(device=device).manual_seed(int(seed))
    out = {}
    for name, spec in model.weight_specs().items():
        if spec.optional:
            continue
        t = _draw(spec, gen, device)
        out[name] = t if spec.integer else t.to(torch.float32 if spec.keep == KEEP_FLOAT32 else dtype)
    return out


class RandomTensors(Mapping):
    """``name -> tensor`` like :func:`random_tensors`, but every tensor is drawn when it is asked for and not kept,
    from a generator of its own (seeded by ``seed`` and the tensor's place in the declarations), so that a model far
    larger than half the GPU's memory can be filled without a second copy of its weights standing by.  Shapes and
    element types can be asked for without drawing (``shape``, ``stored_dtype``, as of a folder of safetensors)."""

    def __init__(self, config: ModelConfig, seed: int, dtype: torch.dtype = torch.bfloat16, device="cpu"):
        model = DecoderModel(config.to_spec(), torch.float32, "cpu")
        self._specs = {n: s for n, s in model.weight_specs().items() if not s.optional}
        self._index = {n: i for i, n in enumerate(self._specs)}
        self.seed, self.dtype, self.device = int(seed), dtype, device

    def __getitem__(self, name: str) -> torch.Tensor:
        spec = self._specs[name]
        gen = torch.Generator(device=self.device).manual_seed(self.seed * 1_000_003 + self._index[name])
        t = _draw(spec, gen, self.device)
        return t if spec.integer else t.to(torch.float32 if spec.keep == KEEP_FLOAT32 else self.dtype)

    def __iter__(self):
        return iter(self._specs)

    def __len__(self):
        return len(self._specs)

    def shape(self, name: str) -> tuple[int, ...]:
        return tuple(self._specs[name].shape)

    def stored_dtype(self, name: str) -> str:
        if self._specs[name].integer:
            return "I32"
        kept32 = self._specs[name].keep == KEEP_FLOAT32 or self.dtype == torch.float32
        return "F32" if kept32 else {torch.bfloat16: "BF16", torch.float16: "F16"}[self.dtype]


def write_model_folder(config: ModelConfig, seed: int, folder: str | Path, dtype: torch.dtype = torch.bfloat16) -> Path:
    """Write ``config.json`` and ``model.safetensors`` (tensors stored in ``dtype``)."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    d = config.to_dict()
    d["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32", torch.float16: "float16"}[dtype]
    import json
    (folder / "config.json").write_text(json.dumps(d, indent=2) + "\n")
    tensors = {k: v.contiguous() for k, v in random_tensors(config, seed, dtype, "cpu").items()}
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder

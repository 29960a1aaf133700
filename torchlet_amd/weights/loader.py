"""Weights from safetensors, by tensor name.

Every ``*.safetensors`` file of the model folder is read (sorted by name, as the
reference does, /root/reference/src/torchlet/v10_triton_paged_gqa/llm.py:70-79), but a
name that appears in two files is an error instead of a silent overwrite.  Names are the
checkpoint's own; nothing is renamed.  Before anything is placed on the GPU the names and
shapes are compared with what the model declares, and **one** error lists every missing
tensor, every unexpected one and every wrong shape; the reference only logs these
(llm.py:52-54) and runs on with initial values.

Tensors are handed to the parts as stored: bfloat16 stays bfloat16 and a tensor stored in
32-bit stays so, except that matrix-product operands take the engine's compute dtype and
a 32-bit engine widens everything (the dtype policy of :class:`~torchlet_amd.parts.base.WeightSpec`).
The engine's compute dtype itself follows the folder unless the caller names one
(:func:`folder_dtype`): the reference types every parameter after its checkpoint tensor
(/root/reference/src/torchlet/utils.py:18-38), so a folder stored in 32-bit runs in 32-bit.
"""
from __future__ import annotations

from collections.abc import Mapping
from pathlib import Path

import torch
from safetensors import safe_open

from ..parts.base import WeightSpec


class WeightError(ValueError):
    """The checkpoint does not fit the model; the message lists every discrepancy."""


class SafetensorsFolder(Mapping):
    """Read-only mapping ``name -> CPU tensor`` over the files of a folder; a tensor is
    read from disk when it is asked for."""

    def __init__(self, folder: str | Path):
        self.folder = Path(folder)
        files = sorted(self.folder.glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"not found safetensors files in {self.folder}")
        self._where: dict[str, Path] = {}
        self._shapes: dict[str, tuple[int, ...]] = {}
        self._dtypes: dict[str, str] = {}
        duplicates = []
        for path in files:
            with safe_open(str(path), framework="pt") as f:
                for name in f.keys():
                    if name in self._where:
                        duplicates.append(f"{name} ({self._where[name].name} and {path.name})")
                        continue
                    self._where[name] = path
                    sl = f.get_slice(name)
                    self._shapes[name] = tuple(sl.get_shape())
                    self._dtypes[name] = sl.get_dtype()
        if duplicates:
            raise WeightError("tensor(s) stored in more than one file: " + "; ".join(duplicates))
        self._open: dict[Path, object] = {}

    def __getitem__(self, name: str) -> torch.Tensor:
        path = self._where[name]
        f = self._open.get(path)
        if f is None:
            f = self._open[path] = safe_open(str(path), framework="pt")
        return f.get_tensor(name)

    def __iter__(self):
        return iter(self._where)

    def __len__(self):
        return len(self._where)

    def shape(self, name: str) -> tuple[int, ...]:
        return self._shapes[name]

    def stored_dtype(self, name: str) -> str:
        return self._dtypes[name]

    def close(self) -> None:
        self._open.clear()


_FLOAT_TAGS = {"F64", "F32", "F16", "BF16"}
_INT_TAGS = {"I64", "I32", "I16", "I8", "U8"}


def check_against(specs: dict[str, WeightSpec], source) -> None:
    """Raise one :class:`WeightError` listing all missing and unexpected tensors and all
    wrong shapes.  ``source`` maps names to tensors or is a :class:`SafetensorsFolder`."""
    def shape_of(name):
        return source.shape(name) if hasattr(source, "shape") else tuple(source[name].shape)

    def kind_ok(name, spec):
        if hasattr(source, "stored_dtype"):
            tag = source.stored_dtype(name)
            return tag in (_INT_TAGS if spec.integer else _FLOAT_TAGS)
        t = source[name]
        return (not t.is_floating_point()) if spec.integer else t.is_floating_point()

    missing = [n for n, s in specs.items() if n not in source and not s.optional]
    unexpected = [n for n in source if n not in specs]
    wrong = []
    for n, s in specs.items():
        if n in source:
            got = shape_of(n)
            if got != tuple(s.shape):
                wrong.append(f"{n}: stored {list(got)}, model wants {list(s.shape)}")
            elif not kind_ok(n, s):
                wrong.append(f"{n}: stored element type does not fit {'an integer table' if s.integer else 'a floating-point tensor'}")
    if missing or unexpected or wrong:
        parts = []
        if missing:
            parts.append(f"missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            parts.append(f"unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            parts.append(f"wrong shape or type ({len(wrong)}): " + "; ".join(wrong))
        raise WeightError("checkpoint does not fit the model -- " + " | ".join(parts))


def load_into(model, source) -> None:
    """Check ``source`` against ``model.weight_specs()`` and hand the tensors over."""
    check_against(model.weight_specs(), source)
    model.load_weights(source)
    if hasattr(source, "close"):
        source.close()


def load_folder(model, folder: str | Path) -> None:
    load_into(model, SafetensorsFolder(folder))


_TAG_DTYPES = {"BF16": "bfloat16", "F32": "float32", "F16": "float16", "F64": "float64"}


def folder_dtype(folder: str | Path, declared: str | None = None, probe: str | None = None) -> str:
    """The compute dtype a model folder asks for: ``declared`` (its ``config.json``'s ``torch_dtype``) if
    the folder says one, else the element type in which it stores ``probe`` (a tensor name; default: its
    first floating-point tensor), as the reference types its parameters and its cache after the checkpoint's
    tensors (/root/reference/src/torchlet/utils.py:18-38, v10_triton_paged_gqa/engine.py:58).  Only
    ``bfloat16`` and ``float32`` engines are built; any other answer is refused by name."""
    name = str(declared).replace("torch.", "").lower() if declared else None
    if name is None:
        source = SafetensorsFolder(folder)
        names = [probe] if probe is not None and probe in source else list(source)
        tags = [source.stored_dtype(n) for n in names if source.stored_dtype(n) in _FLOAT_TAGS]
        if not tags:
            raise WeightError(f"{folder} stores no floating-point tensor to take the compute dtype from")
        name = _TAG_DTYPES[tags[0]]
    name = {"bf16": "bfloat16", "fp32": "float32", "f32": "float32", "float": "float32"}.get(name, name)
    if name not in ("bfloat16", "float32"):
        raise ValueError(f"{folder} asks for a {name} engine; only bfloat16 and float32 are built "
                         f"(name one of them as dtype= to convert the weights at load)")
    return name

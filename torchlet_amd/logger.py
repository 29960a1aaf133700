"""The package's logger and the start-up reports it carries.

As the reference does (/root/reference/src/torchlet/logger.py:12-32, utils.py:41-73 and the
``logger.info`` calls of v10_triton_paged_gqa/llm.py:28-54), the engine reports at INFO level what it
runs on, which tensors the model folder holds and how it was configured; the logger stands at WARNING
unless asked otherwise, so none of it shows by default.  ``python -m torchlet_amd --verbose`` or
``get_logger(level=logging.INFO)`` turn it on.
"""
from __future__ import annotations

import logging
import sys
from typing import TextIO

FORMAT = "%(asctime)s [%(levelname)s] %(name)s %(filename)s:%(lineno)d - %(message)s"
DATE_FORMAT = "%Y-%m-%d %H:%M:%S"


def get_logger(name: str = "torchlet_amd", level: int | None = None, stream: TextIO | None = None) -> logging.Logger:
    """The named logger with one stream handler (standard error unless ``stream`` is given);
    ``level`` changes the level of the logger and of its handler, ``None`` leaves them."""
    log = logging.getLogger(name)
    log.propagate = False
    if not log.handlers:
        handler = logging.StreamHandler(stream or sys.stderr)
        handler.setFormatter(logging.Formatter(FORMAT, datefmt=DATE_FORMAT))
        log.addHandler(handler)
        if level is None:
            level = logging.WARNING
    if level is not None:
        log.setLevel(level)
        for h in log.handlers:
            h.setLevel(level)
    return log


logger = get_logger()


def backend_info() -> str:
    """What the engine runs on: torch, the GPU and its architecture, the kernel libraries loaded so far."""
    import torch

    from .kernels import build, ops

    lines = [f"torch: {torch.__version__} (hip {getattr(torch.version, 'hip', None)})",
             f"gpu visible: {torch.cuda.is_available()}"]
    if torch.cuda.is_available():
        dev = torch.cuda.current_device()
        props = torch.cuda.get_device_properties(dev)
        free, total = torch.cuda.mem_get_info(dev)
        lines += [f"device: cuda:{dev} {props.name} ({getattr(props, 'gcnArchName', '?')}), {props.multi_processor_count} compute units",
                  f"memory: {free / 2**30:.1f} GiB free of {total / 2**30:.1f} GiB"]
    lines += [f"kernels built for: {build.ARCH}, libraries in {build.lib_dir()}",
              "libraries loaded: " + (", ".join(p.rsplit('/', 1)[-1] for p in ops.loaded_libraries()) or "none yet")]
    return "\n".join(lines)


def weights_info(source) -> str:
    """One line per tensor of a model folder: name, shape, stored element type
    (``source``: a :class:`~torchlet_amd.weights.loader.SafetensorsFolder` or a mapping of tensors)."""
    rows = []
    for name in source:
        if hasattr(source, "stored_dtype"):
            rows.append((name, str(list(source.shape(name))), source.stored_dtype(name)))
        else:
            rows.append((name, str(list(source[name].shape)), str(source[name].dtype)))
    if not rows:
        return "(no tensors)"
    w0 = max(len(r[0]) for r in rows)
    w1 = max(len(r[1]) for r in rows)
    return "\n".join(f"{n:<{w0}}  {s:<{w1}}  {d}" for n, s, d in rows)

"""Compiles the HIP sources under ``csrc/`` into shared libraries for gfx950.

Each library is one translation unit built with one ``hipcc`` call, so libraries build
independently and in parallel, and a process compiles only what its model needs (the
attention kernels are compiled per head size).  Libraries live in ``torchlet_amd/lib/``
(or, when the package folder is read-only, in a per-user folder under the temporary
directory) next to a stamp of the source text and flags they were built from; a library
whose stamp no longer matches is rebuilt.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-shared", "-fPIC",
    # packed 32-bit float instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HEADERS = sorted(p.name for p in CSRC.glob("*.h"))      # every header is part of every library's stamp

# head sizes compiled by build_all(): what the tests, the smoke run and the benchmark use (each library also
# serves the seven even head sizes below its own)
DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 256)


class BuildError(RuntimeError):
    pass


def _targets(head_dims) -> dict[str, tuple[str, list[str]]]:
    t = {
        "elementwise": ("elementwise.hip", []),
        "gemm": ("gemm.hip", []),
        "sampling": ("sampling.hip", []),
    }
    for hd in head_dims:
        t[f"attention_hd{hd}"] = ("attention.hip", [f"-DTL_HEAD_DIM={hd}"])
    return t


def target(name: str) -> tuple[str, list[str]]:
    if name.startswith("attention_hd"):
        hd = int(name[len("attention_hd"):])
        if hd % 16 or not 16 <= hd <= 256:
            raise BuildError(f"attention kernels exist for head sizes that are multiples of 16 up to 256, not {hd}")
        return _targets([hd])[name]
    t = _targets([])
    if name not in t:
        raise BuildError(f"unknown kernel library {name!r}")
    return t[name]


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe-{os.getpid()}-{threading.get_ident()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


_lib_dir: Path | None = None


def lib_dir() -> Path:
    global _lib_dir
    if _lib_dir is None:
        in_tree = Path(__file__).resolve().parent.parent / "lib"
        override = os.environ.get("TORCHLET_AMD_LIB_DIR")
        if override and _writable(Path(override)):
            _lib_dir = Path(override)
        elif _writable(in_tree):
            _lib_dir = in_tree
        else:
            _lib_dir = Path(tempfile.gettempdir()) / f"torchlet_amd-{os.getuid()}" / "lib"
            if not _writable(_lib_dir):
                raise BuildError(f"no writable folder for kernel libraries (tried {in_tree} and {_lib_dir})")
    return _lib_dir


def _stamp(name: str) -> str:
    src, extra = target(name)
    h = hashlib.sha256()
    for f in [src] + HEADERS:
        h.update((CSRC / f).read_bytes())
    h.update(" ".join(FLAGS + extra).encode())
    return h.hexdigest()


def lib_path(name: str) -> Path:
    return lib_dir() / f"libtl_{name}.so"


def is_current(name: str) -> bool:
    so, st = lib_path(name), lib_path(name).with_suffix(".stamp")
    return so.exists() and st.exists() and st.read_text().strip() == _stamp(name)


def _say(msg: str) -> None:
    print(f"[torchlet_amd] {msg}", file=sys.stderr, flush=True)


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not Path(exe).exists():
        raise BuildError("hipcc not found: the HIP kernels cannot be compiled (looked on PATH and in /opt/rocm/bin)")
    return exe


def build(name: str, force: bool = False, quiet: bool = False) -> Path:
    """Compile one library unless it is current; returns its path."""
    if not force and is_current(name):
        return lib_path(name)
    src, extra = target(name)
    so = lib_path(name)
    tmp = so.with_name(f".{so.name}.{os.getpid()}.{threading.get_ident()}.tmp")
    cmd = [hipcc(), *FLAGS, *extra, f"-I{CSRC}", str(CSRC / src), "-o", str(tmp)]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())   # the compiler wants some HOME for its caches
    t0 = time.time()
    if not quiet:
        _say(f"compiling {name} for {ARCH} ...")
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    out: list[str] = []
    reader = threading.Thread(target=lambda: out.append(proc.stdout.read()), daemon=True)
    reader.start()
    last = t0
    while proc.poll() is None:
        time.sleep(0.2)
        if not quiet and time.time() - last > 10:
            last = time.time()
            _say(f"  still compiling {name} ({int(last - t0)} s)")
    reader.join()
    text = "".join(out)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise BuildError(f"hipcc failed for {name} (exit {proc.returncode}):\n{' '.join(cmd)}\n{text}")
    os.replace(tmp, so)
    so.with_suffix(".stamp").write_text(_stamp(name) + "\n")
    if not quiet:
        _say(f"built {so.name} in {time.time() - t0:.1f} s")
    return so


def build_many(names, force: bool = False, jobs: int | None = None, quiet: bool = False) -> list[Path]:
    names = list(dict.fromkeys(names))
    lib_dir()                                   # settle the folder before the threads start
    jobs = jobs or min(8, os.cpu_count() or 1, max(1, len(names)))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        return list(pool.map(lambda n: build(n, force=force, quiet=quiet), names))


def build_all(head_dims=DEFAULT_HEAD_DIMS, force: bool = False, quiet: bool = False) -> list[Path]:
    """Compile every library: the common ones and the attention kernels of ``head_dims``."""
    return build_many(list(_targets(head_dims)), force=force, quiet=quiet)

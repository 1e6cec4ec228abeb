"""Compiles the HIP sources under ``csrc/`` for gfx950 into shared libraries and loads them.

Each library is built from one or more ``.hip`` files with ``hipcc`` (no torch headers, so a
build takes seconds) and loaded with ``ctypes``.  A library's file name carries a hash of
its sources, of the headers they include and of the flags, so a changed source is never served by a
stale build.  Libraries are kept beside this file (``_lib/``); if that folder cannot be
written they go to a per-user folder under the temporary directory.  What is missing is
compiled at first use, with a progress line per file.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import re
import shutil
import subprocess
import sys
import tempfile
import time
from pathlib import Path
from typing import Dict, Iterable, Optional, Sequence

CSRC = Path(__file__).resolve().parent.parent / "csrc"
LIB_DIR = Path(__file__).resolve().parent / "_lib"
ARCH = "gfx950"

# -packed-fp32-ops off: the compiler must not form packed float instructions by itself.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # MFMA results in ordinary vector registers: the attention kernels rescale and exponentiate them, and
    # with accumulation registers every such touch costs two extra moves.
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]

# name -> sources.  "core" is everything a model needs in either dtype; further libraries
# are specialisations compiled for the sizes a model has (see ``specialised``).
LIBRARIES: Dict[str, Sequence[str]] = {
    "core": ("elementwise.hip", "rope_cache.hip", "attention_generic.hip", "gemm_generic.hip", "gemm_skinny.hip",
             "sampling.hip", "bandwidth.hip", "block.hip"),
    # the vendor's BLAS library called directly (the products of steps of many tokens); optional: without it those
    # products go through torch
    "blas": ("library_product.hip",),
}

# what a library links beside the HIP runtime
LINK_FLAGS: Dict[str, Sequence[str]] = {
    "blas": ("-L/opt/rocm/lib", "-lhipblaslt"),
}

# compiler flags of the libraries built from one source, beside HIPCC_FLAGS
SOURCE_FLAGS: Dict[str, Sequence[str]] = {
    # scores are never NaN (masked ones are -inf): a maximum then needs no quieting of signalling NaNs first, which
    # costs an instruction per operand in the softmax of every tile
    "attention_mfma.hip": ("-fno-honor-nans",),
}


def _source_flags(sources: Sequence[str]) -> list:
    return [flag for src in sources for flag in SOURCE_FLAGS.get(Path(src).name, ())]


class KernelBuildError(RuntimeError):
    pass


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise KernelBuildError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH)")


_INCLUDE = re.compile(r'^\s*#\s*include\s+"([^"]+)"', re.M)


def _headers_of(sources: Iterable[Path]) -> list:
    """The headers under ``csrc/`` that the sources include, directly or through one another, sorted by name."""
    found, todo = {}, list(sources)
    while todo:
        for name in _INCLUDE.findall(todo.pop().read_text()):
            path = CSRC / name
            if name not in found and path.is_file():
                found[name] = path
                todo.append(path)
    return [found[name] for name in sorted(found)]


def _digest(sources: Sequence[Path], defines: Sequence[str], link: Sequence[str] = ()) -> str:
    h = hashlib.sha256()
    for path in list(sources) + _headers_of(sources):
        h.update(path.name.encode())
        h.update(path.read_bytes())
    h.update(" ".join(list(HIPCC_FLAGS) + _source_flags([p.name for p in sources]) + list(defines) + list(link)).encode())
    return h.hexdigest()[:12]


def _writable_dir() -> Path:
    try:
        LIB_DIR.mkdir(exist_ok=True)
        probe = LIB_DIR / f".probe{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return LIB_DIR
    except OSError:
        alt = Path(tempfile.gettempdir()) / f"simple_inference_amd_{os.getuid()}" / "_lib"
        alt.mkdir(parents=True, exist_ok=True)
        return alt


def library_path(name: str, sources: Sequence[str], defines: Sequence[str] = ()) -> Path:
    digest = _digest([CSRC / s for s in sources], defines, LINK_FLAGS.get(name, ()))
    file = f"libsia_{name}_{digest}.so"
    if (LIB_DIR / file).is_file():
        return LIB_DIR / file
    return _writable_dir() / file


def compile_library(name: str, sources: Sequence[str], defines: Sequence[str] = (), force: bool = False,
                    verbose: bool = True) -> Path:
    """Builds (if missing or ``force``) and returns the path of the shared library."""
    out = library_path(name, sources, defines)
    if out.is_file() and not force:
        return out
    hipcc = find_hipcc()
    out.parent.mkdir(parents=True, exist_ok=True)
    tmp = out.with_suffix(f".tmp{os.getpid()}.so")
    cmd = [hipcc, *HIPCC_FLAGS, *_source_flags(sources), *[f"-D{d}" for d in defines], f"-I{CSRC}",
           *[str(CSRC / s) for s in sources], "-o", str(tmp), *LINK_FLAGS.get(name, ())]
    if verbose:
        print(f"[simple-inference_amd] compiling {name} ({', '.join(sources)}) for {ARCH} ...",
              file=sys.stderr, flush=True)
    t0 = time.time()
    env = dict(os.environ)
    if not env.get("HOME") or not os.access(env.get("HOME", "/nonexistent"), os.W_OK):
        env["HOME"] = tempfile.gettempdir()  # the compiler driver wants a writable home for its temporaries
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if proc.returncode != 0:
        try:
            tmp.unlink()
        except OSError:
            pass
        raise KernelBuildError(f"hipcc failed for {name}:\n{' '.join(cmd)}\n{proc.stdout}")
    os.replace(tmp, out)
    pattern = re.compile(rf"libsia_{re.escape(name)}_[0-9a-f]{{12}}\.so$")
    for stale in out.parent.iterdir():
        if stale != out and pattern.match(stale.name):
            try:
                stale.unlink()
            except OSError:
                pass
    if verbose:
        print(f"[simple-inference_amd] built {out.name} in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    return out


_loaded: Dict[str, ctypes.CDLL] = {}


def load_library(name: str, sources: Optional[Sequence[str]] = None, defines: Sequence[str] = ()) -> ctypes.CDLL:
    sources = sources if sources is not None else LIBRARIES[name]
    key = name + "|" + ",".join(defines)
    if key not in _loaded:
        path = compile_library(name, sources, defines)
        _loaded[key] = ctypes.CDLL(str(path))
    return _loaded[key]


def build_all(force: bool = True, verbose: bool = True, extra=()) -> None:
    """Compiles every library (the build check); ``extra`` lists (name, sources, defines)."""
    for name, sources in LIBRARIES.items():
        compile_library(name, sources, force=force, verbose=verbose)
    for name, sources, defines in extra:
        compile_library(name, sources, defines, force=force, verbose=verbose)

"""Building and loading the HIP kernel libraries.

Each ``csrc/*.hip`` file becomes one shared library under ``csrc/_build/``, compiled with
hipcc for gfx950 and loaded with ctypes.  A library's file name carries a hash of its
source, the shared header, the flags and the ``-D`` options, so a library that is found is
never stale.  A library that is not found is compiled at its first use; while hipcc runs, a
line is printed every few seconds.  There is no other implementation of these operations:
without hipcc and without a built library the call fails.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Mapping, Optional, Tuple

__all__ = ["KernelBuildError", "load_library", "build_library", "csrc_dir", "build_dir", "ARCH", "HIPCC_FLAGS"]

ARCH = "gfx950"
# Packed float32 instructions are switched off for all device code.
HIPCC_FLAGS = ("-O3", "-std=c++17", f"--offload-arch={ARCH}", "-shared", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops")

# Flags of single sources.  The matrix-core attention takes maxima of scores that are never NaN
# (masked ones are -inf): told so, the compiler drops the instruction that would quiet a signalling
# NaN before every maximum, a third of the vector instructions of its softmax.
SOURCE_FLAGS = {"attention_mfma": ("-fno-honor-nans",)}

_loaded: Dict[Tuple[str, Tuple[Tuple[str, str], ...]], ctypes.CDLL] = {}
_lock = threading.Lock()


class KernelBuildError(RuntimeError):
    """A kernel library is missing and could not be compiled."""


def csrc_dir() -> str:
    return os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")


def build_dir() -> str:
    """Where built libraries live: ``csrc/_build`` if it can be written, else a per-user
    folder under the temporary directory."""
    override = os.environ.get("QWEN25VL_LITE_AMD_BUILD_DIR")
    if override:
        os.makedirs(override, exist_ok=True)
        return override
    path = os.path.join(csrc_dir(), "_build")
    try:
        os.makedirs(path, exist_ok=True)
        probe = os.path.join(path, f".write-{os.getpid()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return path
    except OSError:
        path = os.path.join(tempfile.gettempdir(), f"qwen25vl_lite_amd-build-{os.getuid()}")
        os.makedirs(path, exist_ok=True)
        return path


def _hipcc() -> Optional[str]:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    return None


def _digest(source: str, defines: Mapping[str, object]) -> str:
    h = hashlib.sha1()
    headers = sorted(os.path.join(csrc_dir(), f) for f in os.listdir(csrc_dir()) if f.endswith(".h"))
    for path in (*headers, source):
        with open(path, "rb") as fh:
            h.update(fh.read())
    stem = os.path.splitext(os.path.basename(source))[0]
    h.update(" ".join(HIPCC_FLAGS + SOURCE_FLAGS.get(stem, ())).encode())
    for k in sorted(defines):
        h.update(f"|{k}={defines[k]}".encode())
    return h.hexdigest()[:12]


def library_path(stem: str, defines: Optional[Mapping[str, object]] = None, directory: Optional[str] = None) -> str:
    defines = dict(defines or {})
    source = os.path.join(csrc_dir(), stem + ".hip")
    tag = "".join(f"-{k.lower()}{v}" for k, v in sorted(defines.items()))
    return os.path.join(directory or build_dir(), f"{stem}{tag}-{_digest(source, defines)}.so")


def _find_built(stem: str, defines: Mapping[str, object]) -> Optional[str]:
    """A built library with the right hash, in the tree or in the per-user folder."""
    name = os.path.basename(library_path(stem, defines, directory="/"))
    for directory in (os.environ.get("QWEN25VL_LITE_AMD_BUILD_DIR"), os.path.join(csrc_dir(), "_build"),
                      os.path.join(tempfile.gettempdir(), f"qwen25vl_lite_amd-build-{os.getuid()}")):
        if directory and os.path.isfile(os.path.join(directory, name)):
            return os.path.join(directory, name)
    return None


def build_library(stem: str, defines: Optional[Mapping[str, object]] = None, *, force: bool = False,
                  quiet: bool = False) -> str:
    """Compile ``csrc/<stem>.hip`` (with ``-D`` options) and return the library's path."""
    defines = dict(defines or {})
    source = os.path.join(csrc_dir(), stem + ".hip")
    if not os.path.isfile(source):
        raise KernelBuildError(f"kernel source {source} does not exist")
    if not force:
        found = _find_built(stem, defines)
        if found:
            return found
    out = library_path(stem, defines)
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelBuildError(
            f"the kernel library {os.path.basename(out)} is not built and hipcc was not found; "
            "run __graft_entry__.build() where ROCm is installed")
    tmp = f"{out}.{os.getpid()}.tmp"
    cmd = [hipcc, *HIPCC_FLAGS, *SOURCE_FLAGS.get(stem, ()), f"-I{csrc_dir()}"]
    cmd += [f"-D{k}={v}" for k, v in sorted(defines.items())]
    cmd += [source, "-o", tmp]
    label = stem + "".join(f" {k}={v}" for k, v in sorted(defines.items()))
    if not quiet:
        print(f"[qwen25vl_lite_amd] compiling {label} for {ARCH} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    env = dict(os.environ)
    env.setdefault("TMPDIR", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=tempfile.gettempdir())
    lines = []

    def drain():
        for line in proc.stdout:
            lines.append(line.decode("utf-8", "replace"))

    reader = threading.Thread(target=drain, daemon=True)
    reader.start()
    while True:
        try:
            proc.wait(timeout=10)
            break
        except subprocess.TimeoutExpired:
            if not quiet:
                print(f"[qwen25vl_lite_amd] still compiling {label} ({time.time() - t0:.0f}s)",
                      file=sys.stderr, flush=True)
    reader.join()
    if proc.returncode != 0:
        try:
            os.remove(tmp)
        except OSError:
            pass
        text = "".join(l for l in lines if "not a recognized feature" not in l)
        raise KernelBuildError(f"hipcc failed on {source}:\n{text}")
    os.replace(tmp, out)
    if not quiet:
        print(f"[qwen25vl_lite_amd] built {os.path.basename(out)} in {time.time() - t0:.1f}s",
              file=sys.stderr, flush=True)
    return out


def load_library(stem: str, defines: Optional[Mapping[str, object]] = None) -> ctypes.CDLL:
    """The loaded library of ``csrc/<stem>.hip``; built first if it is not there."""
    defines = dict(defines or {})
    key = (stem, tuple(sorted((k, str(v)) for k, v in defines.items())))
    with _lock:
        lib = _loaded.get(key)
        if lib is None:
            path = build_library(stem, defines)
            lib = ctypes.CDLL(path)
            _loaded[key] = lib
        return lib

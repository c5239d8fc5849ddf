"""Compiling the HIP sources for gfx950 and finding the built libraries.

Every ``<name>.hip`` in this folder becomes one shared library
``lib/<name>-<hash>.so`` beside it, the hash covering the source, the shared headers
and the compiler flags, so a library is never used with a source it was not built
from.  If the package folder cannot be written, the libraries go to a per-user
folder under the system's temporary directory.  ``ensure_built(name)`` compiles on
first need and prints a line now and then while the compiler runs.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from typing import Dict, List

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", f"--offload-arch={ARCH}",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument"]
MODULES = ["elementwise", "gemm_f32", "short_conv", "attention", "attention_fast", "gemv_fused", "gemv_slices", "gemm_rows", "gemm_tiles",
           "sampling"]


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                     "the HIP kernels cannot be built")


def source_path(name: str) -> str:
    return os.path.join(HERE, name + ".hip")


def _digest(name: str) -> str:
    h = hashlib.sha256()
    headers = sorted(f for f in os.listdir(HERE) if f.endswith(".h"))
    for path in [source_path(name)] + [os.path.join(HERE, f) for f in headers]:
        with open(path, "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()[:12]


def _lib_dirs() -> List[str]:
    user = f"celeg_amd-{os.getuid()}"
    return [os.path.join(HERE, "lib"), os.path.join(tempfile.gettempdir(), user, "lib")]


def library_path(name: str):
    """Path of an up-to-date built library of module ``name``, or None."""
    fname = f"{name}-{_digest(name)}.so"
    for d in _lib_dirs():
        path = os.path.join(d, fname)
        if os.path.isfile(path):
            return path
    return None


def _writable_lib_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the built kernels: tried " + ", ".join(_lib_dirs()))


def compile_module(name: str, verbose: bool = True) -> str:
    """Compile ``name``.hip; returns the library's path."""
    if not os.path.isfile(source_path(name)):
        raise BuildError(f"no HIP source {source_path(name)}")
    out_dir = _writable_lib_dir()
    final = os.path.join(out_dir, f"{name}-{_digest(name)}.so")
    tmp = final + f".tmp{os.getpid()}"
    cmd = [_hipcc()] + FLAGS + ["-I", HERE, source_path(name), "-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # the compiler wants a HOME for its caches
    start = time.time()
    if verbose:
        print(f"[celeg_amd] compiling {name}.hip for {ARCH} ...", file=sys.stderr, flush=True)
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env,
                            cwd=out_dir)
    last = start
    while True:
        try:
            output, _ = proc.communicate(timeout=5)
            break
        except subprocess.TimeoutExpired:
            if verbose and time.time() - last >= 10:
                last = time.time()
                print(f"[celeg_amd] ... still compiling {name}.hip ({int(last - start)} s)",
                      file=sys.stderr, flush=True)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"hipcc failed on {name}.hip:\n{output.decode(errors='replace')}")
    os.replace(tmp, final)
    # drop stale builds of this module
    for f in os.listdir(out_dir):
        if f.startswith(name + "-") and f.endswith(".so") and os.path.join(out_dir, f) != final:
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    if verbose:
        print(f"[celeg_amd] built {os.path.basename(final)} in {time.time() - start:.0f} s",
              file=sys.stderr, flush=True)
    return final


def ensure_built(name: str, verbose: bool = True) -> str:
    return library_path(name) or compile_module(name, verbose)


def build_all(force: bool = False, verbose: bool = True) -> Dict[str, str]:
    return {name: (compile_module(name, verbose) if force else ensure_built(name, verbose))
            for name in MODULES}


if __name__ == "__main__":
    for module, path in build_all(force="--force" in sys.argv).items():
        print(module, path)

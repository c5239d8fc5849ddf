"""Compiling the library for gfx950 and finding it.

The kernels (every ``<name>.hip`` in this folder) and the host code (``host/*.cpp``, C++20)
become ONE shared library ``lib/libceleg_amd-<hash>.so``.  Every source is compiled to an
object ``lib/obj/<name>-<hash>.o`` of its own, the hash covering the source, the headers and
the compiler flags, so an object is never used with a source it was not built from and a
change recompiles only what it touches; the library's hash covers its objects.  If the package
folder cannot be written, everything goes to a per-user folder under the system's temporary
directory.  ``ensure_built()`` compiles on first need, several sources at a time, and prints a
line now and then while the compiler runs.
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
from typing import Dict, List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
HOST = os.path.join(HERE, "host")
ARCH = "gfx950"
COMMON_FLAGS = ["-O3", "-fPIC", f"--offload-arch={ARCH}",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                "-Wno-unused-command-line-argument"]
# the first 14 words of a kernel's arguments (what fits the registers a launch can fill) arrive with
# the launch instead of being fetched by every wavefront
KERNEL_FLAGS = ["-std=c++17", "-mllvm", "-amdgpu-kernarg-preload-count=14"] + COMMON_FLAGS
HOST_FLAGS = ["-std=c++20", "-x", "hip", "-Wno-unused-result"] + COMMON_FLAGS
LINK_FLAGS = ["-shared", "-fPIC", f"--offload-arch={ARCH}", "-ldl", "-lpthread"]
# the kernel files, by the name tests and tools know them under
MODULES = ["elementwise", "gemm_f32", "short_conv", "attention", "attention_fast", "gemv_fused", "gemv_slices",
           "gemm_rows", "gemm_tiles", "sampling"]
LIBRARY = "libceleg_amd"
_lock = threading.Lock()


class BuildError(RuntimeError):
    pass


def _hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and os.path.isfile(candidate):
            return candidate
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc); "
                     "the library cannot be built")


def source_path(name: str) -> str:
    return os.path.join(HERE, name + ".hip")


def host_sources() -> List[str]:
    return sorted(os.path.join(HOST, f) for f in os.listdir(HOST) if f.endswith(".cpp"))


def _headers(host: bool) -> List[str]:
    out = [os.path.join(HERE, f) for f in sorted(os.listdir(HERE)) if f.endswith(".h")]
    if host:
        out += [os.path.join(HOST, f) for f in sorted(os.listdir(HOST)) if f.endswith(".hpp")]
        include = os.path.join(HERE, "include")
        out += [os.path.join(include, f) for f in sorted(os.listdir(include)) if f.endswith(".h")]
    return out


def _digest(source: str) -> str:
    host = source.endswith(".cpp")
    h = hashlib.sha256()
    for path in [source] + _headers(host):
        with open(path, "rb") as fh:
            h.update(fh.read())
    h.update(" ".join(HOST_FLAGS if host else KERNEL_FLAGS).encode())
    return h.hexdigest()[:12]


def _sources() -> List[str]:
    return [source_path(m) for m in MODULES] + host_sources()


def _object_name(source: str) -> str:
    stem = os.path.splitext(os.path.basename(source))[0]
    return f"{'host_' if source.endswith('.cpp') else ''}{stem}-{_digest(source)}.o"


def _library_name() -> str:
    h = hashlib.sha256(" ".join(_object_name(s) for s in _sources()).encode())
    h.update(" ".join(LINK_FLAGS).encode())
    return f"{LIBRARY}-{h.hexdigest()[:12]}.so"


def _lib_dirs() -> List[str]:
    user = f"celeg_amd-{os.getuid()}"
    return [os.path.join(HERE, "lib"), os.path.join(tempfile.gettempdir(), user, "lib")]


def library_path(name: Optional[str] = None):
    """Path of an up-to-date built library, or None.  (``name``: a kernel file's name; all of
    them are in the one library.)"""
    fname = _library_name()
    for d in _lib_dirs():
        path = os.path.join(d, fname)
        if os.path.isfile(path):
            return path
    return None


def _writable_lib_dir() -> str:
    for d in _lib_dirs():
        try:
            os.makedirs(os.path.join(d, "obj"), exist_ok=True)
            probe = os.path.join(d, f".probe-{os.getpid()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            return d
        except OSError:
            continue
    raise BuildError("no writable folder for the built library: tried " + ", ".join(_lib_dirs()))


def _run(cmd: List[str], what: str, cwd: str, verbose: bool) -> None:
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # the compiler wants a HOME for its caches
    start = last = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, env=env, cwd=cwd)
    while True:
        try:
            output, _ = proc.communicate(timeout=5)
            break
        except subprocess.TimeoutExpired:
            if verbose and time.time() - last >= 15:
                last = time.time()
                print(f"[celeg_amd] ... still {what} ({int(last - start)} s)", file=sys.stderr, flush=True)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed while {what}:\n{output.decode(errors='replace')}")


def _compile(source: str, out_dir: str, verbose: bool, force: bool) -> str:
    obj = os.path.join(out_dir, "obj", _object_name(source))
    if os.path.isfile(obj) and not force:
        return obj
    host = source.endswith(".cpp")
    name = os.path.basename(source)
    if verbose:
        print(f"[celeg_amd] compiling {name} for {ARCH} ...", file=sys.stderr, flush=True)
    tmp = obj + f".tmp{os.getpid()}-{threading.get_ident()}"
    flags = HOST_FLAGS if host else KERNEL_FLAGS
    start = time.time()
    try:
        _run([_hipcc()] + flags + ["-I", HERE, "-I", HOST, "-c", source, "-o", tmp], f"compiling {name}",
             os.path.join(out_dir, "obj"), verbose)
        os.replace(tmp, obj)
    finally:
        if os.path.exists(tmp):
            os.remove(tmp)
    stem = _object_name(source).rsplit("-", 1)[0]
    for f in os.listdir(os.path.join(out_dir, "obj")):      # drop stale objects of this source
        if f.rsplit("-", 1)[0] == stem and f.endswith(".o") and f != os.path.basename(obj):
            try:
                os.remove(os.path.join(out_dir, "obj", f))
            except OSError:
                pass
    if verbose:
        print(f"[celeg_amd] compiled {name} in {time.time() - start:.0f} s", file=sys.stderr, flush=True)
    return obj


def build(force: bool = False, verbose: bool = True) -> str:
    """Compile what is missing (``force``: everything) and link; returns the library's path."""
    with _lock:
        out_dir = _writable_lib_dir()
        final = os.path.join(out_dir, _library_name())
        if os.path.isfile(final) and not force:
            return final
        sources = _sources()
        workers = max(1, min(8, os.cpu_count() or 1, len(sources)))
        with ThreadPoolExecutor(max_workers=workers) as pool:
            objects = list(pool.map(lambda s: _compile(s, out_dir, verbose, force), sources))
        tmp = final + f".tmp{os.getpid()}"
        if verbose:
            print(f"[celeg_amd] linking {os.path.basename(final)} ...", file=sys.stderr, flush=True)
        try:
            _run([_hipcc()] + objects + LINK_FLAGS + ["-o", tmp], "linking", out_dir, verbose)
            os.replace(tmp, final)
        finally:
            if os.path.exists(tmp):
                os.remove(tmp)
        for f in os.listdir(out_dir):       # drop stale libraries (and those of the one-library-per-kernel layout)
            if f.endswith(".so") and f != os.path.basename(final):
                try:
                    os.remove(os.path.join(out_dir, f))
                except OSError:
                    pass
        return final


SANITIZE_FLAGS = ["-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
                  "-fno-omit-frame-pointer", "-g1"]


def build_sanitized(out_dir: str, verbose: bool = False) -> str:
    """The library with its HOST code under AddressSanitizer and UndefinedBehaviorSanitizer (the
    kernels' objects are the ordinary ones; device code is never instrumented), linked into
    ``out_dir``: what the tests of the host's memory safety run, on the CPU.  Returns its path."""
    with _lock:
        lib_dir = _writable_lib_dir()
        os.makedirs(os.path.join(out_dir, "obj"), exist_ok=True)
        kernels = [_compile(source_path(m), lib_dir, verbose, False) for m in MODULES]

        def sanitized(source: str) -> str:
            obj = os.path.join(out_dir, "obj", "san_" + _object_name(source))
            if not os.path.isfile(obj):
                flags = [f for f in HOST_FLAGS if f != "-O3"] + ["-O1"] + SANITIZE_FLAGS
                _run([_hipcc()] + flags + ["-I", HERE, "-I", HOST, "-c", source, "-o", obj],
                     f"compiling {os.path.basename(source)} with sanitizers", out_dir, verbose)
            return obj
        with ThreadPoolExecutor(max_workers=max(1, min(8, os.cpu_count() or 1))) as pool:
            hosts = list(pool.map(sanitized, host_sources()))
        final = os.path.join(out_dir, LIBRARY + "-sanitized.so")
        _run([_hipcc()] + kernels + hosts + LINK_FLAGS + SANITIZE_FLAGS[:4] + ["-o", final], "linking", out_dir, verbose)
        return final


def compile_module(name: Optional[str] = None, verbose: bool = True) -> str:
    return build(force=False, verbose=verbose)


def ensure_built(name: Optional[str] = None, verbose: bool = True) -> str:
    return library_path() or build(verbose=verbose)


def build_all(force: bool = False, verbose: bool = True) -> Dict[str, str]:
    path = build(force=force, verbose=verbose)
    return {LIBRARY: path}


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))

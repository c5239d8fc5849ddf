"""The library's host code (configuration, weights, page pool, cache manager, scheduler, batch
builder, C interface) compiled with AddressSanitizer and UndefinedBehaviorSanitizer and driven,
without a GPU, by tests/c/host_sanitized.cpp: good and broken model folders, broken
configurations, and hundreds of random calls on the host objects.  A bad access anywhere ends the
program with the sanitizer's report."""
import json
import os
import shutil
import struct
import subprocess

import pytest
import torch

from conftest import TINY_A
from helpers import ROOT


def broken_folders(base, good):
    """Copies of a good model folder, each broken in one way."""
    out = []

    def variant(name):
        folder = os.path.join(base, name)
        shutil.copytree(good, folder)
        out.append(folder)
        return folder, os.path.join(folder, "model.safetensors")

    folder, path = variant("truncated")
    with open(path, "r+b") as fh:
        fh.truncate(os.path.getsize(path) // 2)
    folder, path = variant("tiny")
    with open(path, "wb") as fh:
        fh.write(b"\x01\x02")
    folder, path = variant("header_too_long")
    with open(path, "r+b") as fh:
        fh.write(struct.pack("<Q", 1 << 40))
    folder, path = variant("header_not_json")
    with open(path, "r+b") as fh:
        n = struct.unpack("<Q", fh.read(8))[0]
        fh.write(b"{" * min(n, 64))
    folder, path = variant("offsets_out_of_range")
    with open(path, "rb") as fh:
        n = struct.unpack("<Q", fh.read(8))[0]
        header = json.loads(fh.read(n))
        data = fh.read()
    name = next(k for k in header if k != "__metadata__")
    header[name]["data_offsets"] = [0, len(data) * 4]
    text = json.dumps(header).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)) + text + data)
    folder, path = variant("wrong_shape")
    header[name]["data_offsets"] = [0, 8]
    header[name]["shape"] = [2, 2]
    text = json.dumps(header).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)) + text + data)
    folder, path = variant("config_not_json")
    with open(os.path.join(folder, "config.json"), "w") as fh:
        fh.write("{\"vocab_size\": ")
    folder, path = variant("no_weights")
    os.remove(path)
    folder, path = variant("index_names_missing_shard")
    os.remove(path)
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as fh:
        json.dump({"weight_map": {"model.embed_tokens.weight": "model-00001-of-00002.safetensors"}}, fh)
    return out


def test_host_code_under_sanitizers(tmp_path):
    from celeg_amd.csrc import build
    from celeg_amd.weights import write_random_model
    work = str(tmp_path / "sanitized")
    try:
        library = build.build_sanitized(work)
    except build.BuildError as err:
        if "sanitize" in str(err) or "asan" in str(err).lower():
            pytest.skip(f"the compiler has no sanitizer runtime here: {str(err)[-300:]}")
        raise
    program = os.path.join(work, "host_sanitized")
    subprocess.run([build._hipcc(), "-std=c++17", "-O1", "-g1", "-x", "hip", f"--offload-arch={build.ARCH}"] +
                   build.SANITIZE_FLAGS + ["-I", os.path.join(ROOT, "celeg_amd", "csrc", "include"),
                   os.path.join(ROOT, "tests", "c", "host_sanitized.cpp"), "-o", program,
                   "-L", work, "-l:" + os.path.basename(library), "-Wl,-rpath," + work],
                   check=True, capture_output=True, text=True)
    good = write_random_model(TINY_A, str(tmp_path / "good"), seed=0, dtype=torch.float32, std=0.05)
    broken = broken_folders(str(tmp_path), good)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0:halt_on_error=1",
               UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    proc = subprocess.run([program, good] + broken, capture_output=True, text=True, timeout=600, env=env)
    report = proc.stdout[-3000:] + proc.stderr[-6000:]
    assert "AddressSanitizer" not in proc.stderr and "runtime error:" not in proc.stderr, report
    assert proc.returncode == 0, report
    assert "failures: 0" in proc.stdout
    assert proc.stdout.count("broken ") == len(broken)

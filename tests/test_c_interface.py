"""The C interface from a program written in C (tests/c/drive_engine.c), compiled here against
the library's header and linked to the built library: option defaults and descriptions without
a GPU; submit / step / poll / status on the GPU, its tokens against the plain implementation."""
import json
import os
import shutil
import subprocess

import pytest
import torch

import plain_lfm2 as plain
from helpers import ROOT, WEIGHT_STD, random_tokens


@pytest.fixture(scope="module")
def program(tmp_path_factory):
    from celeg_amd import native
    compiler = shutil.which("gcc") or shutil.which("cc")
    if compiler is None:
        pytest.skip("no C compiler")
    library = native.library_path()
    out = str(tmp_path_factory.mktemp("c_client") / "drive_engine")
    subprocess.run([compiler, "-std=c99", "-Wall", "-Werror", "-O1",
                    "-I", os.path.join(ROOT, "celeg_amd", "csrc", "include"),
                    os.path.join(ROOT, "tests", "c", "drive_engine.c"), "-o", out,
                    "-L", os.path.dirname(library), "-l:" + os.path.basename(library),
                    "-Wl,-rpath," + os.path.dirname(library)], check=True, capture_output=True, text=True)
    return out


def test_defaults_and_descriptions_from_c(program, model_folders):
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    proc = subprocess.run([program, "describe", folder], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0, proc.stderr
    lines = dict(l.split(" ", 1) for l in proc.stdout.splitlines() if " " in l)
    # include/celeg/backend/cuda/concurrency.hpp:18-32; request_types.hpp:16-26; runtime_types.hpp:98-108
    assert lines["engine_defaults"] == "bfloat16 8 2048 1024 16 0"
    assert lines["request_defaults"] == "128 -1 0"
    assert lines["generation_defaults"] == "0.10 50 1.00 1.05 1"
    assert lines["forced_prefix_default"] == "1 0"
    assert "gfx950" in lines["capabilities"] and ("visible" in lines["capabilities"])
    assert "\nchecked\n" in proc.stdout
    assert "config.json" in lines["missing:"]
    assert "must not be null" in lines["refused:"]


@pytest.mark.gpu
@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16")])
def test_submit_step_poll_from_c(program, model_folders, name, dtype):
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, seed=20 + n) for n in (3, 21, 9)]
    proc = subprocess.run([program, "generate", folder, dtype, "10"] + [",".join(map(str, p)) for p in prompts],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr + proc.stdout
    got = {int(l.split(":")[0].split()[1]): [int(t) for t in l.split(":")[1].split()]
           for l in proc.stdout.splitlines() if l.startswith("tokens ")}
    metrics = json.loads([l for l in proc.stdout.splitlines() if l.startswith("metrics ")][0][8:])
    assert metrics["steps"] >= 10 and metrics["failed_steps"] == 0
    for r, prompt in enumerate(prompts):
        seq = list(prompt)
        for _ in range(10):
            seq.append(int(plain.model_logits(cfg, W, seq)[-1].argmax()))
        want = seq[len(prompt):]
        assert len(got[r]) == 10
        if dtype == "float32":
            assert got[r] == want
        else:
            assert got[r][:3] == want[:3]

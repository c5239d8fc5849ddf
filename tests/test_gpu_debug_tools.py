"""The tools for finding a mismatch or a slow phase: the dump of the residual stream after
every layer against the plain implementation's hidden states, and the phase timer."""
import os

import numpy as np
import pytest
import torch

import plain_lfm2 as plain
from helpers import WEIGHT_STD, assert_close_f32, assert_close_bf16, random_tokens

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("D", "bfloat16")])
def test_dump_of_every_layer_equals_the_plain_hidden_state(model_folders, tmp_path, monkeypatch, name, dtype):
    """CELEG_DUMP_HIDDEN: step k writes step<k>_layer<i>.f32, the 32-bit stream after entry i of the
    run order.  A prompt in one step, then two single tokens (the steps that would otherwise be
    replayed from a graph), against the plain implementation layer by layer: the first layer
    that differs is where a fault lies."""
    from celeg_amd.engine import StepEntry, load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    dump = str(tmp_path / "hidden")
    monkeypatch.setenv("CELEG_DUMP_HIDDEN", dump)
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=8, max_requests=2, max_batched_tokens=64)
    monkeypatch.delenv("CELEG_DUMP_HIDDEN")
    tokens = random_tokens(cfg["vocab_size"], 23, seed=3)
    hidden = []
    ref_logits = plain.model_logits(cfg, W, tokens, hidden=hidden)
    n_layers, width = len(hidden), hidden[0].shape[1]
    slot = lm.cache.open()
    assert lm.cache.prepare(slot, 0, 23)
    cuts = [(0, 21), (21, 1), (22, 1)]
    for k, (start, n) in enumerate(cuts):
        got_logits = lm.runner.step([StepEntry(slot, start, tokens[start:start + n], [n - 1])])
        close = assert_close_f32 if dtype == "float32" else assert_close_bf16
        close(got_logits[0], ref_logits[start + n - 1], f"logits of step {k}")
        for i in range(n_layers):
            rows = np.fromfile(os.path.join(dump, f"step{k}_layer{i}.f32"), dtype="<f4").reshape(n, width)
            close(torch.from_numpy(rows), hidden[i][start:start + n], f"step {k}, layer {i}")
    assert sorted(os.listdir(dump)) == sorted(f"step{k}_layer{i}.f32" for k in range(3) for i in range(n_layers))
    assert lm.runner.counters()["graph_replays"] == 0      # a step that is dumped is not replayed
    lm.close()


def test_phase_times_cover_the_step(model_folders):
    from celeg_amd.engine import StepEntry, load_model
    folder = model_folders("D", torch.bfloat16, WEIGHT_STD)
    cfg, _ = plain.load_model_folder(folder)
    kinds = plain.normalise_config(cfg)["layer_types"]
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=8, max_requests=2, max_batched_tokens=64)
    tokens = random_tokens(cfg["vocab_size"], 40, seed=4)
    slot = lm.cache.open()
    assert lm.cache.prepare(slot, 0, 40)
    assert lm.native.phase_times() is None
    plain_run = [lm.runner.step([StepEntry(slot, 0, tokens[:37], [36])])]
    plain_run += [lm.runner.step([StepEntry(slot, p, tokens[p:p + 1], [0])]) for p in (37, 38, 39)]
    assert lm.runner.counters()["graph_replays"] == 3
    lm.cache.close(slot)
    slot = lm.cache.open()
    assert lm.cache.prepare(slot, 0, 40)
    lm.native.time_phases(True)
    timed_run = [lm.runner.step([StepEntry(slot, 0, tokens[:37], [36])])]
    timed_run += [lm.runner.step([StepEntry(slot, p, tokens[p:p + 1], [0])]) for p in (37, 38, 39)]
    times = lm.native.phase_times()
    assert lm.runner.counters()["graph_replays"] == 3      # timed steps run kernel by kernel
    assert times["steps"] == 4 and times["tokens"] == 40
    phases = times["phases"]
    assert list(phases)[:2] == ["step metadata", "embedding"] and list(phases)[-1] == "head"
    assert phases["mixer short_conv"]["calls"] == 4 * kinds.count("conv")
    assert phases["mixer gqa_attention"]["calls"] == 4 * kinds.count("full_attention")
    assert phases["ffn swiglu"]["calls"] == 4 * len(kinds)
    assert all(p["ms"] > 0 for p in phases.values())
    for a, b in zip(plain_run, timed_run):      # the same kernels, timed or not
        assert torch.equal(a, b)
    lm.native.time_phases(False)
    assert lm.native.phase_times() is None
    lm.close()


def test_sync_launches_flag_checks_every_kernel_and_records_no_graph(model_folders, tmp_path):
    """CELEG_SYNC_LAUNCHES=1 (read when the library first launches a kernel, so a process of its own):
    every launch is waited for and checked, which names the kernel behind an asynchronous fault, and no
    step is recorded into or replayed from a graph (the reference's CELEG_DEBUG_SYNC build,
    include/celeg/backend/cuda/utils.cuh:109-116).  The tokens are those of an ordinary run."""
    import json
    import os
    import subprocess
    import sys
    from helpers import ROOT
    folder = model_folders("D", torch.bfloat16, WEIGHT_STD)
    script = tmp_path / "run.py"
    script.write_text(
        "import json, sys\n"
        f"sys.path.insert(0, {ROOT!r})\n"
        "from celeg_amd.engine import Engine\n"
        "from celeg_amd.sampling import GREEDY\n"
        f"e = Engine.from_folder({folder!r}, dtype='bfloat16', max_active_requests=2, n_pages=16, max_batched_tokens=64)\n"
        "out = e.generate([[5, 17, 3, 200, 41], list(range(10, 27))], max_new_tokens=12, generation=GREEDY, eos_token_ids=[])\n"
        "print(json.dumps({'tokens': out, 'replays': e.metrics['graph_replays'], 'captures': e.loaded.runner.counters()['captures']}))\n")
    results = {}
    for flag in ("0", "1"):
        env = dict(os.environ, CELEG_SYNC_LAUNCHES=flag)
        done = subprocess.run([sys.executable, str(script)], env=env, capture_output=True, text=True, timeout=300)
        assert done.returncode == 0, done.stderr[-2000:]
        results[flag] = json.loads(done.stdout.strip().splitlines()[-1])
    assert results["0"]["replays"] > 0 and results["0"]["captures"] > 0
    assert results["1"]["replays"] == 0 and results["1"]["captures"] == 0
    assert results["1"]["tokens"] == results["0"]["tokens"]

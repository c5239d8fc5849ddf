"""``bin/trace_run`` as a user runs it: a child process fed one step at a time, compared
with the plain implementation; whole, tail-decoded, in portions and mixed with reuse of
pages, in both dtypes."""
import pytest
import torch

from helpers import (WEIGHT_STD, TraceClient, assert_close, mixed_schedule, peak_tokens,
                     portions_schedule, tail_decode_schedule, whole_schedule)
from test_engine_modes import plain_logits, requests_of

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "bfloat16"), ("C", "float32")])
def test_trace_run_all_modes_in_one_process(model_folders, tmp_path, name, dtype):
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    reqs = requests_of(name)
    ref = plain_logits(folder, name, storage)
    # one process, four schedules one after the other; request ids made distinct per mode
    all_steps = []
    for tag, make in (("w", whole_schedule), ("t", tail_decode_schedule),
                      ("p", portions_schedule), ("m", mixed_schedule)):
        sub = {f"{tag}{rid}": toks for rid, toks in reqs.items()}
        for s in make(sub):
            s = dict(s, step=len(all_steps))
            all_steps.append(s)
    max_tokens = peak_tokens(all_steps)
    client = TraceClient(folder, dtype, str(tmp_path), max_tokens)
    got = {}
    for s in all_steps:
        logits = client.step(s["step"], s["entries"], s["end"])
        row = 0
        for e in s["entries"]:
            for _ in e["want"]:
                got.setdefault(e["id"], []).append(logits[row])
                row += 1
    assert client.close() == 0
    for rid_tagged, rows in got.items():
        rid = rid_tagged[1:]
        assert_close(torch.stack(rows), ref[rid], dtype, f"{name}/{dtype}/{rid_tagged}")


def test_trace_run_step_without_wanted_logits_and_skipped_request(model_folders, tmp_path):
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    reqs = requests_of("A")
    ref = plain_logits(folder, "A", torch.float32)
    a, b = reqs["r0"], reqs["r1"]
    client = TraceClient(folder, "float32", str(tmp_path), 128)
    assert client.step(0, [{"id": "a", "tokens": a[:10], "want": []}]) is None
    out1 = client.step(1, [{"id": "b", "tokens": b[:5], "want": [4]}])      # a is left out
    out2 = client.step(2, [{"id": "a", "tokens": a[10:12], "want": [1]},
                           {"id": "b", "tokens": b[5:6], "want": [0]}], end=["a", "b"])
    assert client.close() == 0
    assert_close(out1, ref["r1"][4:5], "float32", "b@4")
    assert_close(out2, torch.stack([ref["r0"][11], ref["r1"][5]]), "float32", "a@11,b@5")


def test_trace_run_with_random_weights_and_explicit_pages(tmp_path):
    """``--random-weights CONFIG.json --seed S`` instead of a folder, and a trace that manages pages
    itself: request a reserves all its pages before its first token, request b is refused a
    reservation that the pool cannot give, and ``free`` hands a's pages on to b."""
    import json
    import subprocess
    import sys
    import numpy as np
    import plain_lfm2 as plain
    from conftest import TINY_A
    from celeg_amd.weights import write_random_model
    from helpers import TRACE_RUN, random_tokens
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(TINY_A))
    # the same seed gives the same weights: a tensor's values depend on the seed and its name only
    folder = write_random_model(TINY_A, str(tmp_path / "same"), seed=9, dtype=torch.float32, std=WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    a, b = random_tokens(256, 100, seed=1), random_tokens(256, 90, seed=2)
    base = [sys.executable, TRACE_RUN, "--random-weights", str(cfg_path), "--seed", "9", "--weight-std", str(WEIGHT_STD),
            "--dtype", "float32", "--max-tokens", "128"]

    def run(out, steps):
        return subprocess.run(base + ["--out", str(out)], input="".join(json.dumps(s) + "\n" for s in steps),
                              capture_output=True, text=True, timeout=300)
    steps = [
        {"step": 0, "alloc": [{"id": "a", "tokens": 100}], "entries": [{"id": "a", "tokens": a[:60], "want": [59]}]},
        {"step": 1, "entries": [{"id": "a", "tokens": a[60:], "want": [39]}], "free": ["a"]},
        {"step": 2, "alloc": [{"id": "b", "tokens": 90}], "entries": [{"id": "b", "tokens": b, "want": [0, 89]}], "end": ["b"]},
    ]
    done = run(tmp_path / "ok", steps)
    assert done.returncode == 0 and done.stdout.split() == ["done", "0", "done", "1", "done", "2"], done.stderr
    got = {n: torch.from_numpy(np.fromfile(tmp_path / "ok" / f"{n}.f32", dtype="<f4").reshape(-1, 256).copy()) for n in range(3)}
    ref_a, ref_b = plain.model_logits(cfg, W, a), plain.model_logits(cfg, W, b)
    assert_close(got[0], ref_a[59:60], "float32", "a@59")
    assert_close(got[1], ref_a[99:100], "float32", "a@99")
    assert_close(got[2], ref_b[[0, 89]], "float32", "b@0,89")
    # 112 of the pool's 128 tokens are a's: b's 90 do not fit while a is live
    refused = run(tmp_path / "refused", [steps[0], {"step": 1, "alloc": [{"id": "b", "tokens": 90}], "entries": []}])
    assert refused.returncode != 0 and "out of cache pages" in refused.stderr and refused.stdout.split() == ["done", "0"]

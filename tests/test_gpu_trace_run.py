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

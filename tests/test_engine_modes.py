"""The engine against the plain implementation in every way of cutting and batching:
each request alone and whole; most of it in one step and the last 32 tokens one by
one; portions of changing size down to two tokens; mixed, up to four live requests
with so few pages that they are used again.  On the GPU in 32-bit and bfloat16 (the
real kernels); on the CPU in 32-bit with the test double of the kernels, which checks
the host-side logic (metadata, block tables, state slots) where there is no GPU.
"""
import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY
from helpers import (WEIGHT_STD, EngineDriver, assert_close, mixed_schedule, peak_tokens,
                     portions_schedule, random_tokens, tail_decode_schedule, whole_schedule)

LENGTHS = {"A": [40, 57, 90, 128, 65, 33], "B": [45, 200, 64, 100, 256, 33],
           "C": [70, 33, 150, 97, 48, 260]}
SCHEDULES = {"whole": whole_schedule, "tail32": tail_decode_schedule,
             "portions": portions_schedule, "mixed": mixed_schedule}

_plain_cache = {}


def requests_of(name):
    vocab = TINY[name][0]["vocab_size"]
    return {f"r{i}": random_tokens(vocab, n, seed=100 * TINY[name][1] + i)
            for i, n in enumerate(LENGTHS[name])}


def plain_logits(folder, name, storage):
    key = (name, storage)
    if key not in _plain_cache:
        cfg, W = plain.load_model_folder(folder)
        _plain_cache[key] = {rid: plain.model_logits(cfg, W, toks)
                             for rid, toks in requests_of(name).items()}
    return _plain_cache[key]


def run_mode(model_folders, name, dtype, mode, device, ops=None, subset=None):
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    reqs = requests_of(name)
    if subset:
        reqs = {k: reqs[k] for k in subset}
    steps = SCHEDULES[mode](reqs)
    max_tokens = peak_tokens(steps)
    lm = load_model(folder, dtype=dtype, device=device, page_tokens=16,
                    n_pages=max_tokens // 16, max_requests=4,
                    max_batched_tokens=max(max_tokens, 64), ops=ops)
    got = EngineDriver(lm).run(steps)
    ref = plain_logits(folder, name, storage)
    for rid in reqs:
        assert_close(got[rid], ref[rid], dtype, f"{name}/{dtype}/{mode}/{rid}")
    lm.cache.check()
    assert lm.cache.n_free_slots == 4 and lm.cache.free_pages() == [max_tokens // 16]


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(SCHEDULES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_gpu_engine_matches_plain(model_folders, name, dtype, mode):
    run_mode(model_folders, name, dtype, mode, "cuda:0")


@pytest.mark.parametrize("mode", list(SCHEDULES))
@pytest.mark.parametrize("name", ["A", "B"])
def test_host_logic_with_kernel_double(model_folders, name, mode):
    from cpu_ops import CpuOps
    run_mode(model_folders, name, "float32", mode, "cpu", ops=CpuOps(),
             subset=["r0", "r1", "r5"] if mode != "mixed" else None)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_decode_steps_equal_eager_steps(model_folders, dtype):
    """Decode steps replayed from a captured graph against the same steps run eagerly:
    several replays with other work (portions, other batch sizes) between them, every
    replay checked."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders("B", storage, WEIGHT_STD)
    reqs = requests_of("B")
    steps = mixed_schedule(reqs, max_live=3, seed=4, decode_tail=20)
    out = {}
    for use_graphs in (False, True):
        lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=peak_tokens(steps) // 16,
                        max_requests=4, max_batched_tokens=256)
        lm.runner.use_graphs = use_graphs
        out[use_graphs] = EngineDriver(lm).run(steps)
        if use_graphs:
            assert lm.runner._graphs, "no decode step was replayed from a graph"
    for rid in reqs:
        if dtype == "float32":
            assert torch.equal(out[True][rid], out[False][rid])
        else:
            assert_close(out[True][rid], out[False][rid].double(), dtype, f"graph/{rid}")

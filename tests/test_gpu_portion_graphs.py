"""Steps that are one portion of a prompt, replayed from a recorded graph once their size has
come before: the logits of every portion against the plain implementation, in 32-bit and in
bfloat16, across the context length at which the attention over rows changes its tiles, and
beside steps of other shapes."""
import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY
from helpers import WEIGHT_STD, assert_close, random_tokens

pytestmark = pytest.mark.gpu


def feed_in_portions(lm, tokens, size):
    from celeg_amd.engine import StepEntry
    slot = lm.cache.open()
    rows, pos = [], 0
    while pos < len(tokens):
        n = min(size, len(tokens) - pos)
        assert lm.cache.prepare(slot, pos, n)
        rows.append(lm.runner.step([StepEntry(slot, pos, tokens[pos:pos + n], [n - 1])])[0])
        pos += n
    lm.cache.close(slot)
    return torch.stack(rows)


@pytest.mark.parametrize("name,dtype", [("B", "float32"), ("D", "bfloat16"), ("E", "bfloat16")])
def test_portions_of_a_size_seen_before_are_replayed(model_folders, name, dtype):
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=40, max_requests=2, max_batched_tokens=64)
    tokens = random_tokens(cfg["vocab_size"], 5 * 40 + 13, seed=21)
    ref = plain.model_logits(cfg, W, tokens)
    last_rows = [min(p + 40, len(tokens)) - 1 for p in range(0, len(tokens), 40)]
    got = feed_in_portions(lm, tokens, 40)
    assert_close(got, ref[last_rows], dtype, f"{name}/{dtype}/first request")
    counters = lm.runner.counters()
    assert counters["captures"] == 1 and counters["graph_replays"] == 4     # 40 rows: once eager, four replays; 13 rows: eager
    # another request, other pages (the first one's, given back, in another order), the same recording
    other = random_tokens(cfg["vocab_size"], 3 * 40, seed=22)
    got = feed_in_portions(lm, other, 40)
    assert_close(got, plain.model_logits(cfg, W, other)[[39, 79, 119]], dtype, f"{name}/{dtype}/second request")
    counters = lm.runner.counters()
    assert counters["captures"] == 1 and counters["graph_replays"] == 7
    # portions below the limit are never recorded
    lm.set_knob("portion_graph_min_tokens", 64)
    feed_in_portions(lm, other[:96], 48)
    assert lm.runner.counters()["captures"] == 1
    lm.cache.check()
    lm.close()


def test_portion_graphs_on_both_sides_of_4096_tokens(tmp_path):
    """A prompt of 4,700 tokens in portions of 512: the recording for contexts below 4,096 tokens
    and the one from there on (the attention over rows takes its tiles by the context)."""
    from celeg_amd.engine import load_model
    from celeg_amd.weights import write_random_model
    cfg = dict(TINY["E"][0], max_position_embeddings=8192)
    folder = write_random_model(cfg, str(tmp_path / "long"), seed=5, dtype=torch.bfloat16, std=WEIGHT_STD)
    pcfg, W = plain.load_model_folder(folder)
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=300, max_requests=1, max_batched_tokens=512)
    tokens = random_tokens(cfg["vocab_size"], 4700, seed=23)
    got = feed_in_portions(lm, tokens, 512)
    last_rows = [min(p + 512, len(tokens)) - 1 for p in range(0, len(tokens), 512)]
    ref = plain.model_logits(pcfg, W, tokens)[last_rows]
    assert_close(got, ref, "bfloat16", "portions across 4,096 tokens")
    counters = lm.runner.counters()
    assert counters["captures"] == 2 and counters["graph_replays"] == 8      # 9 portions of 512: one eager
    lm.close()

"""Contexts of thousands of tokens, end to end against the plain implementation.

What only a long context reaches: a second recording of the decode step once a request passes
4,096 tokens (a recording serves contexts up to a bound), the recording of a portion whose rows
end beyond 4,096 tokens (the attention over rows takes other tiles there), parts of 4 rounds of
64 keys in the decode attention over few requests, and both sides of the sizes up to which a
decode-only step's attention prepares and writes the new keys itself.  All knobs are at their
defaults.

The model is tiny (width 128, two query heads on one key/value head of 64, four layers, 300
tokens of vocabulary, 8,192 positions) and its attention is made sharp: the weights of the
query norms are three times their random values, so that a row's attention rests on a handful of
keys somewhere in the context instead of averaging thousands.  A page of 16 keys lost among
4,200 then moves the logits several times further than the bounds allow
(``test_a_lost_page_shows_in_the_logits``, on the CPU, measures that with the plain
implementation); with the weights as drawn it would stay below them.  Only the wanted rows are
compared: the last row of every portion and every decoded token.
"""
import math

import numpy as np
import pytest
import torch

import plain_lfm2 as plain
from helpers import EngineDriver, assert_close, assert_close_bf16, peak_tokens, random_tokens

TINY_F = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 300, "hidden_size": 128, "num_hidden_layers": 4,
    "layer_types": ["conv", "full_attention", "conv", "full_attention"],
    "num_attention_heads": 2, "num_key_value_heads": 1, "head_dim": 64,
    "intermediate_size": 192, "block_auto_adjust_ff_dim": False,
    "rope_theta": 500000.0, "conv_L_cache": 3, "conv_bias": False,
    "tie_word_embeddings": True, "norm_eps": 1e-5, "max_position_embeddings": 8192,
    "bos_token_id": 0, "eos_token_id": 6, "pad_token_id": 1,
}
# four key/value heads, so that a few dozen decoding requests are enough work for the decode
# attention to give every (request, key/value head) a workgroup of its own
TINY_G = dict(TINY_F, num_attention_heads=4, num_key_value_heads=4, hidden_size=256, intermediate_size=320,
              vocab_size=270, conv_L_cache=4, norm_eps=2e-5, rope_theta=100000.0, tie_word_embeddings=False)
SHARP = 3.0
# the spread of the random weights: with 0.03 and the sharpened norms the bfloat16 engine's own
# rounding stays at about half the bounds (measured: 1.6e-2 relative RMS, 1.7e-2 of the largest
# logit at 3,000 tokens) while a lost page is three times beyond them
WEIGHT_STD = 0.03
_made = {}


def sharp_model(tmp_path_factory, cfg, name, storage, sharp=SHARP):
    """Folder, plain configuration and plain weights of ``cfg`` with sharpened query norms."""
    from celeg_amd.weights import SafetensorsFile, write_random_model, write_safetensors
    import os
    key = (name, storage)
    if key not in _made:
        folder = write_random_model(cfg, str(tmp_path_factory.mktemp(f"long_{name}_{str(storage).split('.')[-1]}")),
                                    seed=5, dtype=storage, std=WEIGHT_STD)
        path = os.path.join(folder, "model.safetensors")
        f = SafetensorsFile(path)
        tensors = {n: f.tensor(n).clone() for n in f.names()}
        f.close()
        for n, t in tensors.items():
            if n.endswith("q_layernorm.weight"):
                tensors[n] = (t.float() * sharp).to(t.dtype)
        write_safetensors(path, tensors)
        _made[key] = (folder,) + plain.load_model_folder(folder)
    return _made[key]


def wanted_positions(steps):
    """request id -> the positions whose logits the schedule asks for, in the order they come."""
    seen, out = {}, {}
    for s in steps:
        for e in s["entries"]:
            start = seen.get(e["id"], 0)
            out.setdefault(e["id"], []).extend(start + w for w in e["want"])
            seen[e["id"]] = start + len(e["tokens"])
    return out


def portions_then_tokens(rid, toks, portion, tail, first_step=0):
    """The request's head in portions of ``portion`` tokens (the last row of each wanted), then
    its last ``tail`` tokens one a step."""
    steps, pos, head = [], 0, len(toks) - tail
    while pos < head:
        n = min(portion, head - pos)
        steps.append({"step": first_step + len(steps), "entries": [{"id": rid, "tokens": toks[pos:pos + n], "want": [n - 1]}],
                      "end": []})
        pos += n
    for i in range(head, len(toks)):
        steps.append({"step": first_step + len(steps), "entries": [{"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                      "end": [rid] if i == len(toks) - 1 else []})
    return steps


def compare(got, steps, reqs, cfg, W, dtype, what, only=None):
    positions = wanted_positions(steps)
    for rid, toks in reqs.items():
        if only is not None and rid not in only:
            continue
        ref = plain.model_logits(cfg, W, toks)[positions[rid]]
        assert_close(got[rid], ref, dtype, f"{what}/{dtype}/{rid}")


# --------------------------------------------------------------------------- what the sharp norms are for
def test_a_lost_page_shows_in_the_logits(tmp_path_factory, monkeypatch):
    """The plain implementation with one page of 16 keys hidden from the last 150 rows of 1,500
    tokens: with the query norms as drawn the logits stay inside the bfloat16 bounds (a test at
    that sharpness could not fail), with the sharpened norms they leave them."""
    from celeg_amd.weights import write_random_model
    folder = write_random_model(TINY_F, str(tmp_path_factory.mktemp("lost_page")), seed=5, dtype=torch.float32,
                                std=WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    T, lost = 1500, (752, 768)

    def attention(hide):
        def run(q, k, v, window=None, scale=None):
            q, k, v = q.double(), k.double(), v.double()
            rows, heads, hd = q.shape
            group = heads // k.shape[1]
            mask = torch.ones(rows, rows).tril().bool()
            if hide:
                mask[rows - 150:, lost[0]:lost[1]] = False
            out = torch.zeros(rows, heads, hd, dtype=torch.float64)
            for j in range(heads):
                s = (q[:, j] @ k[:, j // group].T) / math.sqrt(hd)
                out[:, j] = torch.softmax(s.masked_fill(~mask, float("-inf")), dim=1) @ v[:, j // group]
            return out
        return run
    toks = random_tokens(TINY_F["vocab_size"], T, seed=3)
    moved = {}
    for sharp in (1.0, SHARP):
        W2 = {n: (t * sharp if n.endswith("q_layernorm.weight") else t) for n, t in W.items()}
        monkeypatch.setattr(plain, "causal_attention", attention(False))
        ref = plain.model_logits(cfg, W2, toks)[-150:]
        monkeypatch.setattr(plain, "causal_attention", attention(True))
        got = plain.model_logits(cfg, W2, toks)[-150:]
        try:
            assert_close_bf16(got, ref, "a page lost")
            moved[sharp] = False
        except AssertionError:
            moved[sharp] = True
    assert moved == {1.0: False, SHARP: True}


# --------------------------------------------------------------------------- one request
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_request_decodes_and_prefills_across_4096_tokens(tmp_path_factory, dtype):
    """Request a: 4,050 tokens in portions of 512, then 150 tokens one a step, from position 4,050
    to 4,199: the decode step's recording for contexts up to 4,096 hands over to the one for longer
    contexts in the middle.  Request b: 5,120 tokens in portions of 512, the last three of which end
    beyond 4,096 tokens and take the recording of that kind, then 180 tokens one a step."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder, cfg, W = sharp_model(tmp_path_factory, TINY_F, "F", storage)
    reqs = {"a": random_tokens(300, 4200, seed=31), "b": random_tokens(300, 5300, seed=32)}
    steps = portions_then_tokens("a", reqs["a"], 512, 150)
    steps += portions_then_tokens("b", reqs["b"], 512, 180, first_step=len(steps))
    pages = peak_tokens(steps) // 16
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=pages, max_requests=2, max_batched_tokens=512)
    got = EngineDriver(lm).run(steps)
    compare(got, steps, reqs, cfg, W, dtype, "across 4096")
    counters = lm.runner.counters()
    # two recordings of the decode step (contexts up to 4,096 and beyond) and two of the portion of 512
    assert counters["captures"] >= 4, counters
    assert counters["graph_replays"] >= 150 + 180 + 14, counters
    if dtype == "bfloat16":
        assert lm.paths()["attention_decode_fresh"] > 0 and lm.paths()["attention_rows"] > 0
    lm.cache.check()
    assert lm.cache.free_pages() == [pages]
    lm.close()


# --------------------------------------------------------------------------- four live requests
def long_mixed_schedule(requests, max_live=4, seed=0, decode_tail=24):
    """Up to ``max_live`` requests at a time: portions of 64 to 1,024 tokens of some beside the single
    tokens of others, a request now and then left out of a step, new requests admitted as others end."""
    rng = np.random.RandomState(seed)
    waiting, live, steps = list(requests), {}, []
    while waiting or live:
        while waiting and len(live) < max_live:
            live[waiting.pop(0)] = 0
        entries, end = [], []
        for rid in list(live):
            toks, pos = requests[rid], live[rid]
            if len(live) > 1 and rng.rand() < 0.15:
                continue
            if pos >= len(toks) - decode_tail:
                n, want = 1, [0]
            else:
                n = int(min(rng.choice([64, 200, 333, 512, 1024]), len(toks) - decode_tail - pos))
                want = [n - 1]
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": want})
            live[rid] = pos + n
            if pos + n == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_four_live_requests_of_thousands_of_tokens(tmp_path_factory, dtype):
    """Six requests of 3,100 to 6,000 tokens through four slots and a pool of exactly the peak:
    portions beside decoded tokens, pages handed from one request to the next."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder, cfg, W = sharp_model(tmp_path_factory, TINY_F, "F", storage)
    lengths = [3100, 4300, 5200, 6000, 3500, 4700]
    reqs = {f"m{i}": random_tokens(300, n, seed=60 + i) for i, n in enumerate(lengths)}
    steps = long_mixed_schedule(reqs, seed=2)
    assert max(len(s["entries"]) for s in steps) == 4
    assert any(len(s["entries"]) > 1 and {len(e["tokens"]) for e in s["entries"]} >= {1, 512} for s in steps)
    pages = peak_tokens(steps) // 16
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=pages, max_requests=4, max_batched_tokens=4096)
    got = EngineDriver(lm).run(steps)
    compare(got, steps, reqs, cfg, W, dtype, "four live")
    lm.cache.check()
    assert lm.cache.n_free_slots == 4 and lm.cache.free_pages() == [pages]
    lm.close()


# --------------------------------------------------------------------------- who prepares the new keys
def together_schedule(reqs, tail, portion, leave_after, leavers):
    """Every request's head alone (portions of ``portion``), then decode steps that hold all
    requests; after ``leave_after`` of them the ``leavers`` end and the rest decodes on."""
    steps = []
    for rid, toks in reqs.items():
        head = len(toks) - tail
        for pos in range(0, head, portion):
            n = min(portion, head - pos)
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[pos:pos + n], "want": []}], "end": []})
    for k in range(tail):
        ids = [rid for rid in reqs if k < leave_after or rid not in leavers]
        entries = [{"id": rid, "tokens": [reqs[rid][len(reqs[rid]) - tail + k]], "want": [0]} for rid in ids]
        end = [rid for rid in ids if (k == leave_after - 1 and rid in leavers) or k == tail - 1]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


@pytest.mark.gpu
def test_few_requests_beyond_4096_tokens_on_both_sides_of_the_fresh_key_limit(tmp_path_factory):
    """Twenty requests of 4,100 tokens decode together: their contexts are cut into 32 parts of 4
    rounds each, 640 workgroups a key/value head, more than the 512 up to which the attention
    prepares the new keys itself, so the norm-rotate-store kernel runs before it.  Eight requests
    end; the twelve left (a recording for 16) are 512 workgroups and the attention does it all."""
    from celeg_amd.engine import load_model
    folder, cfg, W = sharp_model(tmp_path_factory, TINY_F, "F", torch.bfloat16)
    prompts = [random_tokens(300, 4100 + 3 * i + 12, seed=80 + i) for i in range(4)]
    reqs = {f"q{i}": prompts[i % 4] for i in range(20)}
    leavers = {f"q{i}" for i in range(12, 20)}
    steps = together_schedule(reqs, tail=12, portion=1024, leave_after=6, leavers=leavers)
    pages = peak_tokens(steps) // 16
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=pages, max_requests=20, max_batched_tokens=1024)
    driver = EngineDriver(lm)
    heads = [s for s in steps if len(s["entries"]) == 1]
    driver.run(heads)                      # (a head's last portion may be a single token: such a step counts too)
    start = lm.paths()
    first = [s for s in steps if len(s["entries"]) == 20]
    got = driver.run(first)
    before = lm.paths()
    assert before["attention_decode"] > start["attention_decode"], before
    assert before["attention_decode_fresh"] == start["attention_decode_fresh"], before
    rest = driver.run(steps[len(heads) + len(first):])
    after = lm.paths()
    assert after["attention_decode_fresh"] > before["attention_decode_fresh"], after
    assert after["attention_decode"] == before["attention_decode"], after
    for rid, rows in rest.items():
        got[rid] = torch.cat([got[rid], rows])
    # four different prompts: one request of each, one that left and one that stayed
    compare(got, steps, reqs, cfg, W, "bfloat16", "few beyond 4096", only={"q0", "q1", "q2", "q3", "q13", "q6"})
    assert lm.runner.counters()["graph_replays"] == 12
    lm.cache.check()
    assert lm.cache.free_pages() == [pages]
    lm.close()


@pytest.mark.gpu
def test_many_requests_on_both_sides_of_the_fresh_key_limit(tmp_path_factory):
    """A hundred short requests decode together, a workgroup a request and key/value head: 100
    requests times the 64 rounds that the recording must serve are more than the 4,096 up to which
    that kernel prepares the new keys itself.  Fifty end; the fifty left (a recording for 64) are
    exactly 4,096 and the attention does it all."""
    from celeg_amd.engine import load_model
    # (short contexts: the norms stay as drawn)
    folder, cfg, W = sharp_model(tmp_path_factory, TINY_G, "G", torch.bfloat16, sharp=1.0)
    reqs = {f"w{i}": random_tokens(270, 30 + (11 * i) % 40 + 8, seed=300 + i) for i in range(100)}
    leavers = {f"w{i}" for i in range(0, 100, 2)}
    steps = together_schedule(reqs, tail=8, portion=64, leave_after=4, leavers=leavers)
    pages = sum((len(t) + 15) // 16 for t in reqs.values())
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=pages, max_requests=100, max_batched_tokens=128)
    driver = EngineDriver(lm)
    heads = [s for s in steps if len(s["entries"]) == 1]
    driver.run(heads)                      # (a head's last portion may be a single token: such a step counts too)
    start = lm.paths()
    first = [s for s in steps if len(s["entries"]) == 100]
    got = driver.run(first)
    before = lm.paths()
    assert before["attention_decode"] > start["attention_decode"], before
    assert before["attention_decode_fresh"] == start["attention_decode_fresh"], before
    rest = driver.run(steps[len(heads) + len(first):])
    after = lm.paths()
    assert after["attention_decode_fresh"] > before["attention_decode_fresh"], after
    assert after["attention_decode"] == before["attention_decode"], after
    for rid, rows in rest.items():
        got[rid] = torch.cat([got[rid], rows])
    compare(got, steps, reqs, cfg, W, "bfloat16", "many together", only={f"w{i}" for i in range(0, 100, 9)})
    lm.cache.check()
    assert lm.cache.free_pages() == [pages]
    lm.close()

"""One request at a time through celeg_model_prefill / decode / copy_logits / get_metrics (the
reference's calls of these names, include/celeg/api.h:158-164; semantics src/api/model.cpp:32-77 and
src/backend/cuda/model/prefill.cpp:41-69, execution.cu:168-190: prefill starts a sequence, decode
chooses the next token from the last logits, feeds it and returns it): tokens and logits against
the plain model and sampler."""
import numpy as np
import pytest
import torch

import plain_lfm2 as plain
from helpers import WEIGHT_STD, random_tokens

pytestmark = pytest.mark.gpu


def plain_sequence(cfg, W, prompt, n, temperature, top_k, top_p, penalty, seed, forced=()):
    seq, out = list(prompt), []
    state = seed
    seen = [False] * cfg["vocab_size"]
    for t in seq:
        seen[t] = True
    for i in range(n):
        if i < len(forced):
            token = forced[i]
        else:
            logits = plain.model_logits(cfg, W, seq)[-1].float().tolist()
            token, state = plain.sample(logits, temperature, top_k, top_p, penalty, seen, state)
        seq.append(token); out.append(token); seen[token] = True
    return out, plain.model_logits(cfg, W, seq)[-1]


@pytest.mark.parametrize("name", ["A", "B"])
def test_prefill_decode_and_logits_equal_plain(model_folders, name):
    from celeg_amd.engine import load_model
    folder = model_folders(name, torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    V = cfg["vocab_size"]
    lm = load_model(folder, dtype="float32", max_requests=2, n_pages=8, max_batched_tokens=16)
    m = lm.native
    # greedy; the prompt is longer than a step holds, so it goes in portions
    m.set_generation(temperature=0.0, top_k=1, repetition_penalty=1.0)
    prompt = random_tokens(V, 37, seed=1)
    m.prefill(prompt)
    ref = plain.model_logits(cfg, W, prompt)[-1]
    assert float(np.abs(m.copy_logits() - ref.numpy()).max()) < 1e-4
    got = [m.decode() for _ in range(9)]
    want, last = plain_sequence(cfg, W, prompt, 9, 0.0, 1, 1.0, 1.0, 1)
    assert got == want
    assert float(np.abs(m.copy_logits() - last.numpy()).max()) < 1e-4
    metrics = m.session_metrics()
    assert metrics["prefill_tokens"] == 37 and metrics["decode_tokens"] == 9
    assert metrics["prefill_ms"] > 0 and metrics["decode_ms"] > 0
    # a new prefill starts a new sequence, sampled this time, with forced first tokens; the old
    # one's pages and slot were given back (the pool is too small for both)
    m.set_generation(temperature=0.9, top_k=30, top_p=0.95, repetition_penalty=1.2, seed=5, forced_prefix=(4, 2))
    prompt = random_tokens(V, 100, seed=2)
    m.prefill(prompt)
    got = [m.decode() for _ in range(12)]
    want, last = plain_sequence(cfg, W, prompt, 12, 0.9, 30, 0.95, 1.2, 5, forced=(4, 2))
    assert got == want
    assert float(np.abs(m.copy_logits() - last.numpy()).max()) < 1e-4
    assert m.session_metrics()["decode_tokens"] == 12
    state = lm.cache
    assert state.n_free_slots == 1
    lm.close()


def test_session_calls_refuse_what_cannot_be(model_folders):
    from celeg_amd import native
    from celeg_amd.engine import Engine, load_model
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    lm = load_model(folder, dtype="float32", max_requests=1, n_pages=2, max_batched_tokens=16, max_context=64)
    m = lm.native
    with pytest.raises(Exception, match="decode requires a successful prefill"):
        m.decode()
    with pytest.raises(Exception, match="exceeds max_context"):
        m.prefill([1] * 65)
    with pytest.raises(Exception, match="too few pages"):
        m.prefill([1] * 40)                      # 2 pages of 16 tokens
    with pytest.raises(Exception, match="decode requires a successful prefill"):
        m.decode()
    m.set_generation(temperature=0.0, top_k=1, repetition_penalty=1.0)
    m.prefill([1, 2, 3])                         # the model goes on after the refusals
    assert 0 <= m.decode() < m.logit_width
    with pytest.raises((ValueError, native.NativeArgumentError), match="top_k"):
        m.set_generation(top_k=1000)
    lm.close()
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=1, n_pages=4)
    with pytest.raises(Exception, match="a model of its own"):
        engine.loaded.native.prefill([1, 2, 3])
    engine.close()

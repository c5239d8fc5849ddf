"""Forced first tokens of a request (the reference's ForcedTokenPrefix,
include/celeg/model/runtime_types.hpp:93-104): while the prefix lasts the sampler gives out its
tokens instead of choosing one and leaves the request's generator alone
(src/backend/cpu/sampler.cpp:31-34); the CUDA sampler copies the token in and marks it as seen
(src/backend/cuda/model/sampler.cu:44-54).  The plain sampler below does the same."""
import pytest
import torch

import plain_lfm2 as plain
from helpers import WEIGHT_STD, random_tokens

pytestmark = pytest.mark.gpu


def plain_generate(cfg, W, prompt, n, generation, eos=()):
    seq, out = list(prompt), []
    state = generation.seed
    seen = [False] * cfg["vocab_size"]
    for t in seq:
        seen[t] = True
    for i in range(n):
        if i < len(generation.forced_prefix):
            token = generation.forced_prefix[i]               # no draw: the state stays
        else:
            logits = plain.model_logits(cfg, W, seq)[-1].float().tolist()
            token, state = plain.sample(logits, generation.temperature, generation.top_k, generation.top_p,
                                        generation.repetition_penalty, seen, state)
        seq.append(token); out.append(token); seen[token] = True
        if token in eos:
            break
    return out


def test_forced_tokens_come_first_and_the_rest_is_sampled_as_without_them(model_folders):
    """Requests with forced prefixes of different lengths beside one without, sampled with a
    penalty for seen tokens (the forced ones count as seen): each equals the plain model and
    sampler; and what follows a prefix equals what a request gets whose prompt ends with the
    prefix (the generator was not advanced, the same tokens are seen)."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GenerationConfig
    folder = model_folders("B", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    V = cfg["vocab_size"]
    prompts = [random_tokens(V, n, seed=300 + n) for n in (5, 40, 70, 9)]
    forced = [(), (3, V - 1, 3), tuple(random_tokens(V, 7, seed=9)), (11,)]
    gens = [GenerationConfig(temperature=0.8, top_k=40, top_p=0.9, repetition_penalty=1.3, seed=7 + i, forced_prefix=f)
            for i, f in enumerate(forced)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=4, n_pages=40,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    outs = engine.generate(prompts, max_new_tokens=12, generations=gens, eos_token_ids=[])
    for prompt, gen, out in zip(prompts, gens, outs):
        assert out[:len(gen.forced_prefix)] == list(gen.forced_prefix)
        assert out == plain_generate(cfg, W, prompt, 12, gen)
    bare = [GenerationConfig(temperature=0.8, top_k=40, top_p=0.9, repetition_penalty=1.3, seed=7 + i) for i in range(4)]
    longer = engine.generate([p + list(f) for p, f in zip(prompts, forced)], max_new_tokens=12, generations=bare,
                             eos_token_ids=[])
    for f, out, other in zip(forced, outs, longer):
        assert out[len(f):] == other[:12 - len(f)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_requests_with_forced_tokens(model_folders, dtype):
    """Greedy rows take the kernel for rows that are all greedy; a row with a forced token in the
    step sends the step to the general kernel.  An end token inside the prefix ends the request."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GenerationConfig
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders("A", storage, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    V = cfg["vocab_size"]
    prompts = [random_tokens(V, n, seed=400 + n) for n in (20, 33, 6)]
    forced = [(5, 6), (), (9, 2, 4, 8)]
    gens = [GenerationConfig(temperature=0.0, top_k=1, top_p=1.0, repetition_penalty=1.0, seed=1, forced_prefix=f)
            for f in forced]
    engine = Engine.from_folder(folder, dtype=dtype, max_active_requests=3, n_pages=30, max_batched_tokens=64,
                                prefill_chunk_tokens=32)
    outs = engine.generate(prompts, max_new_tokens=8, generations=gens, eos_token_ids=[4])
    assert outs[2] == [9, 2, 4]                                 # the end token came from the prefix
    for f, out in zip(forced, outs):
        assert out[:len(f)] == list(f)[:len(out)]
    if dtype == "float32":
        for prompt, gen, out in zip(prompts, gens, outs):
            assert out == plain_generate(cfg, W, prompt, 8, gen, eos=(4,))


def test_a_request_that_is_put_back_goes_on_where_its_prefix_was(model_folders):
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GenerationConfig
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    V = cfg["vocab_size"]
    prompts = [random_tokens(V, 30, seed=90 + i) for i in range(3)]
    gens = [GenerationConfig(temperature=0.0, top_k=1, top_p=1.0, repetition_penalty=1.0, seed=1,
                             forced_prefix=tuple(random_tokens(V, 25, seed=50 + i))) for i in range(3)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=3, n_pages=6,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    outs = engine.generate(prompts, max_new_tokens=40, generations=gens, eos_token_ids=[])
    assert engine.metrics["scheduler"]["preemptions"] > 0
    for prompt, gen, out in zip(prompts, gens, outs):
        assert out == plain_generate(cfg, W, prompt, 40, gen)


def test_forced_tokens_outside_the_vocabulary_are_refused(model_folders):
    from celeg_amd.engine import Engine, RequestOptions
    from celeg_amd.sampling import GenerationConfig
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, _ = plain.load_model_folder(folder)
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=2, n_pages=8)
    for bad in ((cfg["vocab_size"],), (1, -2)):
        with pytest.raises(ValueError):
            engine.submit([1, 2, 3], RequestOptions(max_new_tokens=4, generation=GenerationConfig(forced_prefix=bad)))
    assert not engine.has_work()

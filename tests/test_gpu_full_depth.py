"""The configuration that bench.py measures (LFM2-350M shape: 16 layers, width 1,024, 65,536
tokens of vocabulary, random weights of the benchmark's own spread), whole depth, in bfloat16:
the logits of a prompt fed whole, in portions and with its last tokens decoded one by one, and
greedy tokens through the engine, against the plain implementation."""
import sys

import pytest
import torch

import plain_lfm2 as plain
from helpers import ROOT, EngineDriver, assert_close_bf16, portions_schedule, random_tokens, tail_decode_schedule

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def benchmark_model(tmp_path_factory):
    sys.path.insert(0, ROOT)
    from bench import SHAPES
    from celeg_amd.weights import write_random_model
    cfg = dict(SHAPES["350m"][0])
    folder = write_random_model(cfg, str(tmp_path_factory.mktemp("bench_350m")), seed=0, dtype=torch.bfloat16, std=0.02)
    pcfg, W = plain.load_model_folder(folder)
    return folder, pcfg, W


def test_logits_at_the_benchmarks_configuration(benchmark_model):
    from celeg_amd.engine import load_model
    folder, cfg, W = benchmark_model
    assert len(plain.normalise_config(cfg)["layer_types"]) == 16 and cfg["vocab_size"] == 65536
    reqs = {"a": random_tokens(cfg["vocab_size"], 100, seed=1), "b": random_tokens(cfg["vocab_size"], 61, seed=2)}
    ref = {rid: plain.model_logits(cfg, W, toks).float() for rid, toks in reqs.items()}
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=16, max_requests=2, max_context=256,
                    max_batched_tokens=128)
    for mode, schedule in (("tail32", tail_decode_schedule), ("portions", portions_schedule)):
        got = EngineDriver(lm).run(schedule(reqs))
        for rid in reqs:
            assert_close_bf16(got[rid], ref[rid], f"benchmark configuration/{mode}/{rid}")
    assert lm.runner.counters()["graph_replays"] >= 32       # the single tokens went through recorded steps
    lm.close()


def test_logits_at_the_benchmarks_context(benchmark_model):
    """What bench.py times, with its logits checked: prompts of 2,048 tokens fed in one step each (the
    tiled products, the attention over 2,048 rows), then eight requests decoding together from position
    2,048 on (the recorded step of a batch of 8, keys cut into 33 parts and joined).  Two different
    prompts, four requests each; the last row of every prompt and every decoded token against the plain
    implementation."""
    from celeg_amd.engine import load_model
    folder, cfg, W = benchmark_model
    prompts = [random_tokens(cfg["vocab_size"], 2048 + 8, seed=21 + i) for i in range(2)]
    reqs = {f"b{i}": prompts[i % 2] for i in range(8)}
    steps = [{"step": i, "entries": [{"id": rid, "tokens": toks[:2048], "want": [2047]}], "end": []}
             for i, (rid, toks) in enumerate(reqs.items())]
    for k in range(8):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": [toks[2048 + k]], "want": [0]} for rid, toks in reqs.items()],
                      "end": list(reqs) if k == 7 else []})
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=8 * 129, max_requests=8, max_context=4096,
                    max_batched_tokens=2048)
    got = EngineDriver(lm).run(steps)
    assert lm.runner.counters()["graph_replays"] >= 8
    paths = lm.paths()
    assert paths["tiled"] > 0 and paths["tiled_qkv"] > 0 and paths["attention_rows"] > 0 and paths["attention_decode_fresh"] > 0, paths
    ref = [plain.model_logits(cfg, W, toks)[2047:].float() for toks in prompts]
    for i, rid in enumerate(reqs):
        assert_close_bf16(got[rid], ref[i % 2], f"benchmark context/{rid}")
    lm.close()


def test_32bit_logits_at_the_benchmarks_depth(benchmark_model):
    """All 16 layers in true 32-bit (the same folder, its bfloat16 weights widened exactly):
    two short requests, most in one step and the last tokens one by one, then in portions,
    against the plain implementation at the 32-bit bound."""
    from celeg_amd.engine import load_model
    from helpers import assert_close_f32
    folder, cfg, W = benchmark_model
    reqs = {"a": random_tokens(cfg["vocab_size"], 64, seed=5), "b": random_tokens(cfg["vocab_size"], 41, seed=6)}
    ref = {rid: plain.model_logits(cfg, W, toks) for rid, toks in reqs.items()}
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=8, max_requests=2, max_context=128,
                    max_batched_tokens=64)
    for mode, schedule in (("tail", lambda r: tail_decode_schedule(r, tail=12)), ("portions", portions_schedule)):
        got = EngineDriver(lm).run(schedule(reqs))
        for rid in reqs:
            assert_close_f32(got[rid], ref[rid], f"benchmark depth, 32-bit/{mode}/{rid}")
    lm.close()


def test_greedy_tokens_at_the_benchmarks_configuration(benchmark_model):
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    folder, cfg, W = benchmark_model
    prompts = [random_tokens(cfg["vocab_size"], n, seed=10 + n) for n in (40, 9)]
    engine = Engine.from_folder(folder, dtype="bfloat16", max_active_requests=2, n_pages=16, context=256,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    outs = engine.generate(prompts, max_new_tokens=10, generation=GREEDY, eos_token_ids=[])
    for prompt, out in zip(prompts, outs):
        seq, exact = list(prompt), 0
        for token in out:
            logits = plain.model_logits(cfg, W, seq)[-1]
            assert float(logits[token]) >= float(logits.max()) - 4e-2 * float(logits.abs().max())
            exact += int(token == int(logits.argmax()))
            seq.append(token)
        assert len(out) == 10 and exact >= 8
    assert engine.metrics["graph_replays"] > 0

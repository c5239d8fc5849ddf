"""Generation through the Python entry point and the command line, and the sampling
kernels alone, against the plain implementation."""
import json
import os
import subprocess
import sys

import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY
from helpers import ROOT, WEIGHT_STD, random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def plain_generate(cfg, W, prompt, n, generation=None, eos=()):
    """Greedy (or sampled) continuation with the plain model and the plain sampler."""
    seq = list(prompt)
    out = []
    state = generation.seed if generation else 1
    seen = [False] * cfg["vocab_size"]
    for t in seq:
        seen[t] = True
    for _ in range(n):
        logits = plain.model_logits(cfg, W, seq)[-1].float().tolist()
        if generation is None:
            token, state = plain.sample(logits, 0.0, 1, 1.0, 1.0, seen, state)
        else:
            token, state = plain.sample(logits, generation.temperature, generation.top_k,
                                        generation.top_p, generation.repetition_penalty, seen, state)
        seq.append(token); out.append(token); seen[token] = True
        if token in eos:
            break
    return out


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("B", "float32"), ("A", "bfloat16"),
                                        ("D", "float32"), ("D", "bfloat16")])
def test_greedy_generation_through_the_entry_point(model_folders, name, dtype):
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    vocab = cfg["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=50 + n) for n in (5, 17, 33)]
    engine = Engine.from_folder(folder, dtype=dtype, max_active_requests=3, n_pages=12,
                                max_batched_tokens=32, prefill_chunk_tokens=8)
    outs = engine.generate(prompts, max_new_tokens=16, generation=GREEDY, eos_token_ids=[])
    for prompt, out in zip(prompts, outs):
        want = plain_generate(cfg, W, prompt, 16)
        if dtype == "float32":
            assert out == want
        else:
            # rounding may flip a near-tie, after which the sequences part: every token is held
            # against the plain model run on the engine's own tokens so far, and must be its
            # most likely token or lie within bfloat16's rounding of it (the bound of the
            # logits' comparison, 4e-2 of the largest logit); most are the most likely one
            assert len(out) == 16
            seq, exact = list(prompt), 0
            for token in out:
                logits = plain.model_logits(cfg, W, seq)[-1]
                best = float(logits.max())
                assert float(logits[token]) >= best - 4e-2 * float(logits.abs().max()), \
                    f"token {token} at position {len(seq)}: logit {float(logits[token]):.4f}, best {best:.4f}"
                exact += int(token == int(logits.argmax()))
                seq.append(token)
            assert exact >= 14 and out[:4] == want[:4]
    assert engine.loaded.cache.free_pages() == [12] and engine.loaded.cache.n_free_slots == 3
    # the same requests one at a time give the same tokens: no dependence on batch mates
    alone = [engine.generate([p], max_new_tokens=16, generation=GREEDY, eos_token_ids=[])[0]
             for p in prompts]
    if dtype == "float32":
        assert alone == outs


@pytest.mark.parametrize("name", ["B", "D"])
def test_generation_under_a_steady_load_of_portions_beside_decoding(model_folders, name):
    """A steady load through the entry point: ten requests of equal length under a budget that
    holds one portion and the decoding requests, a granule for the portions the budget cuts.
    Most steps carry a portion of one prompt beside the single tokens of the decoding requests;
    every request's tokens equal the plain implementation's greedy ones."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    folder = model_folders(name, torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    vocab = cfg["vocab_size"]
    prompts = [random_tokens(vocab, 96, seed=300 + i) for i in range(10)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=4, n_pages=64,
                                max_batched_tokens=52, prefill_chunk_tokens=48, portion_granule=8)
    outs = engine.generate(prompts, max_new_tokens=12, generation=GREEDY, eos_token_ids=[])
    assert engine.metrics["scheduler"]["mixed_steps"] > 10, "no step held portions beside single tokens"
    for prompt, out in zip(prompts, outs):
        assert out == plain_generate(cfg, W, prompt, 12)
    assert engine.loaded.cache.free_pages() == [64] and engine.loaded.cache.n_free_slots == 4


def test_sampled_generation_mixed_batch_equals_plain_sampler(model_folders):
    """Tiny B's workload: prompts 1, 9, 64, 100, 200 in portions of 32 beside decoding,
    temperature 0.8, seed 7; every request's tokens equal the plain model + plain sampler,
    whatever its batch mates (one generator per request)."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GenerationConfig
    folder = model_folders("B", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    gen = GenerationConfig(temperature=0.8, top_k=40, top_p=0.9, repetition_penalty=1.3, seed=7)
    prompts = [random_tokens(cfg["vocab_size"], n, seed=70 + n) for n in (1, 9, 64, 100, 200)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=4, n_pages=40,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    outs = engine.generate(prompts, max_new_tokens=6, generation=gen, eos_token_ids=[])
    for prompt, out in zip(prompts, outs):
        assert out == plain_generate(cfg, W, prompt, 6, generation=gen)


def test_generation_with_few_pages_preempts_and_keeps_the_tokens(model_folders):
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], 30, seed=90 + i) for i in range(3)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=3, n_pages=6,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    outs = engine.generate(prompts, max_new_tokens=40, generation=GREEDY, eos_token_ids=[])
    assert engine.metrics["scheduler"]["preemptions"] > 0
    for prompt, out in zip(prompts, outs):
        assert out == plain_generate(cfg, W, prompt, 40)


def test_command_line(model_folders, tmp_path):
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompt = random_tokens(cfg["vocab_size"], 12, seed=5)
    dump = str(tmp_path / "logits.f32")
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "celeg-run"), "--model", folder, "--dtype",
         "float32", "--prompt", ",".join(map(str, prompt)), "--max-new-tokens", "8",
         "--repetition-penalty", "1.0", "--runtime-tokens", "--dump-logits", dump, "--print-top", "2"],
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    line = [l for l in proc.stdout.splitlines() if l.startswith("CELEG_GENERATED_TOKEN_IDS=")][0]
    got = json.loads(line.split("=", 1)[1])
    want = plain_generate(cfg, W, prompt, 8, eos=[7])
    assert got == want
    import numpy as np
    logits = np.fromfile(dump, dtype="<f4")
    ref = plain.model_logits(cfg, W, prompt)[-1]
    assert logits.shape == (cfg["vocab_size"],)
    assert float(np.abs(logits - ref.numpy()).max()) < 1e-4
    assert "top[0] token=" in proc.stderr
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "celeg-run"), "--model", folder,
                          "--prompt", "1 2 3", "--max-new-tokens", "500"],
                         capture_output=True, text=True, timeout=300)
    assert bad.returncode == 1 and "prompt plus output exceeds --context" in bad.stderr


@pytest.mark.parametrize("flags", [["--attention-mode", "single"], ["--attention-mode", "segmented"],
                                   ["--attention-mode", "segmented", "--attention-chunk-tokens", "256"],
                                   ["--attention-chunk-tokens", "1024", "--no-cuda-graph"]])
def test_command_line_attention_modes(model_folders, flags):
    """--attention-mode / --attention-chunk-tokens (bfloat16, heads of 64: the kernels they choose
    between): every token is the plain model's most likely one given the tokens so far, or within
    bfloat16's rounding of it."""
    folder = model_folders("D", torch.bfloat16, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompt = random_tokens(cfg["vocab_size"], 70, seed=8)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "celeg-run"), "--model", folder, "--prompt",
         ",".join(map(str, prompt)), "--max-new-tokens", "10", "--repetition-penalty", "1.0", "--runtime-tokens"] + flags,
        capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    line = [l for l in proc.stdout.splitlines() if l.startswith("CELEG_GENERATED_TOKEN_IDS=")][0]
    out = json.loads(line.split("=", 1)[1])
    assert 1 <= len(out) <= 10
    seq, exact = list(prompt), 0
    for token in out:
        logits = plain.model_logits(cfg, W, seq)[-1]
        assert float(logits[token]) >= float(logits.max()) - 4e-2 * float(logits.abs().max())
        exact += int(token == int(logits.argmax()))
        seq.append(token)
    assert exact >= len(out) - 2
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "celeg-run"), "--model", folder, "--prompt", "1 2 3",
                          "--attention-chunk-tokens", "100"], capture_output=True, text=True, timeout=300)
    assert bad.returncode == 2 and "must be 64, 256 or 1024" in bad.stderr


# ---------------------------------------------------------------- the sampling kernels alone
@pytest.fixture(scope="module")
def ops():
    from kernel_ops import HipOps
    return HipOps(DEV)


def sample_with_draw(logits, temperature, top_k, top_p, penalty, seen, u):
    """The plain sampler with the draw in [0, 1) given instead of taken from its generator."""
    generator = plain.random_unit
    plain.random_unit = lambda state: (state, u)
    try:
        return plain.sample(logits, temperature, top_k, top_p, penalty, seen, 1)[0]
    finally:
        plain.random_unit = generator


def parts_of(logits, cols):
    """What an output head leaves beside its logits: the best (logit, index) of every ``cols`` columns,
    [rows, parts], packed as the kernels pack it (the logit's ordered bits above the inverted index)."""
    import numpy as np
    x = (logits.float() + 0.0).numpy()
    bits = x.view(np.uint32).astype(np.uint64)
    key = np.where(bits & 0x80000000, ~bits & 0xffffffff, bits | 0x80000000)
    R, V = x.shape
    packed = (key << np.uint64(32)) | (np.uint64(0xffffffff) - np.arange(V, dtype=np.uint64))[None, :]
    parts = (V + cols - 1) // cols
    padded = np.zeros((R, parts * cols), dtype=np.uint64)
    padded[:, :V] = packed
    best = padded.reshape(R, parts, cols).max(axis=2).copy()
    return torch.from_numpy(best.view(np.int64)).to(DEV)


def run_sample(ops, logits, rows, all_greedy=False, part_cols=0):
    """rows: list of (temperature, top_k, top_p, penalty, u, seen list or None); part_cols: the kernel also
    gets what an output head would have left beside these logits, a part every part_cols columns"""
    R, V = logits.shape
    f = torch.tensor([[t, p, pen, u] for t, k, p, pen, u, s in rows], dtype=torch.float32)
    seen = torch.zeros(R, V, dtype=torch.uint8)
    i = []
    for r, (t, k, p, pen, u, s) in enumerate(rows):
        if s is not None:
            seen[r, torch.tensor(s, dtype=torch.long)] = 1
        i.append([k, r if s is not None else -1, -1])
    out = torch.empty(R, dtype=torch.int32, device=DEV)
    best = parts_of(logits, part_cols) if part_cols else None
    ops.sample(logits.to(DEV), f.reshape(-1).to(DEV), torch.tensor(i, dtype=torch.int32).reshape(-1).to(DEV),
               seen.to(DEV), out, all_greedy=all_greedy, row_best=best, row_best_parts=best.shape[1] if part_cols else 0,
               row_best_cols=part_cols, penalised=any(s is not None and pen > 1 for t, k, p, pen, u, s in rows))
    return out.tolist()


def test_sampling_kernel_reference_vectors(ops):
    # tests/cpu_sampler_test.cpp:8-43; tests/cuda/sampling_tests.cu:16-60
    logits = torch.tensor([[1., 4., 2., 3.], [2., 5., 5., 1.], [5., 4., 3., 2.], [1., 4., 2., 3.]])
    got = run_sample(ops, logits, [(0.0, 1, 1.0, 1.0, 0.0, None), (0.0, 1, 1.0, 1.0, 0.0, None),
                                   (0.0, 50, 1.0, 2.0, 0.0, [0]), (0.7, 1, 1.0, 1.0, 0.3, None)])
    assert got == [1, 1, 1, 1]
    for u in (0.01, 0.3, 0.6, 0.99):
        assert run_sample(ops, logits[:1], [(1.5, 2, 1.0, 1.0, u, None)])[0] in (1, 3)
        assert run_sample(ops, logits[:1], [(1.5, 4, 0.01, 1.0, u, None)])[0] == 1


@pytest.mark.parametrize("vocab", [331, 4096, 65536, 70001])
def test_sampling_kernel_equals_plain_sampler(ops, vocab):
    g = torch.Generator().manual_seed(vocab)
    R = 6
    logits = torch.randn(R, vocab, generator=g) * 3
    logits[1, 100:140] = logits[1, 7]            # many ties at one value, also at the threshold
    logits[2] = torch.round(logits[2])           # heavy ties everywhere
    seen = [torch.randint(0, vocab, (50,), generator=g).tolist() for _ in range(R)]
    rows = [(0.8, 40, 0.9, 1.3, 0.37, seen[0]), (1.0, 128, 1.0, 1.0, 0.81, None),
            (0.5, 17, 0.5, 1.0, 0.999, None), (0.0, 50, 1.0, 1.7, 0.0, seen[3]),
            (2.0, 128, 0.95, 1.1, 0.05, seen[4]), (1.3, 2, 1.0, 1.0, 0.5, None)]
    got = run_sample(ops, logits, rows)
    want = []
    for r, (t, k, p, pen, u, s) in enumerate(rows):
        flags = [False] * vocab
        for tok in (s or []):
            flags[tok] = True
        want.append(sample_with_draw(logits[r].tolist(), t, k, p, pen, flags, u))
        assert got[r] == want[r], f"row {r}"
    # the same from what an output head leaves beside the logits (the best of every 16, 64 or 7 columns):
    # the candidates are then looked for in the parts whose best logit is large enough, not in the whole row
    for part_cols in (16, 64, 7):
        assert run_sample(ops, logits, rows, part_cols=part_cols) == want, part_cols


@pytest.mark.parametrize("vocab", [4096, 65536])
def test_sampling_from_the_heads_parts_when_penalties_reorder_the_top(ops, vocab):
    """The parts hold the best logit of their columns before any penalty.  Here the 300 largest logits of a
    row have all been seen and a penalty of 3 throws them far down, so the tokens that win come from parts
    whose best logit was nowhere near the top; in another row all logits are equal (nothing bounds anything:
    the kernel reads the row after all); in a third the maximum of every part is the same value."""
    g = torch.Generator().manual_seed(vocab + 7)
    R = 4
    logits = torch.randn(R, vocab, generator=g) * 2
    top = torch.topk(logits[0], 300).indices.tolist()
    logits[1] = 0.5
    logits[2, ::16] = 9.0
    logits[3] = -logits[3].abs() - 1.0              # all negative: a penalty makes seen ones smaller still
    seen3 = torch.topk(logits[3], 100).indices.tolist()
    rows = [(0.7, 50, 0.95, 3.0, 0.42, top), (1.0, 50, 1.0, 1.0, 0.77, None), (0.9, 128, 0.9, 1.2, 0.13, list(range(0, 4096, 32))),
            (0.5, 20, 1.0, 1.5, 0.6, seen3)]
    want = []
    for r, (t, k, p, pen, u, s) in enumerate(rows):
        flags = [False] * vocab
        for tok in (s or []):
            flags[tok] = True
        want.append(sample_with_draw(logits[r].tolist(), t, k, p, pen, flags, u))
    assert want[0] not in top[:50]
    assert run_sample(ops, logits, rows) == want
    for part_cols in (16, 64):
        assert run_sample(ops, logits, rows, part_cols=part_cols) == want, part_cols


@pytest.mark.parametrize("vocab", [5, 331, 4100, 65536, 70001])
def test_arg_max_lowest_index_wins_with_and_without_penalty(ops, vocab):
    g = torch.Generator().manual_seed(vocab + 1)
    R = 7
    logits = torch.randn(R, vocab, generator=g)
    top = float(logits.max()) + 1.0
    for r in range(R):     # the maximum several times, first at a place that differs per row
        first = (r * 977 + vocab // 3) % vocab
        logits[r, first] = top
        logits[r, (first + vocab // 2) % vocab] = top
        logits[r, vocab - 1] = top
    rows, want = [], []
    for r in range(R):
        ties = sorted({(r * 977 + vocab // 3) % vocab, ((r * 977 + vocab // 3) % vocab + vocab // 2) % vocab, vocab - 1})
        if r % 2:    # the first maximum was seen and is pushed down by the penalty
            rows.append((0.0, 1, 1.0, 1.5, 0.0, [ties[0]]))
            want.append(ties[1] if len(ties) > 1 else ties[0])
        else:
            rows.append((0.0, 1, 1.0, 1.0, 0.0, None))
            want.append(ties[0])
    assert run_sample(ops, logits, rows) == want
    # the same by the kernel that cuts every row into parts over many workgroups, twice (it
    # leaves its counters ready for the next launch), and with a zero of either sign as maximum
    assert run_sample(ops, logits, rows, all_greedy=True) == want
    assert run_sample(ops, logits, rows, all_greedy=True) == want
    zeros = -torch.rand(2, vocab) - 0.5
    zeros[0, vocab - 1] = 0.0
    zeros[0, vocab // 2] = -0.0
    zeros[1, vocab // 2] = 0.0
    zeros[1, 0] = -0.0
    plain_rows = [(0.0, 1, 1.0, 1.0, 0.0, None)] * 2
    assert run_sample(ops, zeros, plain_rows, all_greedy=True) == run_sample(ops, zeros, plain_rows) \
        == [min(vocab // 2, vocab - 1), 0]


def test_mark_seen(ops):
    seen = torch.zeros(3, 100, dtype=torch.uint8, device=DEV)
    toks = torch.tensor([5, 99, 5, 17], dtype=torch.int32, device=DEV)
    slots = torch.tensor([0, 2, 2, 3], dtype=torch.int32, device=DEV)   # slot 3 is outside: ignored
    ops.mark_seen(seen, toks, slots, 4)
    assert seen.sum().item() == 3 and seen[0, 5] == 1 and seen[2, 99] == 1 and seen[2, 5] == 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_ahead_of_their_tokens_give_the_same_tokens(model_folders, dtype):
    """Decode steps that take their input token on the device from what the previous step
    sampled, launched before the host has read it (the loop that the benchmark times), against
    steps the host feeds one by one."""
    from celeg_amd.engine import Engine, RequestStatus
    from celeg_amd.engine.benchmark import DecodeBench
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders("B", storage, 0.05)
    runs = {}
    for ahead in (False, True):
        engine = Engine.from_folder(folder, dtype=dtype, page_tokens=16, n_pages=64, max_active_requests=4,
                                    max_batched_tokens=64, prefill_chunk_tokens=16, run_ahead=ahead)
        bench = DecodeBench(engine, 3, 20, new_tokens=60, seed=5)
        bench.run(steps=7, warmup=0)
        result = bench.run(steps=40, warmup=0)
        assert result["steps"] == 40 and result["tokens"] == 120
        assert (engine.metrics["steps_ahead"] > 30) == ahead
        runs[ahead] = [engine.poll(r)[1] for r in bench.ids]
        assert all(engine.status(r) == RequestStatus.DECODING for r in bench.ids)
        assert all(len(t) >= 47 for t in runs[ahead])
        bench.close()
        engine.loaded.cache.check()
        assert engine.loaded.cache.n_free_slots == 4 and engine.loaded.cache.free_pages() == [64]
    assert [t[:47] for t in runs[True]] == [t[:47] for t in runs[False]]


@pytest.mark.parametrize("name,dtype", [("B", "bfloat16"), ("A", "bfloat16"), ("B", "float32")])
def test_greedy_tokens_from_what_the_head_leaves_beside_the_logits(model_folders, name, dtype):
    """In bfloat16 the head's product of up to 64 rows leaves the best logit of every share of a row's
    columns, and greedy rows without a penalty take their token from that instead of reading the
    logits again: the same tokens as with that switched off, in recorded and in eager steps; a request
    with a repetition penalty in the batch sends the whole batch to the kernels that read the logits."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY, GenerationConfig
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, 0.05)
    vocab = plain.load_model_folder(folder)[0]["vocab_size"]
    prompts = [random_tokens(vocab, n, seed=70 + n) for n in (9, 20, 3)]
    outs, merged = {}, {}
    for head_argmax in (1, 0):
        engine = Engine.from_folder(folder, dtype=dtype, max_active_requests=4, n_pages=32, page_tokens=16,
                                    max_batched_tokens=64, prefill_chunk_tokens=16)
        engine.loaded.set_knob("use_head_argmax", head_argmax)
        outs[head_argmax] = engine.generate(prompts, max_new_tokens=24, generation=GREEDY, eos_token_ids=[])
        merged[head_argmax] = engine.loaded.paths()["argmax_merged"]
        if head_argmax:
            penalised = GenerationConfig(temperature=0.0, top_k=1, top_p=1.0, repetition_penalty=1.3)
            before = engine.loaded.paths()["argmax_merged"]
            both = engine.generate(prompts[:2], max_new_tokens=8, generations=[GREEDY, penalised], eos_token_ids=[])
            assert both[0] == outs[1][0][:8]
            # (the first request decodes alone while the other's prompt is still fed: those steps may merge)
            assert engine.loaded.paths()["argmax_merged"] - before <= 4
    assert outs[1] == outs[0]
    assert merged[0] == 0
    assert (merged[1] >= 20) == (dtype == "bfloat16")


def test_generation_ahead_of_the_tokens_with_requests_that_end_early(model_folders):
    """``generate`` launches decode steps before it has read the previous step's tokens.
    With end tokens chosen so that requests end at different steps (a request that ends
    rides along for one dropped row), and with sampling, the tokens equal the plain
    implementation's and those of an engine that never runs ahead."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY, GenerationConfig
    folder = model_folders("B", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, seed=300 + n) for n in (6, 11, 19, 4)]
    free_run = [plain_generate(cfg, W, p, 24) for p in prompts]
    # end tokens: what request 0 says at step 5, request 2 at step 11
    eos = [free_run[0][5], free_run[2][11]]
    outs = {}
    for ahead in (True, False):
        engine = Engine.from_folder(folder, dtype="float32", max_active_requests=4, n_pages=24,
                                    max_batched_tokens=64, prefill_chunk_tokens=32, run_ahead=ahead)
        outs[ahead] = engine.generate(prompts, max_new_tokens=24, generation=GREEDY, eos_token_ids=eos)
        assert (engine.metrics["steps_ahead"] > 10) == ahead
        assert engine.loaded.cache.free_pages() == [24] and engine.loaded.cache.n_free_slots == 4
        engine.loaded.cache.check()
    assert outs[True] == outs[False]
    for run, out in zip(free_run, outs[True]):
        cut = next((i + 1 for i, t in enumerate(run) if t in eos), len(run))
        assert out == run[:cut]
    assert len(outs[True][0]) <= 6 and len(outs[True][2]) <= 12
    # with a generator per request
    gen = GenerationConfig(temperature=0.9, top_k=30, top_p=0.95, repetition_penalty=1.2, seed=11)
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=4, n_pages=24,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    sampled = engine.generate(prompts, max_new_tokens=12, generation=gen, eos_token_ids=[])
    assert engine.metrics["steps_ahead"] > 5
    for prompt, out in zip(prompts, sampled):
        assert out == plain_generate(cfg, W, prompt, 12, generation=gen)


def test_cancelling_while_steps_run_ahead(model_folders):
    """A request cancelled while others decode (steps launched ahead of their tokens): the
    others' tokens are the plain implementation's, the cancelled one keeps what it had, and
    everything is given back.  A request that cannot fit the context is refused at the door."""
    from celeg_amd.engine import Engine, RequestOptions, RequestStatus
    from celeg_amd.sampling import GREEDY
    folder = model_folders("B", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    prompts = [random_tokens(cfg["vocab_size"], n, seed=400 + n) for n in (9, 14, 20)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=3, n_pages=12, context=64,
                                max_batched_tokens=64, prefill_chunk_tokens=32)
    options = RequestOptions(max_new_tokens=30, eos_token_ids=[], generation=GREEDY)
    ids = [engine.submit(p, options) for p in prompts]
    assert engine.native.run_steps(6) == 6
    engine.cancel(ids[1])
    engine.run()
    assert engine.metrics["steps_ahead"] > 20
    results = [engine.poll(r) for r in ids]
    assert [r[0] for r in results] == [RequestStatus.FINISHED, RequestStatus.CANCELLED, RequestStatus.FINISHED]
    want = [plain_generate(cfg, W, p, 30) for p in prompts]
    assert results[0][1] == want[0] and results[2][1] == want[2]
    assert 1 <= len(results[1][1]) <= 8 and results[1][1] == want[1][:len(results[1][1])]
    assert engine.loaded.cache.free_pages() == [12] and engine.loaded.cache.n_free_slots == 3
    engine.loaded.cache.check()
    with pytest.raises(Exception, match="max_context"):
        engine.submit(list(range(41)), options)
    after = engine.submit(prompts[0], options)          # the engine goes on
    with pytest.raises(ValueError, match="has not ended"):
        engine.release(after)                           # queued: a record goes only once its request has ended
    engine.run()
    assert engine.poll(after) == (RequestStatus.FINISHED, want[0], "")
    for rid in ids + [after]:
        engine.release(rid)
    with pytest.raises(Exception, match="unknown request id"):
        engine.status(after)


def test_a_checkpoint_with_tensors_nobody_asks_for_loads_and_generates(model_folders, tmp_path, capfd):
    """A tied model whose checkpoint still carries lm_head.weight (filled with other values) and an
    exported buffer: the reference binds tensors by name and leaves the rest alone
    (include/celeg/checkpoint/weight_repository.hpp:14-20), and so does loading here: a warning
    names them, the description lists them, and the tokens are those of the folder without them.
    With strict_weights the same folder is refused."""
    import shutil
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    from celeg_amd.weights import SafetensorsFile, WeightError, write_safetensors
    src = model_folders("A", torch.float32, WEIGHT_STD)
    folder = str(tmp_path / "extra")
    os.makedirs(folder)
    shutil.copy(os.path.join(src, "config.json"), folder)
    f = SafetensorsFile(os.path.join(src, "model.safetensors"))
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    tensors["lm_head.weight"] = torch.randn_like(tensors["model.embed_tokens.weight"])
    tensors["model.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    prompts = [random_tokens(256, n, seed=70 + n) for n in (9, 21)]
    outs = {}
    for name, where in (("plain", src), ("extra", folder)):
        engine = Engine.from_folder(where, dtype="float32", max_active_requests=2, n_pages=8, max_batched_tokens=32)
        outs[name] = engine.generate(prompts, max_new_tokens=8, generation=GREEDY, eos_token_ids=[])
        if name == "extra":
            assert engine.loaded.native.info["unused_tensors"] == ["lm_head.weight", "model.rotary_emb.inv_freq"]
    assert outs["extra"] == outs["plain"]
    assert "lm_head.weight" in capfd.readouterr().err
    with pytest.raises(WeightError, match="unexpected tensors"):
        Engine.from_folder(folder, dtype="float32", max_active_requests=2, n_pages=8, strict_weights=True)

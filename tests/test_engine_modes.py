"""The engine against the plain implementation in every way of cutting and batching:
each request alone and whole; most of it in one step and the last 32 tokens one by
one; portions of changing size down to two tokens; mixed, up to four live requests
with so few pages that they are used again; in 32-bit and bfloat16, through the library's
step function and cache manager (the ones generation uses).
"""
import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY
from helpers import (WEIGHT_STD, EngineDriver, assert_close, mixed_schedule, peak_tokens,
                     portions_schedule, random_tokens, tail_decode_schedule, whole_schedule)

LENGTHS = {"A": [40, 57, 90, 128, 65, 33], "B": [45, 200, 64, 100, 256, 33],
           "C": [70, 33, 150, 97, 48, 260], "D": [300, 66, 129, 40, 210, 77],
           "E": [300, 150, 97, 260, 70, 200]}
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


def run_mode(model_folders, name, dtype, mode, device, subset=None, gemm_backend="auto", knobs=None):
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
                    max_batched_tokens=max(max_tokens, 64), gemm_backend=gemm_backend)
    for knob, value in (knobs or {}).items():
        lm.set_knob(knob, value)
    got = EngineDriver(lm).run(steps)
    ref = plain_logits(folder, name, storage)
    for rid in reqs:
        assert_close(got[rid], ref[rid], dtype, f"{name}/{dtype}/{mode}/{rid}")
    lm.cache.check()
    assert lm.cache.n_free_slots == 4 and lm.cache.free_pages() == [max_tokens // 16]
    return lm


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(SCHEDULES))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_gpu_engine_matches_plain(model_folders, name, dtype, mode):
    run_mode(model_folders, name, dtype, mode, "cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("mode", list(SCHEDULES))
def test_gpu_engine_with_tiled_products_matches_plain(model_folders, mode):
    """Steps of more than 64 rows through the tiled products (norm, SwiGLU and residual sum
    folded in) instead of the library's: whole prompts of up to 300 tokens, and portions
    beside single tokens."""
    lm = run_mode(model_folders, "E", "bfloat16", mode, "cuda:0", gemm_backend="tiles")
    assert lm.knobs()["use_tiled_products"] == 1 and lm.native.info["gemm_backend"] == "tiles"
    # (q/k norm, rotation and cache write inside the q/k/v product's kernel for long steps, inside the
    # attention kernel for decode-only steps)
    assert lm.knobs()["use_qkv_tail"] == 1 and lm.knobs()["use_fresh_decode"] == 1
    # the same with the q/k norm, the rotation and the cache write as a kernel of their own
    run_mode(model_folders, "E", "bfloat16", mode, "cuda:0", gemm_backend="tiles",
             knobs={"use_qkv_tail": 0, "use_fresh_decode": 0})
    # and with the step's prologue (block-table updates, tokens from the device) as a kernel of its
    # own instead of inside the embedding's
    assert lm.knobs()["defer_prologue"] == 1
    run_mode(model_folders, "E", "bfloat16", mode, "cuda:0", gemm_backend="tiles", knobs={"defer_prologue": 0})
    # and the same configuration through the library's products
    lm = run_mode(model_folders, "E", "bfloat16", mode, "cuda:0", gemm_backend="library")
    assert lm.knobs()["use_tiled_products"] == 0 and lm.native.info["gemm_backend"] == "library"


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_gpu_engine_through_the_library_products_matches_plain(model_folders, name):
    """The other tests take the products that the width of their models selects (the tiled
    ones); here every configuration's prompts go through the library's products."""
    lm = run_mode(model_folders, name, "bfloat16", "whole", "cuda:0", gemm_backend="library")
    assert lm.native.info["gemm_backend"] == "library"


@pytest.mark.gpu
def test_the_products_of_long_steps_follow_the_sizes_of_the_products(model_folders):
    """Steps of many rows take the tiled products where the stream is at most ``tiled_max_width`` wide
    (1,024 as measured) and the library's above; the rule looks at the products, and the knob moves it."""
    lm = run_mode(model_folders, "E", "bfloat16", "whole", "cuda:0")
    assert lm.native.info["gemm_backend"] == "tiles" and lm.native.info["tiled_max_width"] == 1024
    paths = lm.paths()
    heads = len(LENGTHS["E"])          # the output head over all rows of a whole prompt is the library's in either case
    assert paths["tiled"] > 0 and paths["tiled_qkv"] > 0 and paths["linear_library"] == heads, paths
    lm = run_mode(model_folders, "E", "bfloat16", "whole", "cuda:0", knobs={"tiled_max_width": 127})
    paths = lm.paths()
    assert paths["tiled"] == 0 and paths["tiled_qkv"] == 0 and paths["linear_library"] > 10 * heads, paths


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
        replays = lm.runner.counters()["graph_replays"]
        assert (replays > 0) == use_graphs, "decode steps were (not) replayed from a graph"
    for rid in reqs:
        if dtype == "float32":
            assert torch.equal(out[True][rid], out[False][rid])
        else:
            assert_close(out[True][rid], out[False][rid].double(), dtype, f"graph/{rid}")


def merged_schedule(per_request_steps):
    """Steps of several requests laid side by side: step k holds the k-th step of each."""
    merged = []
    for k in range(max(len(v) for v in per_request_steps.values())):
        entries, end = [], []
        for v in per_request_steps.values():
            if k < len(v):
                entries += v[k]["entries"]
                end += v[k]["end"]
        merged.append({"step": k, "entries": entries, "end": end})
    return merged


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_long_decoding(model_folders, name, dtype):
    """Three requests decoded one token a step for most of the context (hundreds of steps
    through the replayed graphs, across many page edges), every position compared with the
    plain implementation."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    cfg = TINY[name][0]
    n = min(cfg["max_position_embeddings"], 250)
    reqs = {f"long{i}": random_tokens(cfg["vocab_size"], n - 7 * i, seed=900 + i) for i in range(3)}
    steps = merged_schedule({rid: tail_decode_schedule({rid: toks}, tail=len(toks) - 20)
                             for rid, toks in reqs.items()})
    max_tokens = peak_tokens(steps)
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=max_tokens // 16, max_requests=4,
                    max_batched_tokens=256)
    got = EngineDriver(lm).run(steps)
    cfgp, W = plain.load_model_folder(folder)
    for rid, toks in reqs.items():
        assert_close(got[rid], plain.model_logits(cfgp, W, toks), dtype, f"{name}/{dtype}/long/{rid}")
    assert lm.runner.counters()["graph_replays"] > 100, "the decode steps were not replayed from a graph"
    lm.cache.check()


@pytest.mark.gpu
@pytest.mark.parametrize("whole", [-1, 1])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_with_the_context_cut_into_parts_of_several_rounds(model_folders, dtype, whole):
    """The decode attention over few requests cuts a context into parts, and a recorded decode step
    fixes how: by the longest context the recording serves (here the model's 512 positions, 8 rounds
    of 64 keys).  With the thresholds lowered to 1 and 8 rounds the recording takes parts of 4
    rounds instead of one round a part, so that two requests decoding from 20 to 330 tokens run
    through parts that are empty at first, half full later and full at the end; every position is
    compared with the plain implementation.  Once more with the kernel of many requests (one
    workgroup a request and key/value head) forced.  (Contexts that cross the bounds between
    recordings, 4,096 tokens and up, are in test_gpu_long_context.py, with the thresholds as shipped.)"""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders("D", storage, WEIGHT_STD)
    cfg = TINY["D"][0]
    reqs = {f"bound{i}": random_tokens(cfg["vocab_size"], 330 - 11 * i, seed=940 + i) for i in range(2)}
    steps = merged_schedule({rid: tail_decode_schedule({rid: toks}, tail=len(toks) - 20)
                             for rid, toks in reqs.items()})
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=peak_tokens(steps) // 16, max_requests=2,
                    max_batched_tokens=256)
    lm.set_knob("decode_parts_few", 1)
    lm.set_knob("decode_parts_some", 8)
    lm.set_knob("attention_decode_whole", whole)
    got = EngineDriver(lm).run(steps)
    cfgp, W = plain.load_model_folder(folder)
    for rid, toks in reqs.items():
        assert_close(got[rid], plain.model_logits(cfgp, W, toks), dtype, f"D/{dtype}/bounds/{rid}")
    assert lm.runner.counters()["graph_replays"] > 300
    lm.cache.check()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(model_folders, name, dtype):
    """Position 0 and its neighbours: requests that start with one, two and three tokens
    side by side, then go on token by token."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    vocab = TINY[name][0]["vocab_size"]
    reqs = {f"first{i}": random_tokens(vocab, 7, seed=950 + i) for i in range(3)}
    per = {}
    for i, (rid, toks) in enumerate(reqs.items()):
        first = i + 1
        mine = [{"step": 0, "entries": [{"id": rid, "tokens": toks[:first], "want": list(range(first))}], "end": []}]
        for p in range(first, len(toks)):
            mine.append({"step": len(mine), "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                         "end": [rid] if p == len(toks) - 1 else []})
        per[rid] = mine
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=8, max_requests=4, max_batched_tokens=64)
    got = EngineDriver(lm).run(merged_schedule(per))
    cfgp, W = plain.load_model_folder(folder)
    for rid, toks in reqs.items():
        assert len(got[rid]) == 7
        assert_close(got[rid], plain.model_logits(cfgp, W, toks), dtype, f"{name}/{dtype}/first/{rid}")
    lm.cache.check()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C"])
def test_portions_of_a_repeated_size(model_folders, name, dtype):
    """Prompts that arrive in equal portions, the last one's last row wanted, with decode
    tokens between them: every wanted row against the plain implementation."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    vocab = TINY[name][0]["vocab_size"]
    reqs = {f"eq{i}": random_tokens(vocab, 48 * 3 + 2, seed=970 + i) for i in range(4)}
    steps = []
    for rid, toks in reqs.items():
        for p in range(3):      # 48, 48 (no logits), then 48 with the last row's logits
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": toks[48 * p:48 * p + 48], "want": [47] if p == 2 else []}], "end": []})
        for p in (144, 145):    # two decode tokens
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": [toks[p]], "want": [0]}], "end": [rid] if p == 145 else []})
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=peak_tokens(steps) // 16 + 1,
                    max_requests=4, max_batched_tokens=64)
    got = EngineDriver(lm).run(steps)
    cfgp, W = plain.load_model_folder(folder)
    for rid, toks in reqs.items():
        ref = plain.model_logits(cfgp, W, toks)
        assert_close(got[rid], ref[[143, 144, 145]], dtype, f"{name}/{dtype}/replayed/{rid}")
    lm.cache.check()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_mixed_steps_of_a_repeated_shape(model_folders, name, dtype):
    """The steady state of serving under a token budget: every step holds portions of prompts
    of the portion size beside the single tokens of the requests that decode, and the entries
    come in changing order (a portion first, between or behind the single tokens).  Every
    wanted row is checked against the plain implementation."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    vocab = TINY[name][0]["vocab_size"]
    P, n_portions, n_decode = 40, 2, 9
    reqs = {f"m{i}": random_tokens(vocab, P * n_portions + n_decode, seed=1200 + i) for i in range(7)}
    ids = list(reqs)
    # request i starts at step stride * i: two steps of a portion, then one token a step
    # (stride 2: one portion a step; stride 1: two portions of different requests a step)
    stride = 2 if name == "B" else 1
    steps, k = [], 0
    while True:
        entries, end = [], []
        for i, rid in enumerate(ids):
            j = k - stride * i
            toks = reqs[rid]
            if 0 <= j < n_portions:
                entries.append({"id": rid, "tokens": toks[P * j:P * j + P],
                                "want": [P - 1] if j == n_portions - 1 else []})
            elif n_portions <= j < n_portions + n_decode:
                pos = P * n_portions + j - n_portions
                entries.append({"id": rid, "tokens": [toks[pos]], "want": [0]})
                if pos == len(toks) - 1:
                    end.append(rid)
        if not entries:
            break
        entries = entries[k % len(entries):] + entries[:k % len(entries)]     # a changing order
        steps.append({"step": k, "entries": entries, "end": end})
        k += 1
    lm = load_model(folder, dtype=dtype, page_tokens=16, n_pages=peak_tokens(steps) // 16 + 8,
                    max_requests=8, max_batched_tokens=128)
    got = EngineDriver(lm).run(steps)
    cfgp, W = plain.load_model_folder(folder)
    first = P * n_portions - 1
    for rid, toks in reqs.items():
        ref = plain.model_logits(cfgp, W, toks)
        assert_close(got[rid], ref[first:], dtype, f"{name}/{dtype}/mixed replay/{rid}")
    lm.cache.check()


def many_requests_schedule(requests, tail, join_every=0):
    """Every request's head in a step of its own, then decode steps that hold ALL requests
    (one token each); with ``join_every`` the heads are spread between the decode steps instead,
    a portion beside the tokens of the requests that already decode."""
    ids = list(requests)
    steps = []
    heads = {rid: len(requests[rid]) - tail for rid in ids}
    started = []
    def head_entry(rid):
        return {"id": rid, "tokens": requests[rid][:heads[rid]], "want": list(range(heads[rid]))}
    if not join_every:
        for rid in ids:
            steps.append({"step": len(steps), "entries": [head_entry(rid)], "end": []})
        started = list(ids)
    done = {rid: 0 for rid in ids}
    waiting = [rid for rid in ids if rid not in started]
    while waiting or any(done[r] < tail for r in started):
        entries = []
        for rid in started:
            if done[rid] < tail:
                i = heads[rid] + done[rid]
                entries.append({"id": rid, "tokens": requests[rid][i:i + 1], "want": [0]})
                done[rid] += 1
        joined = []
        if waiting and (len(steps) % join_every == 0 if join_every else False):
            rid = waiting.pop(0)
            entries.insert(len(entries) // 2, head_entry(rid))     # a portion between single tokens
            joined.append(rid)
        if entries:
            steps.append({"step": len(steps), "entries": entries,
                          "end": [r for r in started if done[r] == tail and r not in
                                  [x for st in steps for x in st["end"]]]})
        else:
            steps.append({"step": len(steps), "entries": [head_entry(waiting.pop(0))], "end": []})
            joined.append(steps[-1]["entries"][0]["id"])
        started += joined
    return steps


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,n_requests,join_every", [("D", 12, 0), ("D", 40, 0), ("B", 23, 0), ("D", 20, 2),
                                                       ("A", 64, 0), ("D", 100, 0)])
def test_many_requests_decoding_together(model_folders, name, n_requests, join_every, dtype):
    """Decode steps of 9 to 64 rows (the products for many rows, their convolution and residual
    epilogues, the decode attention for batches), of 100 rows (the library's products), and
    portions joining between the single tokens of requests that already decode: every
    request's logits equal the plain ones."""
    from celeg_amd.engine import load_model
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    folder = model_folders(name, storage, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    vocab = cfg["vocab_size"]
    tail = 30 if join_every else 6
    lengths = [tail + 3 + (7 * i) % 50 for i in range(n_requests)]
    reqs = {f"m{i}": random_tokens(vocab, n, seed=900 + i) for i, n in enumerate(lengths)}
    steps = many_requests_schedule(reqs, tail, join_every)
    most = max(len(s["entries"]) for s in steps)
    assert most == n_requests if not join_every else most >= 12
    pages = sum((n + 15) // 16 for n in lengths)
    lm = load_model(folder, dtype=dtype, device="cuda:0", page_tokens=16, n_pages=pages,
                    max_requests=n_requests, max_batched_tokens=128)
    got = EngineDriver(lm).run(steps)
    for rid in list(reqs)[::max(1, n_requests // 8)]:
        ref = plain.model_logits(cfg, W, reqs[rid])
        assert_close(got[rid], ref, dtype, f"{name}/{dtype}/{n_requests} together/{rid}")
    lm.cache.check()
    assert lm.cache.n_free_slots == n_requests and lm.cache.free_pages() == [pages]


@pytest.mark.gpu
def test_a_large_reservation_and_a_refused_step_keep_the_device_tables_right(model_folders):
    """Pages reserved hundreds at a time (what guaranteed_no_evict does at admission) are more
    block-table updates than a step's metadata has room for: the step function ships them on
    their own.  A step that is refused after the cache manager handed its updates over (a wanted
    place outside the entry) leaves them queued for the next step, whose logits are then those
    of the plain implementation."""
    from celeg_amd.engine import StepEntry, load_model
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=40, max_requests=4, max_context=128,
                    max_batched_tokens=16)
    slots = [lm.cache.open() for _ in range(4)]
    for s in slots:
        assert lm.cache.prepare(s, 0, 128)          # 8 pages each, 32 updates pending; room for 16/16 + 8 + 8 = 17
    prompts = [random_tokens(256, 9 + i, seed=40 + i) for i in range(4)]
    logits = lm.runner.step([StepEntry(s, 0, p[:3], [2]) for s, p in zip(slots, prompts)])
    for i, p in enumerate(prompts):
        assert_close(logits[i], plain.model_logits(cfg, W, p[:3])[-1], "float32", f"burst/{i}")
    for s in slots:
        lm.cache.close(s)
    slots = [lm.cache.open() for _ in range(2)]
    assert lm.cache.prepare(slots[0], 0, 20) and lm.cache.prepare(slots[1], 0, 4)
    with pytest.raises(ValueError, match="wanted place"):
        lm.runner.step([StepEntry(slots[0], 0, prompts[0][:5], [5])])
    with pytest.raises(ValueError, match="exceed max_batched_tokens"):
        lm.runner.step([StepEntry(slots[0], 0, prompts[0][:5] * 4, [4])])
    logits = lm.runner.step([StepEntry(slots[0], 0, prompts[0][:5], [4]),
                             StepEntry(slots[1], 0, prompts[1][:4], [3])])
    assert_close(logits[0], plain.model_logits(cfg, W, prompts[0][:5])[-1], "float32", "after refusal/0")
    assert_close(logits[1], plain.model_logits(cfg, W, prompts[1][:4])[-1], "float32", "after refusal/1")
    lm.cache.check()


@pytest.mark.gpu
def test_few_rows_and_many_rows_agree_at_norm_weights_far_from_one(model_folders, tmp_path):
    """Steps of up to 64 rows multiply the norm's weight into the bfloat16 matrices (one more
    rounding of every weight); steps of more rows apply it to the rows in 32-bit.  With norm
    weights between 0.3 and 3 the two still give the same logits within the bfloat16 bound,
    and each agrees with the plain implementation."""
    from celeg_amd.engine import load_model
    from celeg_amd.weights import SafetensorsFile, write_safetensors
    import json, os, shutil
    src = model_folders("E", torch.bfloat16, WEIGHT_STD)
    folder = str(tmp_path / "far_from_one")
    os.makedirs(folder)
    shutil.copy(os.path.join(src, "config.json"), folder)
    f = SafetensorsFile(os.path.join(src, "model.safetensors"))
    g = torch.Generator().manual_seed(5)
    tensors = {}
    for name in f.names():
        t = f.tensor(name).clone()
        if name.endswith("norm.weight"):                 # operator_norm, ffn_norm, embedding_norm
            t = (t.float() * torch.exp(torch.empty(t.shape).uniform_(-1.2, 1.1, generator=g))).to(t.dtype)
        tensors[name] = t
    f.close()
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    cfg, W = plain.load_model_folder(folder)
    toks = random_tokens(TINY["E"][0]["vocab_size"], 200, seed=77)
    ref = plain.model_logits(cfg, W, toks)
    reqs = {"r": toks}
    out = {}
    for mode, steps in (("many", whole_schedule(reqs)),
                        ("few", portions_schedule(reqs, sizes=(16, 9, 33, 2, 64, 1)))):
        lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=16, max_requests=2,
                        max_batched_tokens=256)
        out[mode] = EngineDriver(lm).run(steps)["r"]
        assert_close(out[mode], ref, "bfloat16", f"norm weights far from one/{mode}")
    assert_close(out["few"], out["many"].double(), "bfloat16", "few rows against many rows")

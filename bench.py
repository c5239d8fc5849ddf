"""Headline benchmark: decode tokens/s of an LFM2-350M-shaped model (bfloat16, random
weights, synthetic tokens) at batch 8 on ONE MI355X, with prefill throughput at 2,048
tokens, decode at batch 1 and 64, and roofline fractions.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one decode step of the whole batch (greedy sampling on the device included).
Prints ONE JSON line.  Peaks are MI355X's published ones: HBM 8 TB/s, dense bf16 MFMA
2.5 PFLOP/s.
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

# The layer sizes of the LFM2-350M shape: 16 layers, attention at {2,5,8,10,12,14}.
LFM2_350M = {
    "architectures": ["Lfm2ForCausalLM"], "model_type": "lfm2",
    "vocab_size": 65536, "hidden_size": 1024, "num_hidden_layers": 16,
    "layer_types": ["conv", "conv", "full_attention", "conv", "conv", "full_attention", "conv",
                    "conv", "full_attention", "conv", "full_attention", "conv", "full_attention",
                    "conv", "full_attention", "conv"],
    "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 64,
    "intermediate_size": 6656, "block_auto_adjust_ff_dim": True, "block_multiple_of": 256,
    "block_ffn_dim_multiplier": 1.0, "rope_theta": 1000000.0, "conv_L_cache": 3,
    "conv_bias": False, "tie_word_embeddings": True, "norm_eps": 1e-5,
    "max_position_embeddings": 4096, "bos_token_id": 1, "eos_token_id": 7, "pad_token_id": 0,
}
PROMPT_TOKENS = 2048
BATCH = 8


def lfm2_shape(hidden, heads, kv_heads, intermediate, attention_layers, layers, context):
    cfg = dict(LFM2_350M)
    cfg.update(hidden_size=hidden, num_attention_heads=heads, num_key_value_heads=kv_heads,
               intermediate_size=intermediate, num_hidden_layers=layers,
               layer_types=["full_attention" if i in attention_layers else "conv" for i in range(layers)],
               max_position_embeddings=context)
    return cfg


# The other LFM2 shapes, each with the serving workload it is measured on (--phase serve):
# requests, prompt lengths (lowest, highest), new tokens, prefill portion, most tokens a step.
SHAPES = {
    "350m": (LFM2_350M, dict(requests=64, prompt=(2048, 2048), new_tokens=256, chunk=2048, budget=2048)),
    "1.2b": (lfm2_shape(2048, 32, 8, 12288, {2, 5, 8, 10, 12, 14}, 16, 4096),
             dict(requests=64, prompt=(128, 2048), new_tokens=256, chunk=2048, budget=2048)),
    "2.6b": (lfm2_shape(2048, 32, 8, 10752, {2, 6, 10, 14, 18, 21, 24, 27}, 30, 8192),
             dict(requests=32, prompt=(4096, 4096), new_tokens=512, chunk=512, budget=1024)),
}


def prefill_flops(cfg, tokens: int, ff: int, offset: int = 0) -> float:
    H, hq, hkv, hd = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    per_token = 0
    attention = 0.0
    for kind in cfg["layer_types"]:
        if kind == "conv":
            per_token += 2 * (3 * H * H + H * H)
        else:
            per_token += 2 * ((hq + 2 * hkv) * hd * H + hq * hd * H)
            attention += 4.0 * hq * hd * (tokens * (tokens + 1) / 2 + tokens * offset)     # QK^T and PV, causal
        per_token += 2 * 3 * H * ff
    return per_token * tokens + attention + 2.0 * H * cfg["vocab_size"]   # head for one row


def serve(shape: str, chunk: int = 0, budget: int = 0, granule: int = 1, gemm_backend: str = "auto") -> int:
    """The whole engine on a serving workload: every request submitted at once, the scheduler
    cuts the prompts into portions beside the decoding requests, sampling is greedy on the
    device.  Prints one JSON line: generated tokens a second over the whole run."""
    import random
    import torch
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    from celeg_amd.weights import write_random_model

    cfg, load = SHAPES[shape]
    load = dict(load, chunk=chunk or load["chunk"], budget=budget or load["budget"])
    rng = random.Random(0)
    lengths = [rng.randint(*load["prompt"]) for _ in range(load["requests"])]
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(n)] for n in lengths]
    pages = sum((n + load["new_tokens"] + 15) // 16 + 1 for n in lengths)
    with tempfile.TemporaryDirectory(prefix="celeg_bench_") as folder:
        write_random_model(cfg, folder, seed=0, dtype=torch.bfloat16, std=0.02)
        engine = Engine.from_folder(folder, dtype="bfloat16", device="cuda:0", page_tokens=16,
                                    n_pages=pages, max_active_requests=load["requests"],
                                    max_batched_tokens=load["budget"],
                                    prefill_chunk_tokens=load["chunk"], portion_granule=granule,
                                    context=cfg["max_position_embeddings"], gemm_backend=gemm_backend)
    # a short run first: weights re-laid, a graph recorded
    engine.generate(prompts[:2], max_new_tokens=4, generation=GREEDY, eos_token_ids=[])
    before = engine.metrics
    engine.loaded.native.synchronize()
    start = time.perf_counter()
    out = engine.generate(prompts, max_new_tokens=load["new_tokens"], generation=GREEDY, eos_token_ids=[])
    engine.loaded.native.synchronize()
    seconds = time.perf_counter() - start
    after = engine.metrics
    generated = sum(len(o) for o in out)
    print(json.dumps({
        "metric": f"serve: generated tok/s (LFM2-{shape.upper()} shape, bf16, whole engine)",
        "value": round(generated / seconds, 1), "unit": "tokens/s", "phase": "serve",
        "seconds": round(seconds, 3), "generated_tokens": generated,
        "prompt_tokens": sum(lengths),
        "all_tokens_per_second": round((generated + sum(lengths)) / seconds, 1),
        "requests": load["requests"], "prompt_lengths": list(load["prompt"]),
        "new_tokens": load["new_tokens"], "prefill_chunk": load["chunk"],
        "step_token_budget": load["budget"], "portion_granule": granule, "context": cfg["max_position_embeddings"],
        "engine_steps": after["steps"] - before["steps"],
        "decode_steps": after["decode_steps"] - before["decode_steps"],
        "portion_steps": after["portion_steps"] - before["portion_steps"],
        "mixed_steps": after["mixed_steps"] - before["mixed_steps"],
        "steps_launched_ahead": after["steps_ahead"] - before["steps_ahead"],
        "steps_replayed_from_graphs": after["graph_replays"] - before["graph_replays"],
        "graphs_recorded": after["captures"] - before["captures"],
        "recording_seconds": round(after["capture_seconds"] - before["capture_seconds"], 3),
        "prefill_products": engine.loaded.native.info["gemm_backend"], "dtype": "bf16", "data": "synthetic"}))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the shape has")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    ap.add_argument("--gemm-backend", choices=["auto", "library", "tiles"], default="auto",
                    help="products of steps of more than 64 rows (the prefill)")
    ap.add_argument("--batch", type=int, default=BATCH,
                    help="for profiling with --phase decode: another batch size than the headline's 8")
    ap.add_argument("--prefill-chunk", type=int, default=0,
                    help="serve phase: most tokens of a prompt in one step (default: the workload's)")
    ap.add_argument("--portion-granule", type=int, default=1,
                    help="serve phase: portions cut by the budget keep to multiples of this")
    ap.add_argument("--token-budget", type=int, default=0,
                    help="serve phase: most tokens of a step (default: the workload's)")
    ap.add_argument("--context", type=int, default=0,
                    help="with --phase decode: tokens every request holds when decoding starts "
                         "(default 2048, the headline's); with --phase prefill: tokens of the same "
                         "prompt that the cache holds before the measured portion of 2,048 (default 0)")
    ap.add_argument("--phase", choices=["all", "prefill", "decode", "serve"], default="all",
                    help="for profiling: run only the prefill measurement, or only the batch-8 "
                         "decode measurement (the line printed then holds only that part); "
                         "serve: the whole engine on the serving workload of --shape")
    ap.add_argument("--knob", action="append", default=[], metavar="NAME=VALUE",
                    help="set a knob of the step function or the kernels' dispatch before measuring "
                         "(tuning runs; the names are those of celeg_model_knobs)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="350m",
                    help="the LFM2 shape (the headline line is the 350m one)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {args.gpus} is not supported "
              "(this engine runs on a single MI355X)")
        return 2

    if args.phase == "serve":
        return serve(args.shape, args.prefill_chunk, args.token_budget, args.portion_granule, args.gemm_backend)

    import torch
    import celeg_amd  # noqa: F401
    from celeg_amd.engine import Engine
    from celeg_amd.engine.benchmark import DecodeBench, measure_prefill
    from celeg_amd.weights import write_random_model

    cfg = dict(SHAPES[args.shape][0])
    full_layers = cfg["num_hidden_layers"]
    if args.layers and args.layers < full_layers:
        cfg["num_hidden_layers"] = args.layers
        cfg["layer_types"] = cfg["layer_types"][:args.layers]
    decode_context = args.context if args.context > 0 and args.phase == "decode" else PROMPT_TOKENS
    prefill_offset = args.context if args.context > 0 and args.phase == "prefill" else 0
    max_batch = max(BATCH, args.batch) if args.no_points or args.phase != "all" else 64
    # (a request decodes along while the others' prompts are fed, a step for every portion of a prompt)
    portions = (decode_context + PROMPT_TOKENS - 1) // PROMPT_TOKENS
    need = max(decode_context + args.steps + args.warmup + max_batch * portions + 3, prefill_offset + PROMPT_TOKENS)
    if decode_context != PROMPT_TOKENS or prefill_offset:
        cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], need)
    context = cfg["max_position_embeddings"]
    if need > context:
        raise SystemExit(f"--steps + --warmup exceed the context of {context}")
    with tempfile.TemporaryDirectory(prefix="celeg_bench_") as folder:
        write_random_model(cfg, folder, seed=0, dtype=torch.bfloat16, std=0.02)
        pages_per_request = (need + 15) // 16 + 1
        engine = Engine.from_folder(folder, dtype="bfloat16", device="cuda:0", page_tokens=16,
                                    n_pages=pages_per_request * max_batch, max_active_requests=max_batch,
                                    context=context, max_batched_tokens=PROMPT_TOKENS,
                                    prefill_chunk_tokens=PROMPT_TOKENS, gemm_backend=args.gemm_backend)
    lm = engine.loaded
    for knob in args.knob:
        name, _, value = knob.partition("=")
        lm.set_knob(name, int(value))
    ff = int(lm.native.info["spec"]["layers"][0]["ffn"]["params"]["ff"])      # from the parts list, whatever the architecture
    w_bytes = lm.native.info["weights"] * 2          # every weight once, bfloat16
    kv_per_token = lm.native.info["kv_bytes_per_token"]

    flops = prefill_flops(cfg, PROMPT_TOKENS, ff, prefill_offset)
    if args.phase == "decode":
        prefill = None
    else:
        prefill = measure_prefill(lm, PROMPT_TOKENS, repeats=7, warmup=3, offset=prefill_offset)
    if args.phase == "prefill":
        where = f" after {prefill_offset} tokens of the same prompt" if prefill_offset else ""
        print(json.dumps({"metric": f"prefill tok/s @ 2048 tokens{where} (LFM2-{args.shape.upper()} shape, bf16)",
                          "value": round(prefill["tokens_per_second"], 1), "unit": "tokens/s",
                          "ms": round(prefill["ms"], 4), "phase": "prefill",
                          "frac": round(flops / (prefill["ms"] * 1e-3) / PEAK_FLOPS["bf16"], 5)}))
        return 0

    def decode(batch: int):
        bench = DecodeBench(engine, batch, decode_context, args.steps + args.warmup + batch * portions + 2, seed=batch)
        result = bench.run(args.steps, args.warmup)
        bench.close()
        return result

    if args.phase == "decode" and (args.batch != BATCH or decode_context != PROMPT_TOKENS):
        result = decode(args.batch)
        step_bytes = w_bytes + kv_per_token * result["mean_context"] * args.batch
        achieved = step_bytes / (result["ms_per_step"] * 1e-3) / 1e9
        print(json.dumps({"metric": f"decode tok/s @ batch {args.batch}, context {decode_context} "
                                    f"(LFM2-{args.shape.upper()} shape, bf16)",
                          "value": round(result["tokens_per_second"], 1), "unit": "tokens/s",
                          "ms_per_step": round(result["ms_per_step"], 4), "phase": "decode",
                          "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                                       "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5)}}))
        return 0
    main_run = decode(BATCH)
    points = {}
    if not args.no_points and args.phase == "all":
        points = {"decode_b1": round(decode(1)["tokens_per_second"], 1),
                  "decode_b64": round(decode(64)["tokens_per_second"], 1)}
    mean_context = main_run["mean_context"]
    step_bytes = w_bytes + kv_per_token * mean_context * BATCH
    achieved = step_bytes / (main_run["ms_per_step"] * 1e-3) / 1e9
    line = {
        "metric": f"decode tok/s @ batch 8 (LFM2-{args.shape.upper()} shape, bf16, context 2048+)",
        "value": round(main_run["tokens_per_second"], 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(main_run["ms_per_step"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"model": f"LFM2-{args.shape.upper()} shape, random weights", "global_batch": BATCH,
                   "seq_len": context, "prompt_tokens": PROMPT_TOKENS, "parallelism": "single GPU",
                   "layers": cfg["num_hidden_layers"], "layers_of_shape": full_layers,
                   "attention_layers": cfg["layer_types"].count("full_attention"),
                   "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"],
                   "kv_heads": cfg["num_key_value_heads"], "head_dim": cfg["head_dim"],
                   "ff": ff, "vocab_size": cfg["vocab_size"], "conv_L_cache": cfg["conv_L_cache"],
                   "rope_theta": cfg["rope_theta"], "tied_embeddings": True, "page_tokens": 16,
                   "prefill_products": lm.native.info["gemm_backend"]},
        "prefill": None if prefill is None else {
            "value": round(prefill["tokens_per_second"], 1), "tokens": PROMPT_TOKENS,
            "ms": round(prefill["ms"], 4),
            "frac": round(flops / (prefill["ms"] * 1e-3) / PEAK_FLOPS["bf16"], 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 5)},
        "points": points,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())

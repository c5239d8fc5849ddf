"""``celeg-run``: load a model folder, feed a prompt, generate.

Option names, meanings and defaults are those of the reference's ``celeg-run``
(src/app/cuda/main.cpp:38-95 defaults, 105-160 flags, 204-272 validation) where it
has them: greedy by default (``--top-k 1``), ``--temperature 0.1``, ``--top-p 1.0``,
``--repetition-penalty 1.05``, ``--seed 1``, ``--max-new-tokens 128``, ``--context
4096``, ``--prefill-chunk 256``, ``--benchmark-warmup 8``.  This engine starts at token
ids (it has no tokenizer), so ``--prompt`` takes token ids ("5 17 3" or "5,17,3") and
the generated ids are printed; options of the reference that belong to parts this
engine does not have (chat templates, quantized weights and caches, expert offload,
speculative decoding, sessions) are not accepted.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
from typing import List, Optional


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="celeg-run", description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("model_positional", nargs="?", default=None, metavar="DIR")
    ap.add_argument("--model", default=None, help="folder with config.json and model.safetensors")
    ap.add_argument("--random-weights", default=None, metavar="CONFIG.json",
                    help="write a model folder with random weights for this config.json and run it")
    ap.add_argument("--random-weights-seed", type=int, default=0)
    ap.add_argument("--prompt", default=None, help="token ids, separated by spaces or commas")
    ap.add_argument("--prompt-file", default=None, help="file with token ids")
    ap.add_argument("--random-prompt", type=int, default=0, metavar="N",
                    help="N uniform random token ids as the prompt")
    ap.add_argument("--max-new-tokens", type=int, default=128)
    ap.add_argument("--context", type=int, default=None,
                    help="most tokens of a request (default: 4096 or the model's maximum if smaller)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--temperature", type=float, default=0.1)
    ap.add_argument("--top-k", type=int, default=1)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--repetition-penalty", type=float, default=1.05)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--dump-logits", default=None, metavar="FILE.f32",
                    help="write the logits after the prompt as raw 32-bit floats")
    ap.add_argument("--print-top", type=int, default=0, metavar="N")
    ap.add_argument("--tokens-only", action="store_true", help="print the prompt's ids and exit")
    ap.add_argument("--runtime-tokens", action="store_true",
                    help="print CELEG_GENERATED_TOKEN_IDS=[...]")
    ap.add_argument("--print-config", action="store_true")
    ap.add_argument("--memory-report", action="store_true")
    ap.add_argument("--runtime-metrics", action="store_true")
    ap.add_argument("--benchmark-decode", type=int, default=0, metavar="N")
    ap.add_argument("--benchmark-warmup", type=int, default=8, metavar="N")
    ap.add_argument("--benchmark-prefill-tokens", type=int, default=0, metavar="N")
    ap.add_argument("--batch", type=int, default=1, help="requests decoded together in benchmarks")
    ap.add_argument("--max-requests", type=int, default=0,
                    help="requests the engine holds at a time (default: --batch)")
    ap.add_argument("--prefill-chunk", type=int, default=256)
    ap.add_argument("--max-batched-tokens", type=int, default=0,
                    help="token budget of a step (default: the larger of 512 and --prefill-chunk)")
    ap.add_argument("--page-tokens", type=int, default=16)
    ap.add_argument("--pages", type=int, default=0, help="pages of the cache pool (default: enough)")
    ap.add_argument("--kv-cache", default="bf16", choices=["bf16"],
                    help="cache storage (quantized caches are not built)")
    ap.add_argument("--no-cuda-graph", "--no-graph", dest="no_graph", action="store_true",
                    help="do not replay decode steps from a captured graph")
    ap.add_argument("--profile", action="store_true",
                    help="time every step's phases (embedding, each layer's mixer and feed-forward, head) "
                         "with events and print ms per step by phase; such steps are not replayed from graphs "
                         "(the reference's CELEG_PROFILE_DECODE / CELEG_PROFILE_PREFILL)")
    ap.add_argument("--dump-hidden", default="", metavar="DIR",
                    help="write the 32-bit residual stream after every layer of every step to "
                         "DIR/step<k>_layer<i>.f32 (the reference's CELEG_DEBUG_HIDDEN_DIR)")
    ap.add_argument("--gemm-backend", default="auto", choices=["auto", "library", "tiles"],
                    help="bfloat16 steps of more than 64 rows: the library's matrix products, this "
                         "package's tiled products with norm, SwiGLU and residual sum folded in, or "
                         "(auto) the one that was measured faster at the model's width")
    ap.add_argument("--attention-mode", default="auto", choices=["single", "segmented", "auto"],
                    help="attention of a decoding request: one workgroup per request and key/value head "
                         "over the whole context (single), the context cut into parts that workgroups of "
                         "their own take and a second kernel joins (segmented), or (auto) segmented for few "
                         "requests and single for batches that fill the chip by themselves (the reference's "
                         "flag of this name, src/app/cuda/main.cpp:129; its auto goes by the position)")
    ap.add_argument("--attention-chunk-tokens", type=int, default=0, metavar="N",
                    help="keys of a part of segmented attention: 64, 256 or 1024 (default: by the context, "
                         "64 up to 4,096 tokens, 256 up to 16,384, 1024 above)")
    ap.add_argument("--strict-weights", action="store_true",
                    help="refuse a checkpoint that holds tensors the model has no use for (default: a warning)")
    ap.add_argument("--device", default="cuda:0")
    return ap


def parse_token_ids(text: str) -> List[int]:
    try:
        return [int(t) for t in text.replace(",", " ").split()]
    except ValueError as err:
        raise SystemExit(f"error: --prompt takes token ids: {err}")


def validate(args, ap) -> None:
    """The reference's checks (src/app/cuda/main.cpp:204-221)."""
    if args.model is None:
        args.model = args.model_positional
    if args.model is None and args.random_weights is None:
        ap.error("--model or --random-weights is required")
    if args.model is not None and args.random_weights is not None:
        ap.error("--model and --random-weights are mutually exclusive")
    has_prompt = args.prompt is not None or args.prompt_file is not None or args.random_prompt > 0 \
        or args.benchmark_prefill_tokens > 0
    if not args.print_config and not has_prompt:
        ap.error("--prompt is required unless --print-config is used")
    if (args.context is not None and args.context <= 0) or args.max_new_tokens < 0 or args.print_top < 0 or args.top_k <= 0 \
            or args.temperature < 0.0 or args.top_p <= 0.0 or args.top_p > 1.0 \
            or args.repetition_penalty < 1.0 or args.seed == 0 or args.benchmark_decode < 0 \
            or args.benchmark_warmup < 0 or args.benchmark_prefill_tokens < 0 \
            or args.prefill_chunk <= 0 or args.batch <= 0 or args.page_tokens <= 0:
        ap.error("invalid numeric argument")
    if args.attention_chunk_tokens not in (0, 64, 256, 1024):
        ap.error("--attention-chunk-tokens must be 64, 256 or 1024")


def main(argv: Optional[List[str]] = None) -> int:
    ap = build_parser()
    args = ap.parse_args(argv)
    validate(args, ap)
    try:
        return run(args)
    except (ValueError, RuntimeError, FileNotFoundError) as err:
        print(f"error: {err}", file=sys.stderr)
        return 1


def run(args) -> int:
    import celeg_amd  # noqa: F401
    from celeg_amd.engine import Engine, RequestOptions, read_model_folder
    from celeg_amd.engine.benchmark import DecodeBench, measure_prefill, random_prompt
    from celeg_amd.sampling import GenerationConfig
    from celeg_amd.weights import write_random_model

    tmp = None
    model_dir = args.model
    if args.random_weights is not None:
        with open(args.random_weights) as fh:
            cfg = json.load(fh)
        tmp = tempfile.TemporaryDirectory(prefix="celeg_random_")
        model_dir = write_random_model(cfg, tmp.name, args.random_weights_seed)
    config, spec = read_model_folder(model_dir)
    if args.print_config:
        typed = config if isinstance(config, dict) else vars(config)
        print(json.dumps({"architecture": spec.architecture,
                          "config": {k: (list(v) if isinstance(v, tuple) else v) for k, v in typed.items()},
                          "layers": [layer.mixer.kind for layer in spec.layers],
                          "feed_forward_width": typed.get("ff_dim")}, indent=1))
        return 0
    context = min(4096, spec.max_context) if args.context is None else args.context
    if context > spec.max_context:
        raise ValueError(f"--context exceeds model maximum {spec.max_context}")

    # the prompt
    if args.prompt is not None:
        prompt = parse_token_ids(args.prompt)
    elif args.prompt_file is not None:
        with open(args.prompt_file) as fh:
            prompt = parse_token_ids(fh.read())
    elif args.random_prompt > 0:
        prompt = random_prompt(spec.vocab_size, args.random_prompt, args.seed)
    else:
        prompt = [spec.bos_token_id or 0]
    if args.benchmark_prefill_tokens > 0:
        # pad with the last token or cut, as src/app/cuda/main.cpp:368-376
        n = args.benchmark_prefill_tokens
        prompt = prompt[:n] + [prompt[-1]] * max(0, n - len(prompt))
    if not prompt:
        raise ValueError("request prompt is empty")
    if args.tokens_only:
        print(" ".join(str(t) for t in prompt))
        return 0
    new_tokens = args.benchmark_decode + args.benchmark_warmup + 2 if args.benchmark_decode > 0 else args.max_new_tokens
    if len(prompt) + new_tokens > context:
        raise ValueError("prompt plus output exceeds --context")

    batch = args.batch if args.benchmark_decode > 0 else 1
    budget = args.max_batched_tokens or max(512, args.prefill_chunk)
    if args.benchmark_prefill_tokens > 0:
        budget = max(budget, args.benchmark_prefill_tokens)
    pages_per_request = (context + args.page_tokens - 1) // args.page_tokens
    if args.dump_hidden:
        os.environ["CELEG_DUMP_HIDDEN"] = args.dump_hidden      # read by the library when it loads the model
    engine = Engine.from_folder(model_dir, dtype=args.dtype, device=args.device, page_tokens=args.page_tokens,
                                n_pages=args.pages or pages_per_request * max(batch, args.max_requests, 1), max_active_requests=max(batch, args.max_requests, 1),
                                context=context, max_batched_tokens=budget,
                                prefill_chunk_tokens=min(args.prefill_chunk, budget),
                                gemm_backend=args.gemm_backend, use_graphs=not args.no_graph,
                                strict_weights=args.strict_weights)
    lm = engine.loaded
    if args.profile:
        lm.native.time_phases(True)
    if args.attention_mode != "auto":
        lm.set_knob("attention_decode_whole", 1 if args.attention_mode == "single" else 0)
    if args.attention_chunk_tokens:
        # parts of 1, 4 or 16 rounds of 64 keys: the two bounds on the context's rounds choose
        big = 1 << 30
        few, some = {64: (big, big), 256: (0, big), 1024: (0, 0)}[args.attention_chunk_tokens]
        lm.set_knob("decode_parts_few", few)
        lm.set_knob("decode_parts_some", some)

    if args.benchmark_decode > 0:
        if args.benchmark_prefill_tokens > 0:
            p = measure_prefill(lm, len(prompt))
            print(f"benchmark.prefill_tokens={p['tokens']}\nbenchmark.prefill_ms={p['ms']:.3f}\n"
                  f"benchmark.prefill_tokens_per_second={p['tokens_per_second']:.3f}",
                  file=sys.stderr)
        bench = DecodeBench(engine, batch, len(prompt), new_tokens, seed=args.seed)
        d = bench.run(args.benchmark_decode, args.benchmark_warmup)
        bench.close()
        print(f"benchmark.decode_warmup={args.benchmark_warmup}\n"
              f"benchmark.decode_tokens={d['tokens']}\n"
              f"benchmark.decode_ms={d['ms_per_step'] * d['steps']:.3f}\n"
              f"benchmark.decode_ms_per_token={d['ms_per_step'] / batch:.4f}\n"
              f"benchmark.decode_tokens_per_second={d['tokens_per_second']:.3f}", file=sys.stderr)
        _reports(args, engine)
        return 0

    generation = GenerationConfig(temperature=args.temperature, top_k=args.top_k, top_p=args.top_p,
                                  repetition_penalty=args.repetition_penalty, seed=args.seed)
    rid = engine.submit(prompt, RequestOptions(max_new_tokens=max(args.max_new_tokens, 1),
                                               generation=generation))
    generated: List[int] = []
    first = True
    while engine.has_work():
        engine.step()
        status, tokens, error = engine.poll(rid)
        if tokens and first:
            first = False
            if args.dump_logits or args.print_top > 0:
                logits = engine.last_logits[0].numpy().astype("<f4")
                if args.dump_logits:
                    with open(args.dump_logits, "wb") as fh:
                        fh.write(logits.tobytes())
                if args.print_top > 0:
                    order = sorted(range(len(logits)), key=lambda t: (-float(logits[t]), t))
                    for i, t in enumerate(order[:args.print_top]):
                        print(f"top[{i}] token={t} logit={float(logits[t]):g}", file=sys.stderr)
            if args.max_new_tokens == 0:
                engine.cancel(rid)
                tokens = []
        for t in tokens:
            generated.append(t)
            print(t, end=" ", flush=True)
        if error:
            raise RuntimeError(error)
    print()
    if args.runtime_tokens:
        print("CELEG_GENERATED_TOKEN_IDS=[" + ",".join(str(t) for t in generated) + "]")
    _reports(args, engine, rid)
    if tmp is not None:
        tmp.cleanup()
    return 0


def _reports(args, engine, request_id=None) -> None:
    """--memory-report and --runtime-metrics, in the reference's ``key=value`` lines on stderr."""
    m = engine.metrics
    if args.profile:
        times = engine.loaded.native.phase_times() or {"steps": 0, "phases": {}}
        steps = max(times["steps"], 1)
        total = sum(p["ms"] for p in times["phases"].values()) or 1.0
        for name, p in times["phases"].items():
            print(f"profile.{name.replace(' ', '_')}_ms_per_step={p['ms'] / steps:.4f} ({100 * p['ms'] / total:.1f}%)",
                  file=sys.stderr)
        print(f"profile.steps={times['steps']}\nprofile.ms_per_step={total / steps:.4f}", file=sys.stderr)
    if args.memory_report:
        info = engine.loaded.native.info
        weights = info["weights"] * (2 if info["dtype"] == "bfloat16" else 4)
        for key, value in (("weights", weights), ("kv_cache", m["cache"]["kv_cache"]),
                           ("conv_state", m["cache"]["state"]), ("activations", m["workspace_bytes"])):
            print(f"memory.{key}={value}", file=sys.stderr)
    if args.runtime_metrics:
        s = m["scheduler"]
        print(f"runtime.prefill_tokens={s['prefill_tokens']}\nruntime.decode_tokens={s['decode_tokens']}\n"
              f"runtime.steps={s['steps']}\nruntime.seconds={m['step_seconds']:.4f}\n"
              f"runtime.graph_replays={m['graph_replays']}", file=sys.stderr)
        if request_id is not None:
            r = engine.request_metrics(request_id)
            for key in ("ttft_seconds", "itl_mean_seconds", "itl_max_seconds"):
                if r.get(key) is not None:
                    print(f"runtime.{key}={r[key]:.6f}", file=sys.stderr)


if __name__ == "__main__":
    sys.exit(main())

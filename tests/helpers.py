"""Shared helpers of the tests: tolerances (fixed here once), trace building, and a
client for ``bin/trace_run``."""
from __future__ import annotations

import json
import os
import subprocess
import sys
from typing import Dict, List, Sequence

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRACE_RUN = os.path.join(ROOT, "bin", "trace_run")

# Random test weights are N(0, WEIGHT_STD): wide enough that attention scores and gates
# move the logits, so that a fault shows above rounding.
WEIGHT_STD = 0.05


def assert_close_f32(got, ref, what=""):
    """32-bit engine against the plain implementation (float64):
    max |d| <= 1e-4 * max(1, max |ref|)."""
    got = torch.as_tensor(got).double()
    ref = torch.as_tensor(ref).double()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    bound = 1e-4 * max(1.0, float(ref.abs().max()))
    err = float((got - ref).abs().max())
    if err > bound:
        bad = int((got - ref).abs().max(dim=-1).values.argmax()) if got.dim() > 1 else 0
        raise AssertionError(f"{what}: max |d| {err:.3e} > {bound:.3e}; worst row {bad}")


def assert_close_bf16(got, ref, what=""):
    """bfloat16 engine against the plain implementation run on the same (bfloat16-stored)
    weights: relative RMS error <= 2.5e-2 and max |d| <= 4e-2 * max |ref|, about three
    times the rounding noise measured for these tiny models at WEIGHT_STD."""
    got = torch.as_tensor(got).double()
    ref = torch.as_tensor(ref).double()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite logits"
    d = got - ref
    rel = float(d.pow(2).mean().sqrt() / ref.pow(2).mean().sqrt())
    mx = float(d.abs().max() / ref.abs().max())
    if rel > 2.5e-2 or mx > 4e-2:
        bad = int(d.abs().max(dim=-1).values.argmax()) if got.dim() > 1 else 0
        raise AssertionError(f"{what}: rel rms {rel:.3e} (<= 2.5e-2), max/|ref|max {mx:.3e} "
                             f"(<= 4e-2); worst row {bad}")


def assert_close(got, ref, dtype, what=""):
    if dtype in ("float32", torch.float32):
        assert_close_f32(got, ref, what)
    else:
        assert_close_bf16(got, ref, what)


def random_tokens(vocab: int, n: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def round_up(n: int, m: int) -> int:
    return (n + m - 1) // m * m


class TraceClient:
    """Runs ``bin/trace_run`` and feeds it steps one at a time, waiting for ``done``."""

    def __init__(self, model_dir: str, dtype: str, out_dir: str, max_tokens: int,
                 extra: Sequence[str] = ()):
        self.out_dir = out_dir
        self.proc = subprocess.Popen(
            [sys.executable, TRACE_RUN, "--model", model_dir, "--dtype", dtype, "--out", out_dir,
             "--max-tokens", str(max_tokens), *extra],
            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
        self.vocab = None

    def step(self, number: int, entries, end=()):
        line = json.dumps({"step": number, "entries": entries, "end": list(end)})
        self.proc.stdin.write(line + "\n")
        self.proc.stdin.flush()
        answer = self.proc.stdout.readline().strip()
        if answer != f"done {number}":
            self.proc.stdin.close()
            code = self.proc.wait()
            raise RuntimeError(f"trace_run answered {answer!r} to step {number} (exit {code})")
        wanted = sum(len(e.get("want", [])) for e in entries)
        if not wanted:
            return None
        data = np.fromfile(os.path.join(self.out_dir, f"{number}.f32"), dtype="<f4")
        return torch.from_numpy(data.reshape(wanted, -1).copy())

    def close(self) -> int:
        self.proc.stdin.close()
        return self.proc.wait()


# ------------------------------------------------------------------ schedules

def whole_schedule(requests: Dict[str, List[int]]):
    """Each request alone and whole, one step each."""
    return [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
             "end": [rid]} for i, (rid, toks) in enumerate(requests.items())]


def tail_decode_schedule(requests: Dict[str, List[int]], tail: int = 32):
    """Most of a request in one step, then its last ``tail`` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = len(toks) - tail
        assert head >= 1
        steps.append({"step": len(steps), "entries": [
            {"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": toks[i:i + 1], "want": [0]}],
                "end": [rid] if i == len(toks) - 1 else []})
    return steps


def portions_schedule(requests: Dict[str, List[int]], sizes=(7, 2, 13, 2, 5, 3, 2, 16, 1, 11, 4)):
    """Portions of changing size, down to two tokens (and single ones)."""
    steps = []
    for k, (rid, toks) in enumerate(requests.items()):
        pos, i = 0, k  # each request starts at another place of the size list
        while pos < len(toks):
            n = min(sizes[i % len(sizes)], len(toks) - pos)
            i += 1
            steps.append({"step": len(steps), "entries": [
                {"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))}],
                "end": [rid] if pos + n == len(toks) else []})
            pos += n
    return steps


def mixed_schedule(requests: Dict[str, List[int]], max_live: int = 4, seed: int = 0,
                   decode_tail: int = 12):
    """Up to ``max_live`` requests at a time: portions of some beside single decoded
    tokens of others, a request now and then left out of a step, new requests admitted
    as others end (so their pages and slots are used again)."""
    rng = np.random.RandomState(seed)
    waiting = list(requests.items())
    live: Dict[str, int] = {}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, end = [], []
        ids = list(live)
        for rid in ids:
            toks = requests[rid]
            pos = live[rid]
            if len(ids) > 1 and rng.rand() < 0.2:
                continue  # left out of this step
            if pos >= len(toks) - decode_tail:
                n = 1
            else:
                n = int(min(rng.choice([2, 3, 5, 8, 13, 21]), len(toks) - decode_tail - pos))
            entries.append({"id": rid, "tokens": toks[pos:pos + n], "want": list(range(n))})
            live[rid] = pos + n
            if pos + n == len(toks):
                end.append(rid)
                del live[rid]
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    return steps


def peak_tokens(steps, page_round: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to 64."""
    held: Dict[str, int] = {}
    peak = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(round_up(n, page_round) for n in held.values()))
        for rid in s["end"]:
            del held[rid]
    return peak


class EngineDriver:
    """Drives the framework's step function and cache manager over a schedule, as
    ``bin/trace_run`` does, in this process.  Returns {request id: [logits per position]}."""

    def __init__(self, loaded):
        self.lm = loaded
        self.live = {}

    def run(self, steps):
        from celeg_amd.engine import StepEntry
        out: Dict[str, List[torch.Tensor]] = {}
        for s in steps:
            entries = []
            for e in s["entries"]:
                rid = e["id"]
                if rid not in self.live:
                    slot = self.lm.cache.open()
                    assert slot is not None, "no free slot"
                    self.live[rid] = [slot, 0]
                slot, seen = self.live[rid]
                assert self.lm.cache.prepare(slot, seen, len(e["tokens"])), "out of pages"
                entries.append(StepEntry(slot, seen, e["tokens"], e["want"]))
                self.live[rid][1] = seen + len(e["tokens"])
            logits = self.lm.runner.step(entries).detach().to("cpu").clone()
            row = 0
            for e in s["entries"]:
                for _ in e["want"]:
                    out.setdefault(e["id"], []).append(logits[row])
                    row += 1
            for rid in s["end"]:
                self.lm.cache.close(self.live.pop(rid)[0])
            self.lm.cache.check()
        return {rid: torch.stack(rows) for rid, rows in out.items()}


def reordered_lfm2():
    """An architecture registered from the tests: LFM2's parts under the run order that the
    configuration's "run_order" gives ([layer, kv_from or None] pairs)."""
    import dataclasses
    from celeg_amd.config import RunStep, register_architecture, registered_architectures, spec_from_config
    if "Lfm2Reordered" in registered_architectures():
        return

    def build(cfg, shapes):
        _, spec = spec_from_config(dict(cfg, architectures=["Lfm2ForCausalLM"]), shapes)
        order = tuple(RunStep(layer, kv_from) for layer, kv_from in cfg["run_order"])
        return dataclasses.replace(spec, architecture="Lfm2Reordered", order=order)
    register_architecture("Lfm2Reordered", build)

"""Each part of a layer alone against its plain function, and the generality of the
assembly: toy parts defined here (a mixer with state of its own, a feed-forward with routing,
another position encoding) and toy architectures are registered through the library's
interface, built and stepped without touching the framework's files; a run order that names a
layer twice and lets a layer read another layer's cache.

A part runs alone inside a block whose other parts are the neutral ones ("identity" norm,
"none" mixer or feed-forward) under the head "hidden", which gives the rows of the stream
back: with the inputs as the embedding table and the tokens 0..T-1 the step returns
x + part(x), cut into steps like any other model.
"""
import json
import os

import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY
from helpers import (WEIGHT_STD, EngineDriver, assert_close_f32, portions_schedule, random_tokens,
                     reordered_lfm2)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def write_folder(folder, cfg, replace=None, seed=0, std=0.2):
    """A model folder of random 32-bit tensors for ``cfg`` (what the library says the model
    wants), some of them replaced."""
    from celeg_amd import native
    from celeg_amd.weights import random_tensors
    from celeg_amd.weights.safetensors_io import write_safetensors
    expected = native.describe_config(cfg)["expected_tensors"]
    tensors = random_tensors(expected, seed, std, torch.float32)
    for name, t in (replace or {}).items():
        assert tensors[name].shape == t.shape
        tensors[name] = t.float().contiguous()
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(cfg, fh)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder, tensors


def parts_alone_architecture():
    """"PartsAlone": one block of the parts that the configuration spells out, neutral ones
    where it says nothing; the embedding table is the input, the head returns the stream."""
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    if "PartsAlone" in registered_architectures():
        return

    def build(cfg, shapes):
        H, rows = cfg["width"], cfg["rows"]
        part = lambda key, neutral: PartSpec.from_json(cfg[key]) if cfg.get(key) else neutral
        layer = LayerSpec(part("mixer", PartSpec("none", {"width": H})), part("mixer_norm", PartSpec("identity")),
                          part("ffn", PartSpec("none")), part("ffn_norm", PartSpec("identity")))
        return ModelSpec("PartsAlone", rows, H, 256, PartSpec("embedding", {"vocab": rows, "width": H}, {"table": "x"}),
                         (layer,), (RunStep(0),), part("final_norm", PartSpec("identity")),
                         PartSpec("hidden", {"width": H}))
    register_architecture("PartsAlone", build)


def run_part_alone(tmp_path, x, cuts, **parts):
    """x + part(x) (or norm(x)) for the rows of x fed in steps of ``cuts`` rows, and the
    folder's tensors."""
    from celeg_amd.engine import StepEntry, load_model
    parts_alone_architecture()
    cfg = {"architectures": ["PartsAlone"], "width": x.shape[1], "rows": x.shape[0]}
    cfg.update({k: v.to_json() for k, v in parts.items()})
    folder, tensors = write_folder(str(tmp_path / "alone"), cfg, {"x": x})
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=16, max_requests=2, max_batched_tokens=64)
    slot = lm.cache.open()
    outs, pos = [], 0
    for n in cuts:
        assert lm.cache.prepare(slot, pos, n)
        outs.append(lm.runner.step([StepEntry(slot, pos, list(range(pos, pos + n)), list(range(n)))]))
        pos += n
    lm.cache.close(slot)
    lm.cache.check()
    lm.close()
    return torch.cat(outs).double(), tensors


def test_short_conv_mixer_alone(tmp_path):
    from celeg_amd.config import PartSpec
    names = {"in_proj": "conv.in_proj.weight", "in_proj_bias": "conv.in_proj.bias", "conv": "conv.conv.weight",
             "conv_bias": "conv.conv.bias", "out_proj": "conv.out_proj.weight", "out_proj_bias": "conv.out_proj.bias"}
    spec = PartSpec("short_conv", {"width": 40, "taps": 4, "bias": True}, names)
    x = torch.randn(29, 40, generator=torch.Generator().manual_seed(1))
    for i, cuts in enumerate(([29], [5, 1, 2, 21])):
        got, W = run_part_alone(tmp_path / str(i), x, cuts, mixer=spec)
        ref = plain.conv_mixer(x, W, "", True)
        torch.testing.assert_close(got - x.double(), ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("window", [None, 7])
def test_attention_mixer_alone(tmp_path, window):
    from celeg_amd.config import PartSpec
    cfg = {"num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 16, "norm_eps": 1e-5, "rope_theta": 1e4}
    names = {"q_proj": "self_attn.q_proj.weight", "k_proj": "self_attn.k_proj.weight", "v_proj": "self_attn.v_proj.weight",
             "out_proj": "self_attn.out_proj.weight", "q_norm": "self_attn.q_layernorm.weight",
             "k_norm": "self_attn.k_layernorm.weight"}
    spec = PartSpec("gqa_attention", {
        "width": 40, "heads": 6, "kv_heads": 2, "head_dim": 16, "qk_norm": True, "eps": 1e-5,
        "window": window, "position": PartSpec("rope", {"theta": 1e4, "head_dim": 16})}, names)
    x = torch.randn(37, 40, generator=torch.Generator().manual_seed(2))
    for i, cuts in enumerate(([37], [9, 1, 1, 20, 6])):
        got, W = run_part_alone(tmp_path / str(i), x, cuts, mixer=spec)
        ref, _ = plain.attention_mixer(x, W, "", cfg, list(range(37)), window=window)
        torch.testing.assert_close(got - x.double(), ref, rtol=1e-4, atol=1e-5)


def test_attention_without_norm_or_rotation_is_library_attention(tmp_path):
    import torch.nn.functional as F
    from celeg_amd.config import PartSpec
    spec = PartSpec("gqa_attention", {"width": 32, "heads": 2, "kv_heads": 2, "head_dim": 16, "qk_norm": False,
                                      "position": PartSpec("none")},
                    {"q_proj": "q", "k_proj": "k", "v_proj": "v", "out_proj": "o"})
    x = torch.randn(21, 32, generator=torch.Generator().manual_seed(3))
    got, W = run_part_alone(tmp_path, x, [4, 17], mixer=spec)
    xd = x.double()
    q, k, v = (F.linear(xd, W[n].double()).reshape(21, 2, 16).transpose(0, 1)[None] for n in ("q", "k", "v"))
    att = F.scaled_dot_product_attention(q, k, v, is_causal=True)[0].transpose(0, 1).reshape(21, 32)
    ref = F.linear(att, W["o"].double())
    torch.testing.assert_close(got - xd, ref, rtol=1e-4, atol=1e-5)


def test_feed_forward_and_norm_alone(tmp_path):
    from celeg_amd.config import PartSpec
    x = torch.randn(9, 24, generator=torch.Generator().manual_seed(4))
    ffn = PartSpec("swiglu", {"width": 24, "ff": 50}, {"gate": "g", "up": "u", "down": "d"})
    got, W = run_part_alone(tmp_path / "ffn", x, [9], ffn=ffn)
    ref = plain.swiglu_ffn(x, W["g"], W["u"], W["d"])
    torch.testing.assert_close(got - x.double(), ref, rtol=1e-4, atol=1e-5)
    norm = PartSpec("rmsnorm", {"width": 24, "eps": 1e-3}, {"weight": "w"})
    got, W = run_part_alone(tmp_path / "norm", x, [4, 5], final_norm=norm)
    torch.testing.assert_close(got, plain.rmsnorm(x, W["w"], 1e-3), rtol=1e-5, atol=1e-6)
    # the norm in front of a part: the feed-forward of the normalised rows, added to the rows
    got, W = run_part_alone(tmp_path / "both", x, [3, 6], ffn=ffn, ffn_norm=norm)
    ref = x.double() + plain.swiglu_ffn(plain.rmsnorm(x, W["w"], 1e-3), W["g"], W["u"], W["d"])
    torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------- a toy mixer and architecture
def register_toy():
    """A mixer whose state is its own: the running sum of its inputs and their count.
    out[t] = (sum of x[0..t]) / (t+1) @ W^T.  It is written with torch (a toy may be), on the
    memory the library hands it, and plans on the host from the step's host arrays."""
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    from celeg_amd.parts import as_tensor, on_stream, register_part, registered_parts

    class RunningMean:
        def __init__(self, spec):
            self.width = int(spec["params"]["width"])
            self.w = None

        def describe(self):
            return {"weights": {"proj": {"shape": [self.width, self.width]}},
                    "states": [{"name": "sum", "shape": [self.width], "dtype": "float32"},
                               {"name": "count", "shape": [1], "dtype": "float32"}],
                    "graph_safe": False, "out_width": self.width}

        def load(self, tensors):
            self.w = as_tensor(tensors["proj"])

        def forward(self, args):
            with on_stream(args):
                x, out = as_tensor(args.x), as_tensor(args.out)
                states = {args.cache.state_names[i].decode(): as_tensor(args.cache.states[i])
                          for i in range(args.cache.n_states)}
                total, count = states["sum"], states["count"]
                step = args.step
                for s in range(step.n_seqs):
                    slot, lo, hi = step.host_seq_slot[s], step.host_cu_seqlens[s], step.host_cu_seqlens[s + 1]
                    rows = x[lo:hi].float()
                    running = total[slot] + torch.cumsum(rows, dim=0)
                    n = count[slot] + torch.arange(1, rows.shape[0] + 1, device=x.device)[:, None]
                    out[lo:hi] = ((running / n) @ self.w.float().t()).to(out.dtype)
                    total[slot] = running[-1]
                    count[slot] = n[-1]

    if "running_mean" not in registered_parts("mixer"):
        register_part("mixer", "running_mean", RunningMean)

    def build_spec(cfg, shapes):
        H = cfg["width"]
        norm = lambda name: PartSpec("rmsnorm", {"width": H, "eps": 1e-5}, {"weight": name})
        layers = []
        for i, kind in enumerate(cfg["layers"]):
            p = f"blocks.{i}."
            if kind == "mean":
                mixer = PartSpec("running_mean", {"width": H}, {"proj": p + "mean.proj"})
            else:
                mixer = PartSpec("gqa_attention",
                                 {"width": H, "heads": 2, "kv_heads": 1, "head_dim": 16,
                                  "qk_norm": False, "position": PartSpec("rope", {"theta": 100.0, "head_dim": 16})},
                                 {"q_proj": p + "att.q", "k_proj": p + "att.k", "v_proj": p + "att.v",
                                  "out_proj": p + "att.o"})
            layers.append(LayerSpec(mixer, norm(p + "n1"),
                                    PartSpec("swiglu", {"width": H, "ff": 2 * H},
                                             {"gate": p + "ff.g", "up": p + "ff.u", "down": p + "ff.d"}),
                                    norm(p + "n2")))
        return ModelSpec("ToyForCausalLM", cfg["vocab"], H, 128,
                         PartSpec("embedding", {"vocab": cfg["vocab"], "width": H}, {"table": "emb"}),
                         tuple(layers), tuple(RunStep(i) for i in range(len(layers))),
                         norm("final"), PartSpec("tied_head", {"vocab": cfg["vocab"], "width": H}))

    if "ToyForCausalLM" not in registered_architectures():
        register_architecture("ToyForCausalLM", build_spec)


def toy_plain_logits(cfg, W, tokens):
    """Whole-sequence reference of the toy model, from the plain parts."""
    h = plain.embedding(W["emb"], tokens)
    T = len(tokens)
    for i, kind in enumerate(cfg["layers"]):
        p = f"blocks.{i}."
        n = plain.rmsnorm(h, W[p + "n1"], 1e-5)
        if kind == "mean":
            mean = torch.cumsum(n, dim=0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None]
            m = plain.linear(mean, W[p + "mean.proj"])
        else:
            q = plain.linear(n, W[p + "att.q"]).reshape(T, 2, 16)
            k = plain.linear(n, W[p + "att.k"]).reshape(T, 1, 16)
            v = plain.linear(n, W[p + "att.v"]).reshape(T, 1, 16)
            cos, sin = plain.rope_cos_sin(range(T), 100.0, 16)
            o = plain.causal_attention(plain.rope_apply(q, cos, sin), plain.rope_apply(k, cos, sin), v)
            m = plain.linear(o.reshape(T, -1), W[p + "att.o"])
        h = h + m
        h = h + plain.swiglu_ffn(plain.rmsnorm(h, W[p + "n2"], 1e-5), W[p + "ff.g"], W[p + "ff.u"], W[p + "ff.d"])
    return plain.linear(plain.rmsnorm(h, W["final"], 1e-5), W["emb"])


def test_toy_mixer_with_its_own_state_is_registered_built_and_stepped(tmp_path):
    from celeg_amd.engine import load_model
    from celeg_amd.weights import write_random_model
    register_toy()
    cfg = {"architectures": ["ToyForCausalLM"], "width": 32, "vocab": 77,
           "layers": ["mean", "attention", "mean"]}
    folder = write_random_model(cfg, str(tmp_path / "toy"), seed=4, dtype=torch.float32, std=0.2)
    _, W = plain.load_model_folder(folder)
    reqs = {"x": random_tokens(77, 45, 1), "y": random_tokens(77, 30, 2)}
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=8, max_requests=2,
                    max_batched_tokens=64)
    assert [s["name"] for s in lm.cache.layout["states"]] == ["sum", "count", "sum", "count"]
    assert not lm.graph_safe      # the toy plans on the host: its steps are never replayed
    got = EngineDriver(lm).run(portions_schedule(reqs))
    # the slots are used again by other requests: a new request starts from zeroed state
    got2 = EngineDriver(lm).run(portions_schedule(dict(reversed(list(reqs.items())))))
    for rid, toks in reqs.items():
        ref = toy_plain_logits(cfg, W, toks)
        assert_close_f32(got[rid], ref, f"toy/{rid}")
        assert_close_f32(got2[rid], ref, f"toy again/{rid}")
    assert lm.runner.counters()["graph_replays"] == 0


def test_toy_model_generates_through_the_engine(tmp_path):
    """The same toy model under the scheduler and the sampler: greedy tokens equal the plain ones."""
    from celeg_amd.engine import Engine
    from celeg_amd.sampling import GREEDY
    from celeg_amd.weights import write_random_model
    register_toy()
    cfg = {"architectures": ["ToyForCausalLM"], "width": 32, "vocab": 77, "layers": ["attention", "mean"]}
    folder = write_random_model(cfg, str(tmp_path / "toy"), seed=6, dtype=torch.float32, std=0.2)
    _, W = plain.load_model_folder(folder)
    prompts = [random_tokens(77, n, 10 + n) for n in (3, 19, 8)]
    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=2, n_pages=8, max_batched_tokens=16,
                                prefill_chunk_tokens=8)
    outs = engine.generate(prompts, max_new_tokens=6, generation=GREEDY, eos_token_ids=[])
    for prompt, out in zip(prompts, outs):
        seq = list(prompt)
        for _ in range(6):
            seq.append(int(toy_plain_logits(cfg, W, seq)[-1].argmax()))
        assert out == seq[len(prompt):]


# ---------------------------------------------------------------- a toy routed feed-forward and position encoding
def register_toy_routed():
    """A feed-forward that routes every token to the one expert its router scores highest
    (SwiGLU experts, the router's score in 32-bit, written with torch), and a rotary
    encoding whose frequencies are the usual ones divided by a factor (positions stretched).
    Both are registered here, from outside the framework, with an architecture that mixes
    routed and dense layers."""
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    from celeg_amd.parts import as_tensor, on_stream, register_part, registered_parts

    class TopOneExperts:
        def __init__(self, spec):
            p = spec["params"]
            self.width, self.ff, self.experts = int(p["width"]), int(p["ff"]), int(p["experts"])

        def describe(self):
            weights = {"router": {"shape": [self.experts, self.width]}}
            for e in range(self.experts):
                weights[f"gate{e}"] = {"shape": [self.ff, self.width]}
                weights[f"up{e}"] = {"shape": [self.ff, self.width]}
                weights[f"down{e}"] = {"shape": [self.width, self.ff]}
            return {"weights": weights, "graph_safe": False, "out_width": self.width}

        def load(self, tensors):
            self.w = {role: as_tensor(view) for role, view in tensors.items()}

        def forward(self, args):
            with on_stream(args):
                x, out = as_tensor(args.x), as_tensor(args.out)
                xf = x.float()
                choice = (xf @ self.w["router"].float().t()).argmax(dim=1)
                for e in range(self.experts):
                    rows = (choice == e).nonzero().flatten()
                    if rows.numel() == 0:
                        continue
                    xe = xf[rows]
                    act = torch.nn.functional.silu(xe @ self.w[f"gate{e}"].float().t()) * (xe @ self.w[f"up{e}"].float().t())
                    out[rows] = (act @ self.w[f"down{e}"].float().t()).to(out.dtype)

    class StretchedRope:
        def __init__(self, spec):
            p = spec["params"]
            self.theta, self.factor, self.rotary_dim = float(p["theta"]), float(p["factor"]), int(p["rotary_dim"])

        def describe(self):
            return {"inv_freq": [self.theta ** (-2.0 * i / self.rotary_dim) / self.factor
                                 for i in range(self.rotary_dim // 2)], "rotary_dim": self.rotary_dim}

        def forward(self, args):
            raise RuntimeError("a position encoding gives tables; it is never called")

    if "toy_top_one" not in registered_parts("ffn"):
        register_part("ffn", "toy_top_one", TopOneExperts)
    if "toy_stretched_rope" not in registered_parts("position"):
        register_part("position", "toy_stretched_rope", StretchedRope)

    def build_spec(cfg, shapes):
        H, ff, E = cfg["width"], cfg["ff"], cfg["experts"]
        norm = lambda name: PartSpec("rmsnorm", {"width": H, "eps": 1e-5}, {"weight": name})
        layers = []
        for i, kind in enumerate(cfg["layers"]):
            p = f"blocks.{i}."
            mixer = PartSpec("gqa_attention",
                             {"width": H, "heads": 3, "kv_heads": 1, "head_dim": 16, "qk_norm": False,
                              "position": PartSpec("toy_stretched_rope",
                                                   {"theta": 50.0, "factor": cfg["stretch"], "rotary_dim": 8})},
                             {"q_proj": p + "att.q", "k_proj": p + "att.k", "v_proj": p + "att.v",
                              "out_proj": p + "att.o"})
            if kind == "routed":
                names = {"router": p + "router"}
                for e in range(E):
                    names.update({f"gate{e}": p + f"e{e}.g", f"up{e}": p + f"e{e}.u", f"down{e}": p + f"e{e}.d"})
                ffn = PartSpec("toy_top_one", {"width": H, "ff": ff, "experts": E}, names)
            else:
                ffn = PartSpec("swiglu", {"width": H, "ff": ff},
                               {"gate": p + "ff.g", "up": p + "ff.u", "down": p + "ff.d"})
            layers.append(LayerSpec(mixer, norm(p + "n1"), ffn, norm(p + "n2")))
        return ModelSpec("ToyRoutedForCausalLM", cfg["vocab"], H, 128,
                         PartSpec("embedding", {"vocab": cfg["vocab"], "width": H}, {"table": "emb"}),
                         tuple(layers), tuple(RunStep(i) for i in range(len(layers))),
                         norm("final"), PartSpec("tied_head", {"vocab": cfg["vocab"], "width": H}))

    if "ToyRoutedForCausalLM" not in registered_architectures():
        register_architecture("ToyRoutedForCausalLM", build_spec)


def toy_routed_plain_logits(cfg, W, tokens):
    """Whole-sequence reference of the routed toy model, from the plain parts; also the
    expert every token took in every routed layer."""
    h = plain.embedding(W["emb"], tokens)
    T = len(tokens)
    taken = []
    for i, kind in enumerate(cfg["layers"]):
        p = f"blocks.{i}."
        n = plain.rmsnorm(h, W[p + "n1"], 1e-5)
        q = plain.linear(n, W[p + "att.q"]).reshape(T, 3, 16)
        k = plain.linear(n, W[p + "att.k"]).reshape(T, 1, 16)
        v = plain.linear(n, W[p + "att.v"]).reshape(T, 1, 16)
        # stretched positions: the angle is position / factor times the usual frequency
        cos, sin = plain.rope_cos_sin([t / cfg["stretch"] for t in range(T)], 50.0, 8)
        o = plain.causal_attention(plain.rope_apply(q, cos, sin), plain.rope_apply(k, cos, sin), v)
        h = h + plain.linear(o.reshape(T, -1), W[p + "att.o"])
        n = plain.rmsnorm(h, W[p + "n2"], 1e-5)
        if kind == "routed":
            scores = plain.linear(n, W[p + "router"])
            choice = scores.argmax(dim=1)
            taken.append((choice, scores))
            out = torch.zeros_like(h)
            for t in range(T):
                e = int(choice[t])
                out[t] = plain.swiglu_ffn(n[t:t + 1], W[p + f"e{e}.g"], W[p + f"e{e}.u"], W[p + f"e{e}.d"])[0]
            h = h + out
        else:
            h = h + plain.swiglu_ffn(n, W[p + "ff.g"], W[p + "ff.u"], W[p + "ff.d"])
    return plain.linear(plain.rmsnorm(h, W["final"], 1e-5), W["emb"]), taken


def test_toy_routed_feed_forward_and_position_encoding_are_registered_and_stepped(tmp_path):
    """A feed-forward with routing and a position encoding of their own, registered from
    the test, in an architecture with routed and dense layers: portions of two requests
    against the plain whole-sequence reference.  Tokens whose two best router scores lie too
    close for 32-bit to tell apart are not compared (none is expected with these weights);
    every expert is taken by some token."""
    from celeg_amd.engine import load_model
    from celeg_amd.weights import write_random_model
    register_toy_routed()
    cfg = {"architectures": ["ToyRoutedForCausalLM"], "width": 48, "ff": 40, "experts": 3, "vocab": 91,
           "stretch": 4.0, "layers": ["routed", "dense", "routed"]}
    folder = write_random_model(cfg, str(tmp_path / "toy_routed"), seed=9, dtype=torch.float32, std=0.25)
    _, W = plain.load_model_folder(folder)
    reqs = {"x": random_tokens(91, 50, 3), "y": random_tokens(91, 37, 4)}
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=8, max_requests=2,
                    max_batched_tokens=64)
    got = EngineDriver(lm).run(portions_schedule(reqs))
    experts_seen = set()
    for rid, toks in reqs.items():
        ref, taken = toy_routed_plain_logits(cfg, W, toks)
        clear = torch.ones(len(toks), dtype=torch.bool)
        for choice, scores in taken:
            top2 = scores.topk(2, dim=1).values
            clear &= (top2[:, 0] - top2[:, 1]) > 1e-4
            experts_seen.update(choice.tolist())
        # a token routed the other way changes the rows after it too
        first_unclear = int((~clear).nonzero()[0]) if (~clear).any() else len(toks)
        assert first_unclear > len(toks) // 2, "the weights leave too few tokens with a clear choice"
        assert_close_f32(got[rid][:first_unclear], ref[:first_unclear], f"toy routed/{rid}")
    assert experts_seen == {0, 1, 2}
    # the stretch matters: the same weights with factor 1 give other logits
    toks = reqs["x"]
    other, _ = toy_routed_plain_logits(dict(cfg, stretch=1.0), W, toks)
    ref, _ = toy_routed_plain_logits(cfg, W, toks)
    assert (other - ref).abs().max() > 1e-3


def register_toy_that_fails():
    """A feed-forward that copies its input and refuses a step of more than ``limit`` rows, in a
    model of one block whose head gives the stream back: logits = 2 * embedding row."""
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    from celeg_amd.parts import as_tensor, on_stream, register_part, registered_parts

    class FailsOnManyRows:
        def __init__(self, spec):
            self.limit = int(spec["params"]["limit"])

        def describe(self):
            return {"graph_safe": False}

        def forward(self, args):
            if args.step.n_tokens > self.limit:
                raise RuntimeError("too many rows for this toy")
            with on_stream(args):
                as_tensor(args.out).copy_(as_tensor(args.x))

    if "toy_fails" not in registered_parts("ffn"):
        register_part("ffn", "toy_fails", FailsOnManyRows)

    def build(cfg, shapes):
        H, V = cfg["width"], cfg["vocab"]
        ident = PartSpec("identity")
        layer = LayerSpec(PartSpec("none", {"width": H}), ident, PartSpec("toy_fails", {"limit": cfg["limit"]}), ident)
        return ModelSpec("ToyFails", V, H, 64, PartSpec("embedding", {"vocab": V, "width": H}, {"table": "emb"}),
                         (layer,), (RunStep(0),), ident, PartSpec("hidden", {"width": H}))
    if "ToyFails" not in registered_architectures():
        register_architecture("ToyFails", build)


def test_a_part_that_fails_fails_the_step_and_nothing_else(tmp_path):
    """A part whose forward raises: the step is refused with the part's name, the request's
    slot can be closed, and the model steps other requests afterwards."""
    from celeg_amd.engine import StepEntry, load_model
    from celeg_amd.weights import write_random_model
    register_toy_that_fails()
    cfg = {"architectures": ["ToyFails"], "width": 16, "vocab": 20, "limit": 4}
    folder = write_random_model(cfg, str(tmp_path / "fails"), seed=1, dtype=torch.float32, std=0.5)
    _, W = plain.load_model_folder(folder)
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=4, max_requests=2, max_batched_tokens=32)
    a, b = lm.cache.open(), lm.cache.open()
    assert lm.cache.prepare(a, 0, 6) and lm.cache.prepare(b, 0, 3)
    with pytest.raises(ValueError, match="toy_fails"):
        lm.runner.step([StepEntry(a, 0, [1, 2, 3, 4, 5, 6], [5])])
    lm.cache.close(a)
    got = lm.runner.step([StepEntry(b, 0, [7, 8, 9], [0, 2])])
    ref = 2 * W["emb"][[7, 9]].double()
    torch.testing.assert_close(got.double(), ref, rtol=1e-6, atol=1e-6)
    lm.cache.close(b)
    lm.cache.check()
    assert lm.cache.n_free_slots == 2


def test_a_failed_step_fails_its_requests_and_the_engine_goes_on(tmp_path):
    """Through the engine: a request whose step fails ends FAILED with the message, gives its slot
    back, and requests before and after it finish with the right tokens
    (src/runtime/concurrency/request_lifecycle.cpp:200-218)."""
    from celeg_amd.engine import Engine, RequestOptions, RequestStatus
    from celeg_amd.sampling import GREEDY
    from celeg_amd.weights import write_random_model
    register_toy_that_fails()
    cfg = {"architectures": ["ToyFails"], "width": 16, "vocab": 20, "limit": 4}
    folder = write_random_model(cfg, str(tmp_path / "fails"), seed=1, dtype=torch.float32, std=0.5)
    _, W = plain.load_model_folder(folder)

    def plain_tokens(prompt, n):       # greedy over logits = 2 * embedding row of the last token
        seq = list(prompt)
        for _ in range(n):
            seq.append(int(W["emb"][seq[-1]].argmax()))
        return seq[len(prompt):]

    engine = Engine.from_folder(folder, dtype="float32", max_active_requests=2, n_pages=4, max_batched_tokens=8,
                                prefill_chunk_tokens=8)
    options = RequestOptions(max_new_tokens=5, eos_token_ids=[], generation=GREEDY)
    first = engine.submit([3, 1, 4], options)
    engine.run()
    assert engine.poll(first) == (RequestStatus.FINISHED, plain_tokens([3, 1, 4], 5), "")
    doomed = engine.submit([2, 7, 1, 8, 2, 8, 1], options)      # a portion of 7 rows: more than the toy takes
    engine.run()
    status, tokens, error = engine.poll(doomed)
    assert status == RequestStatus.FAILED and tokens == [] and "toy_fails" in error
    assert engine.metrics["failed_steps"] == 1
    assert engine.loaded.cache.n_free_slots == 2
    after = engine.submit([5, 9], options)
    beside = engine.submit([6], options)
    engine.run()
    assert engine.poll(after) == (RequestStatus.FINISHED, plain_tokens([5, 9], 5), "")
    assert engine.poll(beside) == (RequestStatus.FINISHED, plain_tokens([6], 5), "")
    assert engine.loaded.cache.n_free_slots == 2
    engine.loaded.cache.check()


def test_run_order_with_a_layer_twice_and_a_shared_cache(model_folders, tmp_path):
    """LFM2 parts under another run order: layer 1 runs twice (own cache each time) and
    layer 3 reads the keys and values the first run of layer 1 wrote."""
    from celeg_amd import native
    from celeg_amd.engine import load_model
    from celeg_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
    reordered_lfm2()
    source = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(source)
    config = dict(TINY["A"][0], architectures=["Lfm2Reordered"],
                  run_order=[[0, None], [1, None], [2, None], [1, None], [3, 1]])
    wanted = [e["name"] for e in native.describe_config(config)["expected_tensors"]]
    assert "model.layers.3.self_attn.k_proj.weight" not in wanted
    folder = str(tmp_path / "reordered")
    os.makedirs(folder)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh)
    f = SafetensorsFile(os.path.join(source, "model.safetensors"))
    write_safetensors(os.path.join(folder, "model.safetensors"), {n: f.tensor(n).clone() for n in wanted})
    f.close()
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=8, max_requests=2, max_context=128,
                    max_batched_tokens=64)
    reqs = {"a": random_tokens(256, 50, 8), "b": random_tokens(256, 37, 9)}
    got = EngineDriver(lm).run(portions_schedule(reqs))
    for rid, toks in reqs.items():
        ref = plain.model_logits(cfg, W, toks, order=[0, 1, 2, 1, 3], kv_from={4: 1})
        assert_close_f32(got[rid], ref, f"order/{rid}")

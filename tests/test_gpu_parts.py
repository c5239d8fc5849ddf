"""Each part of a layer alone against its plain function, and the generality of the
assembly: a toy mixer with state of its own and a toy architecture, defined here, are
registered, built and stepped without touching the framework's files; a run order that
names a layer twice and lets a layer read another layer's cache."""
import dataclasses
import os

import pytest
import torch

import plain_lfm2 as plain
from conftest import TINY
from helpers import WEIGHT_STD, EngineDriver, assert_close_f32, portions_schedule, random_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def runtime(dtype=torch.float32):
    from celeg_amd.engine import make_runtime
    return make_runtime(DEV, dtype)


def one_request_batch(rt, cache, slot, start, n):
    from celeg_amd.engine.batch import BatchBuilder
    from celeg_amd.engine import StepEntry
    assert cache.prepare(slot, start, n)
    builder = BatchBuilder(DEV, 1 << 14, len(cache.groups), pin=True)
    batch = builder.build([StepEntry(slot, start, [0] * n)], cache.drain_table_updates(),
                          null_slot=cache.null_slot)
    for g, (upd, cap) in enumerate(zip(batch.table_updates, batch.table_update_caps)):
        if cap:
            rt.ops.apply_table_updates(cache.groups[g].table, upd, cap)
    return batch


def build_mixer(spec, rt, seed=0):
    """A mixer alone: built from its PartSpec, random tensors, and a cache of its own."""
    from celeg_amd.cache import CacheLayout, CacheManager
    from celeg_amd.parts import build_part
    from celeg_amd.weights import random_tensor
    mixer = build_part("mixer", spec)
    tensors = {role: random_tensor(seed, role, w.shape, w.init, 0.2).to(DEV)
               for role, w in mixer.weight_specs().items()}
    mixer.load(dict(tensors), rt)
    layout = CacheLayout()
    if mixer.kv_need() is not None:
        layout.kv_groups, layout.group_layers = [mixer.kv_need()], [1]
        layout.kv_of_step = {0: (0, 0, True)}
    layout.states = [(0, s) for s in mixer.state_needs()]
    cache = CacheManager(layout, page_tokens=16, n_pages=16, max_requests=2, max_context=256,
                         device=DEV, dtype=rt.dtype)
    return mixer, tensors, cache


def run_mixer_in_cuts(mixer, cache, rt, x, cuts):
    slot = cache.open()
    outs, pos = [], 0
    for n in cuts:
        batch = one_request_batch(rt, cache, slot, pos, n)
        outs.append(mixer.forward(x[pos:pos + n].contiguous(), batch, cache.layer_cache(0), rt).clone())
        pos += n
    cache.close(slot)
    return torch.cat(outs).double().cpu()


def test_short_conv_mixer_alone():
    from celeg_amd.config import PartSpec
    rt = runtime()
    spec = PartSpec("short_conv", {"width": 40, "taps": 4, "bias": True})
    mixer, t, cache = build_mixer(spec, rt)
    x = torch.randn(29, 40, generator=torch.Generator().manual_seed(1)).to(DEV)
    W = {"conv.in_proj.weight": t["in_proj"], "conv.in_proj.bias": t["in_proj_bias"],
         "conv.conv.weight": t["conv"], "conv.conv.bias": t["conv_bias"],
         "conv.out_proj.weight": t["out_proj"], "conv.out_proj.bias": t["out_proj_bias"]}
    ref = plain.conv_mixer(x.cpu(), {k: v.cpu() for k, v in W.items()}, "", True)
    for cuts in ([29], [5, 1, 2, 21]):
        torch.testing.assert_close(run_mixer_in_cuts(mixer, cache, rt, x, cuts), ref, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("window", [None, 7])
def test_attention_mixer_alone(window):
    from celeg_amd.config import PartSpec
    rt = runtime()
    cfg = {"num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 16, "norm_eps": 1e-5,
           "rope_theta": 1e4}
    spec = PartSpec("gqa_attention", {
        "width": 40, "heads": 6, "kv_heads": 2, "head_dim": 16, "qk_norm": True, "eps": 1e-5,
        "window": window, "position": PartSpec("rope", {"theta": 1e4, "head_dim": 16})})
    mixer, t, cache = build_mixer(spec, rt)
    x = torch.randn(37, 40, generator=torch.Generator().manual_seed(2)).to(DEV)
    W = {"self_attn.q_proj.weight": t["q_proj"], "self_attn.k_proj.weight": t["k_proj"],
         "self_attn.v_proj.weight": t["v_proj"], "self_attn.out_proj.weight": t["out_proj"],
         "self_attn.q_layernorm.weight": t["q_norm"], "self_attn.k_layernorm.weight": t["k_norm"]}
    ref, _ = plain.attention_mixer(x.cpu(), {k: v.cpu() for k, v in W.items()}, "", cfg,
                                   list(range(37)), window=window)
    for cuts in ([37], [9, 1, 1, 20, 6]):
        torch.testing.assert_close(run_mixer_in_cuts(mixer, cache, rt, x, cuts), ref, rtol=1e-4, atol=1e-5)


def test_attention_without_norm_or_rotation_is_library_attention():
    import torch.nn.functional as F
    from celeg_amd.config import PartSpec
    rt = runtime()
    spec = PartSpec("gqa_attention", {"width": 32, "heads": 2, "kv_heads": 2, "head_dim": 16,
                                      "qk_norm": False, "position": PartSpec("none")})
    mixer, t, cache = build_mixer(spec, rt)
    x = torch.randn(21, 32, generator=torch.Generator().manual_seed(3)).to(DEV)
    xd = x.double().cpu()
    q, k, v = (F.linear(xd, t[n].double().cpu()).reshape(21, 2, 16).transpose(0, 1)[None]
               for n in ("q_proj", "k_proj", "v_proj"))
    att = F.scaled_dot_product_attention(q, k, v, is_causal=True)[0].transpose(0, 1).reshape(21, 32)
    ref = F.linear(att, t["out_proj"].double().cpu())
    torch.testing.assert_close(run_mixer_in_cuts(mixer, cache, rt, x, [4, 17]), ref, rtol=1e-4, atol=1e-5)


def test_feed_forward_and_norm_alone():
    from celeg_amd.config import PartSpec
    from celeg_amd.parts import build_part
    from celeg_amd.weights import random_tensor
    rt = runtime()
    ffn = build_part("ffn", PartSpec("swiglu", {"width": 24, "ff": 50}))
    t = {r: random_tensor(0, r, w.shape, w.init, 0.3).to(DEV) for r, w in ffn.weight_specs().items()}
    ffn.load(dict(t), rt)
    x = torch.randn(9, 24, generator=torch.Generator().manual_seed(4)).to(DEV)
    ref = plain.swiglu_ffn(x.cpu(), t["gate"].cpu(), t["up"].cpu(), t["down"].cpu())
    torch.testing.assert_close(ffn.forward(x, None, rt).double().cpu(), ref, rtol=1e-4, atol=1e-5)
    norm = build_part("norm", PartSpec("rmsnorm", {"width": 24, "eps": 1e-3}))
    w = (1 + 0.1 * torch.randn(24)).to(DEV)
    norm.load({"weight": w}, rt)
    out = torch.empty_like(x)
    norm.forward(x.clone(), out, rt)
    torch.testing.assert_close(out.double().cpu(), plain.rmsnorm(x.cpu(), w.cpu(), 1e-3), rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- a toy mixer and architecture
def register_toy():
    """A mixer whose state is its own: the running sum of its inputs and their count.
    out[t] = (sum of x[0..t]) / (t+1) @ W^T.  It is written with torch (a toy may be) and
    plans on the host from the batch's host arrays."""
    from celeg_amd.config import (Architecture, LayerSpec, ModelSpec, PartSpec, RunStep,
                                  register_architecture, registered_architectures)
    from celeg_amd.parts import Mixer, StateNeed, WeightSpec, register_part, registered_parts

    class RunningMean(Mixer):
        def __init__(self, spec):
            super().__init__(spec)
            self.width = int(self.params["width"])
            self.w = None

        def state_needs(self):
            return [StateNeed("sum", (self.width,), torch.float32),
                    StateNeed("count", (1,), torch.float32)]

        def weight_specs(self):
            return {"proj": WeightSpec((self.width, self.width))}

        def load(self, tensors, rt):
            self.w = tensors["proj"]

        def forward(self, x, batch, cache, rt):
            out = rt.ws.buf("toy_out", (x.shape[0], self.width), rt.dtype)
            total, count = cache.states["sum"], cache.states["count"]
            cu = batch.host["cu_seqlens"]
            for s in range(batch.n_seqs):
                slot = int(batch.host["seq_slot"][s])
                rows = x[cu[s]:cu[s + 1]].float()
                running = total[slot] + torch.cumsum(rows, dim=0)
                n = count[slot] + torch.arange(1, rows.shape[0] + 1, device=x.device)[:, None]
                out[cu[s]:cu[s + 1]] = ((running / n) @ self.w.float().t()).to(rt.dtype)
                total[slot] = running[-1]
                count[slot] = n[-1]
            return out

    if "running_mean" not in registered_parts("mixer"):
        register_part("mixer", "running_mean", RunningMean)

    def build_spec(cfg):
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
        register_architecture(Architecture("ToyForCausalLM", lambda d: d, build_spec))


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
    assert [n.name for _, n in lm.cache.layout.states] == ["sum", "count", "sum", "count"]
    assert not lm.model.graph_safe      # the toy plans on the host: its steps are never replayed
    got = EngineDriver(lm).run(portions_schedule(reqs))
    got2 = EngineDriver(lm).run(portions_schedule(dict(reversed(list(reqs.items())))))   # slots reused
    for rid, toks in reqs.items():
        ref = toy_plain_logits(cfg, W, toks)
        assert_close_f32(got[rid], ref, f"toy/{rid}")
        assert_close_f32(got2[rid], ref, f"toy again/{rid}")


# ---------------------------------------------------------------- a toy routed feed-forward and position encoding
def register_toy_routed():
    """A feed-forward that routes every token to the one expert its router scores highest
    (SwiGLU experts, the router's score in 32-bit, written with torch), and a rotary
    encoding whose frequencies are the usual ones divided by a factor (positions stretched).
    Both are registered here, from outside the framework, with an architecture that mixes
    routed and dense layers."""
    from celeg_amd.config import (Architecture, LayerSpec, ModelSpec, PartSpec, RunStep,
                                  register_architecture, registered_architectures)
    from celeg_amd.parts import (FeedForward, PositionEncoding, WeightSpec, register_part,
                                 registered_parts)

    class TopOneExperts(FeedForward):
        def __init__(self, spec):
            super().__init__(spec)
            self.width, self.ff = int(self.params["width"]), int(self.params["ff"])
            self.experts = int(self.params["experts"])

        def weight_specs(self):
            specs = {"router": WeightSpec((self.experts, self.width))}
            for e in range(self.experts):
                specs[f"gate{e}"] = WeightSpec((self.ff, self.width))
                specs[f"up{e}"] = WeightSpec((self.ff, self.width))
                specs[f"down{e}"] = WeightSpec((self.width, self.ff))
            return specs

        def load(self, tensors, rt):
            self.w = tensors

        def forward(self, x, batch, rt):
            xf = x.float()
            choice = (xf @ self.w["router"].float().t()).argmax(dim=1)
            out = rt.ws.buf("toy_routed_out", (x.shape[0], self.width), rt.dtype)
            for e in range(self.experts):
                rows = (choice == e).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                xe = xf[rows]
                act = torch.nn.functional.silu(xe @ self.w[f"gate{e}"].float().t()) * (xe @ self.w[f"up{e}"].float().t())
                out[rows] = (act @ self.w[f"down{e}"].float().t()).to(rt.dtype)
            return out

    class StretchedRope(PositionEncoding):
        def __init__(self, spec):
            super().__init__(spec)
            self.theta, self.factor = float(self.params["theta"]), float(self.params["factor"])
            self.rotary_dim = int(self.params["rotary_dim"])

        def tables(self, rt):
            freq = [self.theta ** (-2.0 * i / self.rotary_dim) / self.factor for i in range(self.rotary_dim // 2)]
            return {"inv_freq": torch.tensor(freq, dtype=torch.float64).to(torch.float32).to(rt.device),
                    "rotary_dim": self.rotary_dim}

    if "toy_top_one" not in registered_parts("ffn"):
        register_part("ffn", "toy_top_one", TopOneExperts)
    if "toy_stretched_rope" not in registered_parts("position"):
        register_part("position", "toy_stretched_rope", StretchedRope)

    def build_spec(cfg):
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
        register_architecture(Architecture("ToyRoutedForCausalLM", lambda d: d, build_spec))


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


def test_run_order_with_a_layer_twice_and_a_shared_cache(model_folders, tmp_path):
    """LFM2 parts under another run order: layer 1 runs twice (own cache each time) and
    layer 3 reads the keys and values the first run of layer 1 wrote."""
    from celeg_amd.cache import CacheManager
    from celeg_amd.config import RunStep, spec_from_config
    from celeg_amd.engine import Model, ModelRunner, make_runtime
    from celeg_amd.engine.loading import LoadedModel
    from celeg_amd.weights import Checkpoint, load_tensors
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    config, spec = spec_from_config(TINY["A"][0])
    order = (RunStep(0), RunStep(1), RunStep(2), RunStep(1), RunStep(3, kv_from=1))
    spec = dataclasses.replace(spec, order=order)
    model = Model(spec)
    rt = make_runtime(DEV, torch.float32)
    expected = model.expected_tensors()
    assert "model.layers.3.self_attn.k_proj.weight" not in expected
    ck = Checkpoint(folder)
    tensors = {n: ck.tensor(n).float().to(DEV) for n in expected}
    model.load(tensors, rt)
    cache = CacheManager(model.cache_layout(), page_tokens=16, n_pages=8, max_requests=2,
                         max_context=128, device=DEV, dtype=torch.float32)
    lm = LoadedModel(config, spec, model, cache, ModelRunner(model, cache, rt, max_batched_tokens=64), rt)
    reqs = {"a": random_tokens(256, 50, 8), "b": random_tokens(256, 37, 9)}
    got = EngineDriver(lm).run(portions_schedule(reqs))
    for rid, toks in reqs.items():
        ref = plain.model_logits(cfg, W, toks, order=[0, 1, 2, 1, 3], kv_from={4: 1})
        assert_close_f32(got[rid], ref, f"order/{rid}")

"""A mixer defined here that keeps keys and values in the cache manager's pages, with values
three times as wide as its keys: registered through the library's interface, it gets a page
group of its own beside nothing else, writes its keys and values through the block table and
attends over them, cut into portions and single tokens, with so few pages that they are used
again; against the same attention written over whole sequences."""
import math

import pytest
import torch

import plain_lfm2 as plain
from helpers import EngineDriver, assert_close_f32, mixed_schedule, peak_tokens, portions_schedule, random_tokens

pytestmark = pytest.mark.gpu
KD, VD = 8, 24


def register_wide_values():
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    from celeg_amd.native import TensorView
    from celeg_amd.parts import as_tensor, int_array, on_stream, register_part, registered_parts

    def device_view(pointer, dtype, shape):
        view = TensorView()
        view.data, view.dtype, view.ndim = pointer, dtype, 1
        view.shape[0], view.stride[0] = math.prod(shape), 1
        return as_tensor(view).view(shape)

    class WideValueAttention:
        """One head: softmax(q.k / sqrt(KD)) over the keys so far, values of width VD."""
        def __init__(self, spec):
            self.width = int(spec["params"]["width"])

        def describe(self):
            return {"weights": {"q": {"shape": [KD, self.width]}, "k": {"shape": [KD, self.width]},
                                "v": {"shape": [VD, self.width]}, "o": {"shape": [self.width, VD]}},
                    "kv_need": {"kv_heads": 1, "head_dim": KD, "v_head_dim": VD, "window": None},
                    "graph_safe": False, "out_width": self.width}

        def load(self, tensors):
            self.w = {role: as_tensor(view).float() for role, view in tensors.items()}

        def forward(self, args):
            c, step = args.cache, args.step
            assert c.has_kv and c.writes_kv and c.head_dim == KD and c.v_head_dim == VD and c.kv_heads == 1
            P = c.page_tokens
            with on_stream(args):
                x, out = as_tensor(args.x).float(), as_tensor(args.out)
                K = device_view(c.k, c.kv_dtype, (c.n_pages, c.n_layers, 1, P, KD))[:, c.layer, 0]      # [pages, P, KD]
                V = device_view(c.v, c.kv_dtype, (c.n_pages, c.n_layers, 1, VD, P))[:, c.layer, 0]      # [pages, VD, P]
                q, k, v = x @ self.w["q"].t(), x @ self.w["k"].t(), x @ self.w["v"].t()
                for s in range(step.n_seqs):
                    slot, start = step.host_seq_slot[s], step.host_seq_start[s]
                    lo, hi = step.host_cu_seqlens[s], step.host_cu_seqlens[s + 1]
                    end = start + hi - lo
                    pages = int_array(c.table + 4 * slot * c.table_stride, (end + P - 1) // P).long()
                    pos = torch.arange(start, end, device=x.device)
                    K[pages[pos // P], pos % P] = k[lo:hi].to(K.dtype)          # all rows written before any attends
                    V[pages[pos // P], :, pos % P] = v[lo:hi].to(V.dtype)
                    keys = K[pages].reshape(-1, KD)[:end].float()
                    values = V[pages].permute(0, 2, 1).reshape(-1, VD)[:end].float()
                    scores = q[lo:hi] @ keys.t() / math.sqrt(KD)
                    scores = scores.masked_fill(torch.arange(end, device=x.device)[None, :] > pos[:, None], float("-inf"))
                    out[lo:hi] = ((torch.softmax(scores, dim=-1) @ values) @ self.w["o"].t()).to(out.dtype)

    if "toy_wide_values" not in registered_parts("mixer"):
        register_part("mixer", "toy_wide_values", WideValueAttention)

    def build(cfg, shapes):
        H, V = cfg["width"], cfg["vocab"]
        norm = lambda name: PartSpec("rmsnorm", {"width": H, "eps": 1e-5}, {"weight": name})
        layers = tuple(LayerSpec(PartSpec("toy_wide_values", {"width": H}, {r: f"l{i}.{r}" for r in "qkvo"}), norm(f"l{i}.n1"),
                                 PartSpec("swiglu", {"width": H, "ff": 2 * H}, {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"}),
                                 norm(f"l{i}.n2")) for i in range(cfg["layers"]))
        return ModelSpec("ToyWideValues", V, H, 256, PartSpec("embedding", {"vocab": V, "width": H}, {"table": "emb"}), layers,
                         tuple(RunStep(i) for i in range(len(layers))), norm("final"), PartSpec("tied_head", {"vocab": V, "width": H}))
    if "ToyWideValues" not in registered_architectures():
        register_architecture("ToyWideValues", build)


def whole_sequence_logits(cfg, W, tokens):
    h = plain.embedding(W["emb"], tokens)
    T = len(tokens)
    mask = torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1)
    for i in range(cfg["layers"]):
        n = plain.rmsnorm(h, W[f"l{i}.n1"], 1e-5)
        q, k, v = (plain.linear(n, W[f"l{i}.{r}"]) for r in "qkv")
        scores = (q @ k.t() / math.sqrt(KD)).masked_fill(mask, float("-inf"))
        h = h + plain.linear(torch.softmax(scores, dim=-1) @ v, W[f"l{i}.o"])
        h = h + plain.swiglu_ffn(plain.rmsnorm(h, W[f"l{i}.n2"], 1e-5), W[f"l{i}.g"], W[f"l{i}.u"], W[f"l{i}.d"])
    return plain.linear(plain.rmsnorm(h, W["final"], 1e-5), W["emb"])


def test_a_mixer_from_outside_keeps_wide_values_in_pages(tmp_path):
    from celeg_amd.engine import load_model
    from celeg_amd.weights import write_random_model
    register_wide_values()
    cfg = {"architectures": ["ToyWideValues"], "width": 32, "vocab": 61, "layers": 2}
    folder = write_random_model(cfg, str(tmp_path / "wide"), seed=3, dtype=torch.float32, std=0.3)
    _, W = plain.load_model_folder(folder)
    reqs = {f"r{i}": random_tokens(61, n, seed=30 + i) for i, n in enumerate((70, 41, 55, 23, 64, 38))}
    ref = {rid: whole_sequence_logits(cfg, W, toks) for rid, toks in reqs.items()}
    steps = mixed_schedule(reqs, max_live=3, seed=2)
    tokens = peak_tokens(steps, page_round=16)
    lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=tokens // 16, max_requests=3, max_batched_tokens=64)
    layout = lm.cache.layout
    assert [(g["head_dim"], g["v_head_dim"], g["layers"]) for g in layout["kv_groups"]] == [(KD, VD, 2)]
    got = EngineDriver(lm).run(steps)
    for rid in reqs:
        assert_close_f32(got[rid], ref[rid], f"wide values/mixed/{rid}")
    assert lm.cache.free_pages() == [tokens // 16] and lm.cache.n_free_slots == 3
    two = {rid: reqs[rid] for rid in ("r0", "r2")}
    got = EngineDriver(lm).run(portions_schedule(two))
    for rid in two:
        assert_close_f32(got[rid], ref[rid], f"wide values/portions/{rid}")
    lm.close()


def test_the_librarys_attention_refuses_values_of_another_width(tmp_path):
    from celeg_amd import native
    from celeg_amd.config import LayerSpec, ModelSpec, PartSpec, RunStep, register_architecture, registered_architectures
    from celeg_amd.engine import StepEntry, load_model
    from celeg_amd.weights import write_random_model
    register_wide_values()

    def build(cfg, shapes):       # a layer of the toy and the library's attention reading ITS pages
        H = 32
        norm = lambda name: PartSpec("rmsnorm", {"width": H, "eps": 1e-5}, {"weight": name})
        ffn = lambda i: PartSpec("swiglu", {"width": H, "ff": 64}, {"gate": f"l{i}.g", "up": f"l{i}.u", "down": f"l{i}.d"})
        toy = LayerSpec(PartSpec("toy_wide_values", {"width": H}, {r: f"l0.{r}" for r in "qkvo"}), norm("l0.n1"), ffn(0), norm("l0.n2"))
        own = LayerSpec(PartSpec("gqa_attention", {"width": H, "heads": 1, "kv_heads": 1, "head_dim": KD, "qk_norm": False,
                                                   "position": PartSpec("none")},
                                 {"q_proj": "l1.q", "k_proj": "l1.k", "v_proj": "l1.v", "out_proj": "l1.o"}), norm("l1.n1"), ffn(1), norm("l1.n2"))
        return ModelSpec("ToyMismatch", 61, H, 64, PartSpec("embedding", {"vocab": 61, "width": H}, {"table": "emb"}), (toy, own),
                         (RunStep(0), RunStep(1, kv_from=0)), norm("final"), PartSpec("tied_head", {"vocab": 61, "width": H}))
    if "ToyMismatch" not in registered_architectures():
        register_architecture("ToyMismatch", build)
    with pytest.raises(Exception, match="width of the values"):
        folder = write_random_model({"architectures": ["ToyMismatch"]}, str(tmp_path / "mismatch"), seed=1,
                                    dtype=torch.float32, std=0.1)
        lm = load_model(folder, dtype="float32", page_tokens=16, n_pages=4, max_requests=1, max_batched_tokens=32)
        slot = lm.cache.open()
        lm.cache.prepare(slot, 0, 4)
        lm.runner.step([StepEntry(slot, 0, [1, 2, 3, 4], [3])])

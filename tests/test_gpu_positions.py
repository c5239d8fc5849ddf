"""Position encodings beyond the architecture's own: the rotary encoding that turns
neighbouring values (2i, 2i+1) instead of the two halves of a head, as a parameter of the
built-in "rope" and from a position encoding registered outside the library, over part of a
head; each against a rotation written out here."""
import math

import pytest
import torch

import plain_lfm2 as plain
from test_gpu_parts import run_part_alone


def turn_neighbours(x, inv_freq):
    """x [T, heads, hd] (float64); pair i = (x[2i], x[2i+1]) of the first 2 * len(inv_freq) values
    turns by the 32-bit angle position * inv_freq[i]."""
    out = x.clone()
    T = x.shape[0]
    for i, f in enumerate(inv_freq):
        angle = (torch.arange(T, dtype=torch.float32) * torch.tensor(f, dtype=torch.float32)).double()
        c, s = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def attention_reference(x, W, heads, kv_heads, hd, inv_freq):
    T = x.shape[0]
    q = plain.linear(x, W["q"]).reshape(T, heads, hd)
    k = plain.linear(x, W["k"]).reshape(T, kv_heads, hd)
    v = plain.linear(x, W["v"]).reshape(T, kv_heads, hd)
    o = plain.causal_attention(turn_neighbours(q, inv_freq), turn_neighbours(k, inv_freq), v)
    return plain.linear(o.reshape(T, -1), W["o"])


def test_the_turned_pairs_keep_their_length_and_depend_on_distance_only():
    # what pins the rotation written out above: |pair| is kept, and q.k depends on the distance only
    g = torch.Generator().manual_seed(0)
    q = torch.randn(1, 1, 8, generator=g, dtype=torch.float64).expand(12, 1, 8).clone()
    k = torch.randn(1, 1, 8, generator=g, dtype=torch.float64).expand(12, 1, 8).clone()
    freq = [1.0, 0.3, 0.05]
    tq, tk = turn_neighbours(q, freq), turn_neighbours(k, freq)
    assert torch.allclose(tq.pow(2).sum(-1), q.pow(2).sum(-1), atol=1e-6)   # float32 angles
    assert torch.equal(tq[..., 6:], q[..., 6:])                # beyond the turned part: unchanged
    dots = torch.einsum("thd,shd->ts", tq, tk)
    assert torch.allclose(dots[3, 1], dots[9, 7], atol=1e-5) and not torch.allclose(dots[3, 1], dots[3, 2], atol=1e-3)
    # one pair, frequency 1, position 1: (1, 0) -> (cos 1, sin 1)
    one = turn_neighbours(torch.tensor([[[0.0, 0.0]], [[1.0, 0.0]]], dtype=torch.float64), [1.0])
    assert torch.allclose(one[1, 0], torch.tensor([math.cos(1.0), math.sin(1.0)], dtype=torch.float64), atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("rotary_dim", [16, 8])
def test_rope_over_neighbouring_pairs_as_a_parameter(tmp_path, rotary_dim):
    from celeg_amd.config import PartSpec
    theta = 100.0
    spec = PartSpec("gqa_attention", {
        "width": 40, "heads": 4, "kv_heads": 2, "head_dim": 16, "qk_norm": False,
        "position": PartSpec("rope", {"theta": theta, "head_dim": 16, "rotary_dim": rotary_dim, "pairing": "neighbours"})},
        {"q_proj": "q", "k_proj": "k", "v_proj": "v", "out_proj": "o"})
    x = torch.randn(33, 40, generator=torch.Generator().manual_seed(5))
    inv_freq = [float(torch.tensor(theta ** (-2.0 * i / rotary_dim), dtype=torch.float32)) for i in range(rotary_dim // 2)]
    for i, cuts in enumerate(([33], [7, 1, 1, 24])):
        got, W = run_part_alone(tmp_path / str(i), x, cuts, mixer=spec)
        ref = attention_reference(x.double(), W, 4, 2, 16, inv_freq)
        torch.testing.assert_close(got - x.double(), ref, rtol=1e-4, atol=1e-5)
    # the pairing matters: the same weights with halves give another result
    halves = PartSpec("gqa_attention", dict(spec.params, position=PartSpec("rope", {"theta": theta, "head_dim": 16,
                                                                                  "rotary_dim": rotary_dim})), spec.tensors)
    other, _ = run_part_alone(tmp_path / "halves", x, [33], mixer=halves)
    assert (other - got).abs().max() > 1e-3


@pytest.mark.gpu
def test_a_position_encoding_from_outside_with_neighbouring_pairs(tmp_path):
    from celeg_amd.config import PartSpec
    from celeg_amd.parts import register_part, registered_parts

    class LinearFrequencies:
        """Frequencies 1/(1 + i * step) over neighbouring pairs of the first ``rotary_dim`` values."""
        def __init__(self, spec):
            self.step, self.rotary_dim = float(spec["params"]["step"]), int(spec["params"]["rotary_dim"])

        def describe(self):
            return {"inv_freq": [1.0 / (1.0 + i * self.step) for i in range(self.rotary_dim // 2)],
                    "rotary_dim": self.rotary_dim, "pairing": "neighbours"}

        def forward(self, args):
            raise RuntimeError("a position encoding gives tables; it is never called")

    if "toy_linear_frequencies" not in registered_parts("position"):
        register_part("position", "toy_linear_frequencies", LinearFrequencies)
    spec = PartSpec("gqa_attention", {
        "width": 24, "heads": 2, "kv_heads": 1, "head_dim": 32, "qk_norm": False,
        "position": PartSpec("toy_linear_frequencies", {"step": 0.5, "rotary_dim": 12})},
        {"q_proj": "q", "k_proj": "k", "v_proj": "v", "out_proj": "o"})
    x = torch.randn(21, 24, generator=torch.Generator().manual_seed(6))
    inv_freq = [float(torch.tensor(1.0 / (1.0 + i * 0.5), dtype=torch.float32)) for i in range(6)]
    got, W = run_part_alone(tmp_path, x, [5, 16], mixer=spec)
    ref = attention_reference(x.double(), W, 2, 1, 32, inv_freq)
    torch.testing.assert_close(got - x.double(), ref, rtol=1e-4, atol=1e-5)
    with pytest.raises(Exception, match="pairing"):
        from celeg_amd import native
        register_part("position", "toy_bad_pairing", type("Bad", (), {
            "__init__": lambda self, spec: None,
            "describe": lambda self: {"inv_freq": [1.0], "rotary_dim": 2, "pairing": "thirds"},
            "forward": lambda self, args: None}))
        native.describe_config({"architectures": ["PartsAlone"], "width": 8, "rows": 4, "mixer": PartSpec(
            "gqa_attention", {"width": 8, "heads": 1, "kv_heads": 1, "head_dim": 8, "qk_norm": False,
                              "position": PartSpec("toy_bad_pairing")},
            {"q_proj": "q", "k_proj": "k", "v_proj": "v", "out_proj": "o"}).to_json()})

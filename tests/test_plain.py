"""Pins of the plain implementation: vectors the reference's own tests hold, special
cases that reduce to a library routine, and invariants.  Each is chosen so that a
plausible mistake (a wrong sign or pairing, a norm in the wrong place, a reversed
filter) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_lfm2 as plain
from conftest import TINY
from helpers import WEIGHT_STD, random_tokens


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


# ---------------------------------------------------------------- reference vectors
def test_rmsnorm_vector():
    # tests/reference_test.cpp:29-31
    y = plain.rmsnorm(torch.tensor([1., 2., 3., 4.]), torch.ones(4), 1e-5)
    assert abs(float(y[0]) - 1 / math.sqrt(7.5 + 1e-5)) < 1e-12


def test_rope_vector():
    # tests/reference_test.cpp:33-38: {1,2,3,4}, cos {1,0}, sin {0,1} -> {1,-4,3,2}
    x = torch.tensor([1., 2., 3., 4.]).reshape(1, 1, 4)
    out = plain.rope_apply(x, torch.tensor([[1., 0.]]), torch.tensor([[0., 1.]]))
    assert out.reshape(-1).tolist() == [1., -4., 3., 2.]


def test_conv_vector():
    # tests/reference_test.cpp:68-73
    y = plain.short_conv(torch.tensor([[1., 1., 1., 1., 2., 4.]]),
                         torch.tensor([[1., 2., 3.], [1., 2., 3.]]))
    assert y.tolist() == [[6., 12.]]


def test_conv_vector_tells_the_three_thirds_of_bcx_apart():
    # Worked by hand from src/backend/cpu/kernels/convolution.cpp:14-27 (b = bcx[ch],
    # c = bcx[H + ch], x = bcx[2H + ch]; state = b * x; output = c * conv), H 1, L 2, taps
    # {1, 1}: rows {2,3,5} and {7,11,13} give bx = {10, 91}, y = {3 * 10, 11 * (10 + 91)}.
    # C and x swapped would give {30, 1079}; B and C swapped {30, 1106}.
    y = plain.short_conv(torch.tensor([[2., 3., 5.], [7., 11., 13.]]), torch.tensor([[1., 1.]]))
    assert y.reshape(-1).tolist() == [30., 1111.]
    # taps {2, 1}: tap L-1 multiplies the current token, tap 0 the one before
    # (weight[tap * hidden + channel] with slot (cursor + 1 + tap) % L): 11 * (2 * 10 + 91);
    # the filter reversed would give 11 * (10 + 2 * 91) = 2112
    y = plain.short_conv(torch.tensor([[2., 3., 5.], [7., 11., 13.]]), torch.tensor([[2., 1.]]))
    assert y.reshape(-1).tolist() == [30., 1221.]


# q = {3, 4}, norm weight {1, 2}, eps 0, position 1, head size 2 (one pair, frequency 1):
# src/backend/cpu/kernels/rope.cpp:95-108 normalises first, inv = 1/sqrt(12.5),
# a = 3 inv, b = 4 inv * 2, and rotates the normalised pair by the angle 1:
# {a cos1 - b sin1, b cos1 + a sin1}.  Rotating first and normalising after would give
# {(3 cos1 - 4 sin1) inv, (4 cos1 + 3 sin1) inv * 2} = {-0.4936, 2.6506}.
QK_NORM_THEN_ROPE = [3 / math.sqrt(12.5) * math.cos(1.0) - 8 / math.sqrt(12.5) * math.sin(1.0),
                     8 / math.sqrt(12.5) * math.cos(1.0) + 3 / math.sqrt(12.5) * math.sin(1.0)]


def test_q_and_k_are_normalised_before_they_are_rotated():
    assert abs(QK_NORM_THEN_ROPE[0] - (-1.445570)) < 1e-6 and abs(QK_NORM_THEN_ROPE[1] - 1.936577) < 1e-6
    cfg = {"num_attention_heads": 1, "num_key_value_heads": 1, "head_dim": 2, "norm_eps": 0.0,
           "rope_theta": 10000.0}
    eye = torch.eye(2, dtype=torch.float64)
    W = {"self_attn.q_proj.weight": eye, "self_attn.k_proj.weight": eye, "self_attn.v_proj.weight": eye,
         "self_attn.q_layernorm.weight": torch.tensor([1., 2.]),
         "self_attn.k_layernorm.weight": torch.tensor([1., 2.])}
    n = torch.tensor([[0., 0.], [3., 4.]], dtype=torch.float64)     # the row at position 1 is {3, 4}
    q, k, v = plain.attention_project(n, W, "", cfg, [0, 1])
    for got in (q[1, 0], k[1, 0]):
        assert torch.allclose(got, torch.tensor(QK_NORM_THEN_ROPE, dtype=torch.float64), atol=1e-6)
    assert v[1, 0].tolist() == [3., 4.]


def test_attention_vector():
    # tests/reference_test.cpp:40-53: 2 query heads share 1 kv head; both heads equal and
    # strictly between the two values
    q = torch.tensor([1., 0., 1., 0.]).reshape(1, 2, 2)
    k = torch.tensor([[1., 0.], [0., 1.]]).reshape(2, 1, 2)
    v = torch.tensor([[2., 4.], [6., 8.]]).reshape(2, 1, 2)
    # decode over both keys = last row of a two-row causal pass whose last query is q
    out = plain.causal_attention(torch.cat([q, q]), k, v)[1]
    assert torch.allclose(out[0], out[1])
    assert 2.0 < float(out[0, 0]) < 6.0 and 4.0 < float(out[0, 1]) < 8.0
    w = math.exp(1 / math.sqrt(2)) / (math.exp(1 / math.sqrt(2)) + 1.0)   # scale 1/sqrt(hd), once
    assert abs(float(out[0, 0]) - (2 * w + 6 * (1 - w))) < 1e-12


def test_qk_norm_rope_at_position_zero_is_the_norm():
    # tests/cuda/attention_tests.cu:19-44
    cfg = plain.normalise_config(dict(TINY["A"][0]))
    x = torch.tensor([[1., 2., 3., 4.]]).reshape(1, 1, 4)
    cos, sin = plain.rope_cos_sin([0], 10000.0, 4)
    y = plain.rope_apply(plain.head_rmsnorm(x, torch.ones(4), 1e-5), cos, sin)
    assert torch.allclose(y.reshape(-1), plain.rmsnorm(torch.tensor([1., 2., 3., 4.]), torch.ones(4), 1e-5))


def test_sampler_vectors():
    # tests/cpu_sampler_test.cpp:8-43, tests/cuda/sampling_tests.cu:16-60
    assert plain.sample([1, 4, 2, 3], 0.0, 1, 1.0, 1.0, [False] * 4, 1)[0] == 1
    assert plain.sample([2, 5, 5, 1], 0.0, 1, 1.0, 1.0, [False] * 4, 1)[0] == 1   # ties: lowest id
    assert plain.sample([5, 4, 3, 2], 0.0, 1, 1.0, 2.0, [True, False, False, False], 1)[0] == 1
    a = plain.sample([1, 4, 2, 3], 0.8, 2, 1.0, 1.0, [False] * 4, 7)
    b = plain.sample([1, 4, 2, 3], 0.8, 2, 1.0, 1.0, [False] * 4, 7)
    assert a == b and a[0] in (1, 3)
    for seed in range(1, 40):
        assert plain.sample([1, 4, 2, 3], 1.5, 2, 1.0, 1.0, [False] * 4, seed)[0] in (1, 3)
        assert plain.sample([1, 4, 2, 3], 1.5, 4, 0.01, 1.0, [False] * 4, seed)[0] == 1  # top-p keeps one


def test_xorshift_first_values():
    state, bits = plain.xorshift64star(1)
    # by hand: s=1: s^=s>>12 -> 1; s^=s<<25 -> 1|1<<25; s^=s>>27 -> unchanged (bit 25>>27 = 0)
    assert state == (1 | (1 << 25))
    assert bits == (state * 2685821657736338717) % (1 << 64)
    _, u = plain.random_unit(1)
    assert 0.0 < u < 1.0


# ---------------------------------------------------------------- library special cases
def test_rmsnorm_equals_library():
    x, w = rnd(5, 96, seed=1), rnd(96, seed=2)
    assert torch.allclose(plain.rmsnorm(x, w, 3e-5), F.rms_norm(x, (96,), w, 3e-5), atol=1e-12)
    # norm in the wrong place (1+w, eps outside the root) would break these
    y = plain.rmsnorm(x, torch.ones(96), 1e-6)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=torch.float64), atol=1e-5)
    assert torch.allclose(plain.rmsnorm(1e4 * x, w, 1e-6), plain.rmsnorm(x, w, 1e-6), atol=1e-6)


@pytest.mark.parametrize("L", [1, 3, 4])
def test_short_conv_equals_library_conv1d(L):
    T, H = 19, 12
    bcx, w, b = rnd(T, 3 * H, seed=3), rnd(H, 1, L, seed=4), rnd(H, seed=5)
    B, C, x = bcx[:, :H], bcx[:, H:2 * H], bcx[:, 2 * H:]
    conv = F.conv1d((B * x).T.unsqueeze(0), w, b, padding=L - 1, groups=H)[0, :, :T].T
    assert torch.allclose(plain.short_conv(bcx, w, b), C * conv, atol=1e-12)
    if L == 1:
        assert torch.allclose(plain.short_conv(bcx, w), C * B * x * w[:, 0, 0], atol=1e-12)


def test_attention_equals_library_sdpa():
    T, Hq, Hkv, hd = 17, 6, 2, 16
    q, k, v = rnd(T, Hq, hd, seed=6), rnd(T, Hkv, hd, seed=7), rnd(T, Hkv, hd, seed=8)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                         v.transpose(0, 1)[None], is_causal=True, enable_gqa=True)
    assert torch.allclose(plain.causal_attention(q, k, v), ref[0].transpose(0, 1), atol=1e-12)
    # one head, no mask effect on row 0: output is v[0]
    assert torch.allclose(plain.causal_attention(q, k, v)[0, 0], v[0, 0])
    # MHA special case
    kk, vv = rnd(T, Hq, hd, seed=9), rnd(T, Hq, hd, seed=10)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None],
                                         vv.transpose(0, 1)[None], is_causal=True)
    assert torch.allclose(plain.causal_attention(q, kk, vv), ref[0].transpose(0, 1), atol=1e-12)


def test_window_attention_equals_masked_library_attention():
    T, H, hd, window = 15, 2, 8, 4
    q, k, v = rnd(T, H, hd, seed=11), rnd(T, H, hd, seed=12), rnd(T, H, hd, seed=13)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    mask = (j <= i) & (j > i - window)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None],
                                         v.transpose(0, 1)[None], attn_mask=mask)
    assert torch.allclose(plain.causal_attention(q, k, v, window=window),
                          ref[0].transpose(0, 1), atol=1e-12)


def test_swiglu_and_linear_equal_library():
    x, w1, w3, w2 = rnd(7, 24, seed=14), rnd(40, 24, seed=15), rnd(40, 24, seed=16), rnd(24, 40, seed=17)
    ref = F.linear(F.silu(F.linear(x, w1)) * F.linear(x, w3), w2)
    assert torch.allclose(plain.swiglu_ffn(x, w1, w3, w2), ref, atol=1e-12)
    assert float(plain.silu(torch.zeros(3, dtype=torch.float64)).abs().max()) == 0.0


# ---------------------------------------------------------------- invariants
def test_rope_depends_only_on_distance_and_keeps_norms():
    hd, theta = 32, 1e6
    q, k = rnd(1, 1, hd, seed=18), rnd(1, 1, hd, seed=19)

    def dot(m, n):
        cq, sq = plain.rope_cos_sin([m], theta, hd)
        ck, sk = plain.rope_cos_sin([n], theta, hd)
        return float((plain.rope_apply(q, cq, sq) * plain.rope_apply(k, ck, sk)).sum())
    assert abs(dot(7, 3) - dot(57, 53)) < 1e-4       # 32-bit angles limit the agreement
    assert abs(dot(7, 3) - dot(3, 7)) > 1e-3          # a wrong sign would make these equal
    c, s = plain.rope_cos_sin([11], theta, hd)
    y = plain.rope_apply(q, c, s)
    assert torch.allclose(y[..., :16] ** 2 + y[..., 16:] ** 2, q[..., :16] ** 2 + q[..., 16:] ** 2)
    c0, s0 = plain.rope_cos_sin([0], theta, hd)
    assert torch.equal(plain.rope_apply(q, c0, s0), q)
    f = plain.rope_inverse_frequencies(10000.0, 8)
    assert np.allclose(f, [1.0, 10000 ** -0.25, 10000 ** -0.5, 10000 ** -0.75])


def test_ff_dim_datapoints():
    assert plain.ff_dim(6656, True, 256, 1.0) == 4608
    assert plain.ff_dim(12288, True, 256, 1.0) == 8192
    assert plain.ff_dim(10752, True, 256, 1.0) == 7168
    assert plain.ff_dim(512, True, 32, 1.0) == 352
    assert plain.ff_dim(192, False) == 192


def test_model_shift_invariance_and_tying(model_folders):
    """Only distances between positions count: shifting all positions changes nothing
    (up to the 32-bit angles).  And an untied head equal to the embedding gives the tied
    logits."""
    folder = model_folders("A", torch.float32, WEIGHT_STD)
    cfg, W = plain.load_model_folder(folder)
    toks = random_tokens(cfg["vocab_size"], 20, seed=3)
    base = plain.model_logits(cfg, W, toks)
    shifted = plain.model_logits(cfg, W, toks, first_position=37)
    assert float((base - shifted).abs().max()) < 1e-4
    cfg2 = dict(cfg, tie_word_embeddings=False)
    W2 = dict(W)
    W2["lm_head.weight"] = W["model.embed_tokens.weight"]
    assert torch.equal(plain.model_logits(cfg2, W2, toks), base)
    # causality: a later token does not change earlier logits
    toks2 = toks[:10] + [(toks[10] + 1) % cfg["vocab_size"]] + toks[11:]
    other = plain.model_logits(cfg, W, toks2)
    assert torch.equal(other[:10], base[:10]) and not torch.equal(other[10:], base[10:])

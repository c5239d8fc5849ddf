"""The library's plain C++ functions (one beside each kernel, ``celeg_amd/csrc/host/reference.cpp``) against
the plain Python implementation, on the CPU: the same formulas written twice, from the same lines of the
reference, must agree; and the C++ side works on the kernels' own layouts (pages, block tables, state slots,
rows of several requests side by side), which the Python side does not know."""
import math

import numpy as np
import pytest
import torch

import plain_lfm2 as plain
import reference_ops as ref


def rand(*shape, seed=0, scale=1.0):
    return (np.random.RandomState(seed).randn(*shape) * scale).astype(np.float32)


def close(got, want, tol=2e-5):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), np.abs(got - want).max()


def test_embed_norm_linear_and_swiglu():
    table = rand(50, 24, seed=1)
    ids = [3, 49, 0, 7]
    close(ref.embed(table, ids), plain.embedding(torch.from_numpy(table), ids).numpy(), tol=0)
    with pytest.raises(ref.ReferenceError_, match="out of range"):
        ref.embed(table, [50])
    x, delta, w = rand(5, 96, seed=2), rand(5, 96, seed=3), 1 + rand(96, seed=4, scale=0.1)
    out, summed = ref.rmsnorm(x, w, 3e-5, delta)
    close(summed, x + delta, tol=1e-7)
    close(out, plain.rmsnorm(torch.from_numpy(x + delta), torch.from_numpy(w), 3e-5).numpy())
    wm, b = rand(7, 96, seed=5), rand(7, seed=6)
    close(ref.linear(x, wm, b), plain.linear(torch.from_numpy(x), torch.from_numpy(wm), torch.from_numpy(b)).numpy())
    gu = rand(4, 2 * 33, seed=7)
    g, u = torch.from_numpy(gu[:, :33]).double(), torch.from_numpy(gu[:, 33:]).double()
    close(ref.swiglu(gu), (plain.silu(g) * u).numpy())


@pytest.mark.parametrize("width,taps,bias", [(6, 3, False), (10, 4, True), (4, 1, True), (8, 5, False)])
def test_short_conv_in_portions_of_two_requests_side_by_side(width, taps, bias):
    """Two requests whose sequences arrive in portions (down to one token), their rows side by side in every
    step, their states in slots 2 and 0: the outputs equal the plain convolution over the whole sequences."""
    lengths = {"a": 23, "b": 17}
    slots = {"a": 2, "b": 0}
    bcx = {r: rand(n, 3 * width, seed=10 + i) for i, (r, n) in enumerate(lengths.items())}
    w = rand(width, taps, seed=20)
    cb = rand(width, seed=21) if bias else None
    state = np.zeros((3, taps, width), dtype=np.float32)
    got = {r: [] for r in lengths}
    done = {r: 0 for r in lengths}
    cuts = [5, 1, 2, 7, 1, 1, 3, 4]
    step = 0
    while any(done[r] < lengths[r] for r in lengths):
        rows, seq_slot, seq_start, cu, owners = [], [], [], [0], []
        for i, r in enumerate(lengths):
            n = min(cuts[(step + 3 * i) % len(cuts)], lengths[r] - done[r])
            if n <= 0:
                continue
            rows.append(bcx[r][done[r]:done[r] + n])
            seq_slot.append(slots[r]); seq_start.append(done[r]); cu.append(cu[-1] + n); owners.append((r, n))
            done[r] += n
        out = ref.short_conv(np.concatenate(rows), w, cb, state, seq_slot, seq_start, cu)
        at = 0
        for r, n in owners:
            got[r].append(out[at:at + n]); at += n
        step += 1
    for r in lengths:
        want = plain.short_conv(torch.from_numpy(bcx[r]), torch.from_numpy(w), torch.from_numpy(cb) if bias else None).numpy()
        close(np.concatenate(got[r]), want)


@pytest.mark.parametrize("head_dim,rotary_dim,normed", [(16, 16, True), (32, 16, True), (8, 8, False)])
def test_head_norm_then_rotation(head_dim, rotary_dim, normed):
    rows, heads = 9, 3
    x = rand(rows, heads, head_dim, seed=30)
    w = (1 + rand(head_dim, seed=31, scale=0.2)) if normed else None
    positions = [0, 1, 2, 77, 78, 500, 3, 4000, 12]
    inv_freq = plain.rope_inverse_frequencies(10000.0, rotary_dim).astype(np.float32)
    got = ref.qk_norm_rope(x, w, 1e-5, inv_freq, rotary_dim, 0, positions)
    want = torch.from_numpy(x).double()
    if normed:
        want = plain.head_rmsnorm(want, torch.from_numpy(w), 1e-5)
    cos, sin = plain.rope_cos_sin(positions, 10000.0, rotary_dim)
    close(got, plain.rope_apply(want, cos, sin).numpy(), tol=1e-5)
    # pairs of neighbours instead of halves: the same numbers in other places
    paired = ref.qk_norm_rope(x, w, 1e-5, inv_freq, rotary_dim, 1, positions)
    half = rotary_dim // 2
    perm = np.arange(head_dim)
    perm[:rotary_dim] = np.concatenate([np.arange(0, rotary_dim, 2), np.arange(1, rotary_dim, 2)])   # halves order -> neighbours' places
    halves_of_permuted = ref.qk_norm_rope(x[:, :, perm], w[perm] if normed else None, 1e-5, inv_freq, rotary_dim, 0, positions)
    close(paired[:, :, perm], halves_of_permuted, tol=1e-6)


@pytest.mark.parametrize("window", [0, 11])
def test_attention_over_pages_in_steps(window):
    """Two requests whose keys and values go into pages of 4 tokens handed out in a scrambled order, a few
    rows a step, two layers in the pool: every row attends over its own request's pages only, and the result
    equals plain attention over the whole sequences."""
    heads, kv_heads, hd, page_tokens, n_layers, layer = 4, 2, 8, 4, 2, 1
    lengths = {0: 21, 1: 14}
    cache = ref.PagedCache(n_pages=12, n_layers=n_layers, kv_heads=kv_heads, head_dim=hd, page_tokens=page_tokens, slots=2,
                           pages_per_request=6)
    free = [7, 2, 11, 0, 5, 9, 3, 1, 10, 4, 8, 6]
    q = {s: rand(n, heads * hd, seed=40 + s) for s, n in lengths.items()}
    k = {s: rand(n, kv_heads * hd, seed=50 + s) for s, n in lengths.items()}
    v = {s: rand(n, kv_heads * hd, seed=60 + s) for s, n in lengths.items()}
    cache.k[:] = np.nan                      # nothing but a request's own pages may be read
    cache.v[:] = np.nan
    got = {s: [] for s in lengths}
    done = {s: 0 for s in lengths}
    cuts = [3, 1, 6, 2]
    step = 0
    while any(done[s] < lengths[s] for s in lengths):
        rows_q, rows_k, rows_v, slot_of, pos_of, owners = [], [], [], [], [], []
        for s in lengths:
            n = min(cuts[(step + s) % len(cuts)], lengths[s] - done[s])
            if n <= 0:
                continue
            for p in range(done[s], done[s] + n):
                if cache.table[s, p // page_tokens] < 0:
                    page = free.pop(0)
                    cache.table[s, p // page_tokens] = page
                    cache.k[page, layer] = 0; cache.v[page, layer] = 0          # (stale but finite contents)
            rows_q.append(q[s][done[s]:done[s] + n]); rows_k.append(k[s][done[s]:done[s] + n]); rows_v.append(v[s][done[s]:done[s] + n])
            slot_of += [s] * n; pos_of += list(range(done[s], done[s] + n)); owners.append((s, n))
            done[s] += n
        cache.store(np.concatenate(rows_k), np.concatenate(rows_v), slot_of, pos_of, layer)
        out = cache.attend(np.concatenate(rows_q), slot_of, pos_of, layer, heads, 1 / math.sqrt(hd), window)
        at = 0
        for s, n in owners:
            got[s].append(out[at:at + n]); at += n
        step += 1
    assert np.isnan(cache.k[:, 0]).all() and np.isnan(cache.v[:, 0]).all()      # the other layer was never written
    for s, n in lengths.items():
        want = plain.causal_attention(torch.from_numpy(q[s]).reshape(n, heads, hd), torch.from_numpy(k[s]).reshape(n, kv_heads, hd),
                                      torch.from_numpy(v[s]).reshape(n, kv_heads, hd), window=window or None).reshape(n, -1).numpy()
        close(np.concatenate(got[s]), want, tol=1e-5)


@pytest.mark.parametrize("temperature,top_k,top_p,penalty", [(0.0, 50, 1.0, 1.0), (0.8, 1, 1.0, 1.3), (0.7, 12, 1.0, 1.0),
                                                             (1.3, 40, 0.6, 1.1), (0.1, 50, 1.0, 1.05), (2.0, 500, 0.95, 1.0)])
def test_sampler_equals_the_plain_sampler(temperature, top_k, top_p, penalty):
    vocab = 200
    rng = np.random.RandomState(5)
    for trial in range(12):
        logits = (rng.randn(vocab) * 3).astype(np.float32)
        logits[17] = logits[90] = logits.max()                  # a tie for the largest
        seen = rng.rand(vocab) < 0.2
        state = 1000 + trial
        want, _ = plain.sample(logits, temperature, top_k, top_p, penalty, seen, state)
        _, u = plain.random_unit(state)
        assert ref.sample(logits, temperature, top_k, top_p, penalty, seen, u) == want

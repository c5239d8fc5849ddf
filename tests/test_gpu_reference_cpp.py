"""The kernels against the library's plain C++ functions (``celeg_amd/csrc/host/reference.cpp``, one beside
each kernel), through the library's dispatcher: the same arguments, the same pages, block tables and state
slots on both sides, so that what the kernels leave in the cache is compared too, place by place."""
import math

import numpy as np
import pytest
import torch

import plain_lfm2 as plain
import reference_ops as ref
from kernel_harness import DEV, build_batch, make_cache

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from kernel_ops import HipOps
    return HipOps(DEV)


def rand(*shape, seed=0, scale=1.0):
    return (np.random.RandomState(seed).randn(*shape) * scale).astype(np.float32)


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV).to(dtype)


def close(got, want, tol):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), np.abs(got - want).max()


@pytest.mark.parametrize("rows,width", [(5, 96), (70, 1024), (3, 1030)])
def test_rmsnorm_and_swiglu(ops, rows, width):
    x, delta, w = rand(rows, width, seed=1), rand(rows, width, seed=2), 1 + rand(width, seed=3, scale=0.1)
    want, summed = ref.rmsnorm(x, w, 1e-5, delta)
    xd, out = dev(x), torch.empty(rows, width, device=DEV)
    ops.rmsnorm(xd, dev(w), 1e-5, out, delta=dev(delta))
    close(out.cpu().numpy(), want, 1e-5)
    close(xd.cpu().numpy(), summed, 1e-6)
    gu = rand(rows, 2 * width, seed=4)
    act = torch.empty(rows, width, device=DEV)
    ops.swiglu(dev(gu), act)
    close(act.cpu().numpy(), ref.swiglu(gu), 1e-5)


@pytest.mark.parametrize("M,N,K", [(3, 50, 96), (70, 130, 77)])
def test_32bit_product(ops, M, N, K):
    x, w, b = rand(M, K, seed=5), rand(N, K, seed=6, scale=0.1), rand(N, seed=7)
    out = torch.empty(M, N, device=DEV)
    ops.linear(dev(x), dev(w), out, bias=dev(b))
    close(out.cpu().numpy(), ref.linear(x, w, b), 1e-5)


@pytest.mark.parametrize("width,taps,bias", [(96, 3, False), (1032, 4, True), (64, 2, True)])
def test_short_conv_and_its_state(ops, width, taps, bias):
    """Three requests in portions of changing size (long ones, single tokens), their rows side by side: the
    kernel's outputs AND the state it leaves in every slot after every step equal the C++ function's."""
    from celeg_amd.engine import StepEntry
    lengths = [70, 41, 23]
    cache = make_cache(0, 0, 1, torch.float32, slots=4, states=[(0, "conv", (taps, width))])
    state_gpu = cache.layer_cache(0).states["conv"]
    state_ref = np.zeros((5, taps, width), dtype=np.float32)
    bcx = [rand(n, 3 * width, seed=10 + i) for i, n in enumerate(lengths)]
    w = rand(width, taps, seed=20)
    cb = rand(width, seed=21) if bias else None
    slots = [cache.open() for _ in lengths]
    done = [0] * len(lengths)
    cuts = [33, 1, 17, 2, 1, 20]
    step = 0
    while any(d < n for d, n in zip(done, lengths)):
        entries, parts = [], []
        for i, n in enumerate(lengths):
            c = min(cuts[(step + 2 * i) % len(cuts)], n - done[i])
            if c <= 0:
                continue
            entries.append(StepEntry(slots[i], done[i], [0] * c))
            parts.append((i, done[i], c))
            done[i] += c
        batch, keep = build_batch(ops, cache, entries)
        parts = [parts[j] for j in batch.entry_order]
        rows = np.concatenate([bcx[i][p:p + c] for i, p, c in parts])
        out = torch.empty(len(rows), width, device=DEV)
        ops.short_conv(dev(rows), dev(w), dev(cb) if bias else None, state_gpu, out, batch)
        cu = np.cumsum([0] + [c for _, _, c in parts])
        want = ref.short_conv(rows, w, cb, state_ref, [slots[i] for i, _, _ in parts], [p for _, p, _ in parts], cu)
        close(out.cpu().numpy(), want, 1e-5)
        for i in range(len(lengths)):
            close(state_gpu[slots[i]].cpu().numpy(), state_ref[slots[i]], 1e-6)
        step += 1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,page_tokens,window", [(4, 2, 64, 16, 0), (6, 2, 48, 8, 0), (2, 1, 128, 16, 37)])
def test_norm_rotation_cache_write_and_attention(ops, dtype, heads, kv_heads, hd, page_tokens, window):
    """Two requests in steps of changing size: q and k normalised and rotated, k and v written into the pages,
    then attention over the pages.  The kernel's pools are compared with the C++ function's, page by page
    (the same block table on both sides: a key or value in another place than the C++ layout says fails), and
    the outputs with its attention."""
    from celeg_amd.engine import StepEntry
    lengths, n_layers, layer = [150, 67], 2, 1
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    cache = make_cache(kv_heads, hd, n_layers, dtype, page_tokens=page_tokens, n_pages=40, max_context=160, slots=2)
    kv = cache.layer_cache(layer).kv
    host = ref.PagedCache(n_pages=41, n_layers=n_layers, kv_heads=kv_heads, head_dim=hd, page_tokens=page_tokens, slots=3,
                          pages_per_request=kv.table.shape[1])
    qw, kw = 1 + rand(hd, seed=31, scale=0.1), 1 + rand(hd, seed=32, scale=0.1)
    inv_freq = plain.rope_inverse_frequencies(10000.0, hd).astype(np.float32)
    data = [[rand(n, h * hd, seed=40 + 3 * i + j) for j, h in enumerate((heads, kv_heads, kv_heads))] for i, n in enumerate(lengths)]
    if dtype == torch.bfloat16:     # both sides start from the same rounded rows
        data = [[torch.from_numpy(t).bfloat16().float().numpy() for t in req] for req in data]
    slots = [cache.open() for _ in lengths]
    done = [0] * len(lengths)
    cuts = [70, 1, 9, 1, 40]
    step = 0
    while any(d < n for d, n in zip(done, lengths)):
        entries, parts = [], []
        for i, n in enumerate(lengths):
            c = min(cuts[(step + i) % len(cuts)], n - done[i])
            if c <= 0:
                continue
            assert cache.prepare(slots[i], done[i], c)
            entries.append(StepEntry(slots[i], done[i], [0] * c))
            parts.append((i, done[i], c))
            done[i] += c
        batch, keep = build_batch(ops, cache, entries)
        parts = [parts[j] for j in batch.entry_order]
        host.table[:kv.table.shape[0]] = kv.table.cpu().numpy()[:host.table.shape[0]]        # the same pages on both sides
        q, k, v = (np.concatenate([data[i][j][p:p + c] for i, p, c in parts]) for j in range(3))
        slot_of = [slots[i] for i, p, c in parts for _ in range(c)]
        pos_of = [p + t for i, p, c in parts for t in range(c)]
        qd, kd, vd = dev(q, dtype), dev(k, dtype), dev(v, dtype)
        ops.qk_norm_rope_store(qd, kd, vd, dev(qw), dev(kw), 1e-5, dev(inv_freq), hd, heads, kv_heads, hd, batch, kv)
        out = torch.empty_like(qd)
        ops.paged_attention(qd, out, heads, kv_heads, hd, 1 / math.sqrt(hd), window, batch, kv)
        rows = len(pos_of)
        q_ref = ref.qk_norm_rope(q.reshape(rows, heads, hd), qw, 1e-5, inv_freq, hd, 0, pos_of).reshape(rows, -1)
        k_ref = ref.qk_norm_rope(k.reshape(rows, kv_heads, hd), kw, 1e-5, inv_freq, hd, 0, pos_of).reshape(rows, -1)
        if dtype == torch.bfloat16:
            q_ref = torch.from_numpy(q_ref).bfloat16().float().numpy()
            k_ref = torch.from_numpy(k_ref).bfloat16().float().numpy()
        host.store(k_ref, v, slot_of, pos_of, layer)
        want = host.attend(q_ref, slot_of, pos_of, layer, heads, 1 / math.sqrt(hd), window)
        close(qd.float().cpu().numpy(), q_ref, tol)
        close(out.float().cpu().numpy(), want, tol)
        step += 1
    used = sorted({int(p) for s in slots for p in kv.table[s].cpu().tolist() if p >= 0})
    close(kv.k[used, layer].float().cpu().numpy(), host.k[used, layer], tol)
    assert np.array_equal(kv.v[used, layer].float().cpu().numpy(), host.v[used, layer])       # values are copied as they came
    assert float(kv.k[:, 0].float().abs().max()) == 0                                        # the other layer's pages


def test_sampling_kernel_equals_the_cpp_sampler(ops):
    vocab, rows = 1000, 6
    rng = np.random.RandomState(9)
    logits = (rng.randn(rows, vocab) * 3).astype(np.float32)
    seen = (rng.rand(rows, vocab) < 0.1).astype(np.uint8)
    settings = [(0.0, 50, 1.0, 1.0), (0.8, 1, 1.0, 1.3), (0.7, 12, 1.0, 1.0), (1.3, 40, 0.6, 1.1), (0.1, 50, 1.0, 1.05), (2.0, 128, 0.95, 1.0)]
    u = rng.rand(rows).astype(np.float32)
    fparams = np.array([[t, p, pen, u[i]] for i, (t, k, p, pen) in enumerate(settings)], dtype=np.float32)
    iparams = np.array([[k, i, -1] for i, (t, k, p, pen) in enumerate(settings)], dtype=np.int32)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    seen_gpu = torch.from_numpy(seen).to(DEV)
    ops.sample(dev(logits), dev(fparams).reshape(-1), torch.from_numpy(iparams).to(DEV).reshape(-1), seen_gpu, out)
    want = [ref.sample(logits[i], t, k, p, pen, seen[i], u[i]) for i, (t, k, p, pen) in enumerate(settings)]
    assert out.cpu().tolist() == want

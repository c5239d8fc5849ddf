"""Each HIP kernel alone against a plain torch / plain-implementation reference, at sizes
other than the engine's tiny configurations (widths and vocabularies that are no power
of two, head sizes in steps of 16, odd head counts and groups)."""
import math

import pytest
import torch

import plain_lfm2 as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from kernel_ops import HipOps
    return HipOps(DEV)


def randn(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1.6e-2)


# ---------------------------------------------------------------- row-wise kernels
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("vocab,width,rows", [(331, 96, 7), (1000, 1030, 33)])
def test_embed(ops, dtype, vocab, width, rows):
    table = randn(vocab, width, seed=1, dtype=dtype)
    ids = torch.randint(0, vocab, (rows,), generator=torch.Generator().manual_seed(2),
                        dtype=torch.int32).to(DEV)
    out = torch.empty(rows, width, device=DEV)
    ops.embed(table, ids, out)
    assert torch.equal(out, table[ids.long()].float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(5, 96), (3, 1000), (9, 4100), (7, 1024), (4, 4096), (3, 516), (5, 2052), (70, 1024), (131, 260), (65, 1000)])
def test_rmsnorm_with_delta_and_rows(ops, dtype, rows, width):
    x = randn(rows, width, seed=3)
    delta = randn(rows, width, seed=4, dtype=dtype)
    w = 1 + randn(width, seed=5, scale=0.1)
    eps = 3e-5
    ref_sum = x.double() + delta.double()
    ref = plain.rmsnorm(ref_sum.cpu(), w.cpu(), eps)
    # all rows, sum written back
    x1 = x.clone()
    out = torch.empty(rows, width, dtype=dtype, device=DEV)
    ops.rmsnorm(x1, w, eps, out, delta=delta)
    torch.testing.assert_close(x1.double().cpu(), ref_sum.cpu(), rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(out.double().cpu(), ref, **tol(dtype))
    # listed rows only, x untouched
    x2 = x.clone()
    picked = list(range(rows - 1, -1, -1)) if rows >= 64 else [rows - 1, 0, rows // 2]
    idx = torch.tensor(picked, dtype=torch.int32, device=DEV)
    out2 = torch.empty(len(picked), width, dtype=dtype, device=DEV)
    ops.rmsnorm(x2, w, eps, out2, delta=delta, rows=idx)
    assert torch.equal(x2, x)
    torch.testing.assert_close(out2.double().cpu(), ref[idx.long().cpu()], **tol(dtype))
    # no delta
    out3 = torch.empty(rows, width, dtype=dtype, device=DEV)
    ops.rmsnorm(x2, w, eps, out3)
    torch.testing.assert_close(out3.double().cpu(), plain.rmsnorm(x.cpu(), w.cpu(), eps), **tol(dtype))


def test_rmsnorm_reference_vector(ops):
    # tests/reference_test.cpp:29-31: {1,2,3,4}, w = 1, eps 1e-5 -> y0 = 1/sqrt(7.5 + 1e-5)
    x = torch.tensor([[1., 2., 3., 4.]], device=DEV)
    out = torch.empty_like(x)
    ops.rmsnorm(x, torch.ones(4, device=DEV), 1e-5, out)
    assert abs(float(out[0, 0]) - 1 / math.sqrt(7.5 + 1e-5)) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,ff", [(11, 352), (3, 4608), (5, 100), (2, 8)])
def test_swiglu(ops, dtype, rows, ff):
    gu = randn(rows, 2 * ff, seed=6, scale=2.0, dtype=dtype)
    out = torch.empty(rows, ff, dtype=dtype, device=DEV)
    ops.swiglu(gu, out)
    g, u = gu[:, :ff].double().cpu(), gu[:, ff:].double().cpu()
    torch.testing.assert_close(out.double().cpu(), plain.silu(g) * u, **tol(dtype))
    zero = torch.zeros(2, 2 * ff, dtype=dtype, device=DEV)
    zero[:, ff:] = 3.0
    out0 = torch.empty(2, ff, dtype=dtype, device=DEV)
    ops.swiglu(zero, out0)   # gate 0 -> 0
    assert float(out0.abs().max()) == 0.0


@pytest.mark.parametrize("M,N,K", [(1, 331, 96), (67, 130, 77), (200, 65, 1030), (5, 1000, 64)])
def test_gemm_f32_is_true_32bit_and_row_independent(ops, M, N, K):
    x, w, b = randn(M, K, seed=7), randn(N, K, seed=8), randn(N, seed=9)
    out = torch.empty(M, N, device=DEV)
    ops.linear(x, w, out, bias=b)
    ref = x.double().cpu() @ w.double().cpu().T + b.double().cpu()
    torch.testing.assert_close(out.double().cpu(), ref, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    # a row gives the same bits alone as inside the batch
    one = torch.empty(1, N, device=DEV)
    ops.linear(x[M // 2:M // 2 + 1], w, one, bias=b)
    assert torch.equal(one[0], out[M // 2])


def test_linear_bf16_and_stored_f32_matrix(ops):
    M, N, K = 9, 200, 96
    x = randn(M, K, seed=10, dtype=torch.bfloat16)
    w = randn(N, K, seed=11, scale=0.1, dtype=torch.bfloat16)
    ref = x.double().cpu() @ w.double().cpu().T
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(x, w, out)
    torch.testing.assert_close(out.double().cpu(), ref, rtol=1.6e-2, atol=1.6e-2)
    out32 = torch.empty(M, N, device=DEV)
    ops.linear(x, w.float(), out32)     # matrix kept in 32-bit
    torch.testing.assert_close(out32.double().cpu(), ref, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("M,N,K", [(1, 331, 96), (77, 130, 96), (300, 1000, 352), (129, 48, 40),
                                   (512, 2048, 1024), (2041, 272, 4608)])
def test_library_product_called_directly(ops, M, N, K):
    """The bfloat16 products of many rows go to hipBLASLt directly; where it has a kernel
    the result is what torch's call of the libraries gives, with rows of x that are not
    dense and with a 32-bit output too, and a recorded call replays to the same bits."""
    big = randn(M, K + 8, seed=20, dtype=torch.bfloat16)
    x = big[:, :K]                                     # rows K + 8 apart
    w = randn(N, K, seed=21, scale=0.1, dtype=torch.bfloat16)
    ref = x.double().cpu() @ w.double().cpu().T
    outs = {}
    for direct in (True, False):
        ops.use_blaslt = direct
        try:
            out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            ops.linear(x, w, out)
            out32 = torch.empty(M, N, device=DEV)
            ops.linear(x, w, out32)
            outs[direct] = (out, out32)
        finally:
            ops.use_blaslt = True
    bound = 1.6e-2 * max(1.0, float(ref.abs().max()))
    for out, out32 in outs.values():
        assert float((out.double().cpu() - ref).abs().max()) <= bound
        assert torch.equal(out32, out.float())
    assert float((outs[True][0].float() - outs[False][0].float()).abs().max()) <= bound
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.linear(x, w, out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.linear(x, w, out)
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, outs[True][0])


# ---------------------------------------------------------------- cache-backed kernels
from kernel_harness import build_batch, make_cache  # noqa: E402


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,taps,bias", [(2, 3, False), (96, 5, True), (1030, 4, False), (64, 1, True)])
def test_short_conv_whole_chunked_and_token_by_token(ops, dtype, width, taps, bias):
    from celeg_amd.engine import StepEntry
    T = 23
    bcx = randn(T, 3 * width, seed=12, dtype=dtype)
    w = randn(width, taps, seed=13)
    b = randn(width, seed=14) if bias else None
    ref = plain.short_conv(bcx.cpu(), w.cpu(), b.cpu() if bias else None)
    for cuts in ([T], [1] * T, [7, 2, 1, 9, 4], [3, 20], [20, 3], [1, 1, 21]):
        cache = make_cache(0, 0, 0, dtype, states=[(0, "bx", (taps, width))])
        slot_other = cache.open()     # a neighbour slot whose state must stay zero
        slot = cache.open()
        state = cache.layer_cache(0).states["bx"]
        outs, pos = [], 0
        for n in cuts:
            batch, keep = build_batch(ops, cache, [StepEntry(slot, pos, [0] * n)])
            out = torch.empty(n, width, dtype=dtype, device=DEV)
            ops.short_conv(bcx[pos:pos + n].contiguous(), w, b, state, out, batch)
            torch.cuda.synchronize()
            outs.append(out)
            pos += n
        got = torch.cat(outs).double().cpu()
        torch.testing.assert_close(got, ref, **tol(dtype))
        assert float(state[slot_other].abs().max()) == 0.0
        bx = (bcx[:, :width].float() * bcx[:, 2 * width:].float())
        want_state = torch.zeros(taps, width, device=DEV)
        want_state[max(0, taps - T):] = bx[max(0, T - taps):]
        torch.testing.assert_close(state[slot], want_state, rtol=0, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,taps,bias", [(128, 3, True), (1032, 4, False), (96, 2, True), (64, 5, False)])
def test_short_conv_long_portions_of_several_requests(ops, dtype, width, taps, bias):
    """Steps of 64 and more tokens (the kernel that takes eight tokens in a row per thread):
    two requests per step, so that blocks of eight tokens straddle the border between them, begin
    at a request's first token, and continue from its state at positions inside a block."""
    from celeg_amd.engine import StepEntry
    lengths = [131, 77]
    data = [randn(n, 3 * width, seed=60 + i, dtype=dtype) for i, n in enumerate(lengths)]
    w = randn(width, taps, seed=63)
    b = randn(width, seed=64) if bias else None
    cache = make_cache(0, 0, 0, dtype, states=[(0, "bx", (taps, width))], slots=4)
    slots = [cache.open() for _ in lengths]
    state = cache.layer_cache(0).states["bx"]
    got = [[] for _ in lengths]
    pos = [0, 0]
    for cuts in ((70, 37), (33, 40), (28, 0)):
        entries, parts = [], []
        for i, n in enumerate(cuts):
            if n:
                entries.append(StepEntry(slots[i], pos[i], [0] * n))
                parts.append((i, pos[i], n))
        batch, keep = build_batch(ops, cache, entries)
        parts = [parts[j] for j in batch.entry_order]
        bcx = torch.cat([data[i][p:p + n] for i, p, n in parts]).contiguous()
        out = torch.empty(bcx.shape[0], width, dtype=dtype, device=DEV)
        ops.short_conv(bcx, w, b, state, out, batch)
        torch.cuda.synchronize()
        row = 0
        for i, p, n in parts:
            got[i].append(out[row:row + n].double().cpu())
            row += n
            pos[i] += n
    assert pos == lengths
    for i in range(len(lengths)):
        ref = plain.short_conv(data[i].cpu(), w.cpu(), b.cpu() if bias else None)
        torch.testing.assert_close(torch.cat(got[i]), ref, **tol(dtype))
        bx = data[i][:, :width].float() * data[i][:, 2 * width:].float()
        torch.testing.assert_close(state[slots[i]], bx[-taps:], rtol=0, atol=0)


@pytest.mark.parametrize("block_tokens", [0, 4])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,taps", [(128, 3), (264, 4), (96, 2)])
def test_short_conv_long_steps_with_single_tokens_and_short_portions(ops, dtype, width, taps, block_tokens):
    """The kernel for long steps updates the state itself: steps that hold a long portion beside
    requests that bring one, two or three tokens (several requests begin inside one block of
    tokens; portions shorter than the taps keep part of the old state).  Outputs and every
    request's state after every step against the plain convolution."""
    from celeg_amd.engine import StepEntry
    force = ops._lib("short_conv").celeg_short_conv_force_block_tokens
    force(block_tokens)          # tokens a thread: the default, or 4
    plans = [[66, 1, 1, 2, 3, 1], [65, 1, 2, 1, 1, 3], [70, 3, 1, 1, 2, 1], [64, 1, 1, 1, 1, 1]]
    n_req = len(plans[0])
    lengths = [sum(plan[i] for plan in plans) for i in range(n_req)]
    data = [randn(n, 3 * width, seed=80 + i, dtype=dtype) for i, n in enumerate(lengths)]
    w = randn(width, taps, seed=90)
    cache = make_cache(0, 0, 0, dtype, states=[(0, "bx", (taps, width))], slots=n_req + 1)
    idle = cache.open()
    slots = [cache.open() for _ in range(n_req)]
    state = cache.layer_cache(0).states["bx"]
    got = [[] for _ in range(n_req)]
    pos = [0] * n_req
    for plan in plans:
        entries = [StepEntry(slots[i], pos[i], [0] * n) for i, n in enumerate(plan)]
        batch, keep = build_batch(ops, cache, entries)
        parts = [(i, pos[i], plan[i]) for i in batch.entry_order]
        bcx = torch.cat([data[i][p:p + n] for i, p, n in parts]).contiguous()
        assert bcx.shape[0] >= 64
        out = torch.empty(bcx.shape[0], width, dtype=dtype, device=DEV)
        ops.short_conv(bcx, w, None, state, out, batch)
        torch.cuda.synchronize()
        row = 0
        for i, p, n in parts:
            got[i].append(out[row:row + n].double().cpu())
            row += n
            pos[i] += n
        for i in range(n_req):
            bx = data[i][:pos[i], :width].float() * data[i][:pos[i], 2 * width:].float()
            want = torch.zeros(taps, width, device=DEV)
            want[max(0, taps - pos[i]):] = bx[max(0, pos[i] - taps):]
            torch.testing.assert_close(state[slots[i]], want, rtol=0, atol=0)
        assert float(state[idle].abs().max()) == 0.0
    force(0)
    for i in range(n_req):
        ref = plain.short_conv(data[i].cpu(), w.cpu(), None)
        torch.testing.assert_close(torch.cat(got[i]), ref, **tol(dtype))


def test_short_conv_reference_vector(ops):
    # tests/reference_test.cpp:68-73: hidden 2, L 3, bcx {1,1 | 1,1 | 2,4}, weights
    # {1,2,3 ; 1,2,3} channel-major, position 0, zero state -> {6, 12}
    from celeg_amd.engine import StepEntry
    cache = make_cache(0, 0, 0, torch.float32, states=[(0, "bx", (3, 2))])
    slot = cache.open()
    batch, keep = build_batch(ops, cache, [StepEntry(slot, 0, [0])])
    bcx = torch.tensor([[1., 1., 1., 1., 2., 4.]], device=DEV)
    w = torch.tensor([[1., 2., 3.], [1., 2., 3.]], device=DEV)
    out = torch.empty(1, 2, device=DEV)
    ops.short_conv(bcx, w, None, cache.layer_cache(0).states["bx"], out, batch)
    assert out.cpu().tolist() == [[6.0, 12.0]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_short_conv_vector_tells_the_three_thirds_of_bcx_apart(ops, dtype):
    # worked by hand from src/backend/cpu/kernels/convolution.cpp:14-27 (see test_plain.py):
    # rows {2,3,5}, {7,11,13}; taps {1,1} -> {30, 1111} (C and x swapped: 1079; B and C: 1106);
    # taps {2,1} -> {30, 1221} (the filter reversed: 2112).  In one step, and token by token
    # through the saved state.  All values are exact in bfloat16 except 1111 and 1221.
    from celeg_amd.engine import StepEntry
    rows = torch.tensor([[2., 3., 5.], [7., 11., 13.]], device=DEV).to(dtype)
    for taps, want in (([1., 1.], [30., 1111.]), ([2., 1.], [30., 1221.])):
        w = torch.tensor([taps], device=DEV)
        for cuts in ([2], [1, 1]):
            cache = make_cache(0, 0, 0, dtype, states=[(0, "bx", (2, 1))])
            slot = cache.open()
            got, pos = [], 0
            for c in cuts:
                batch, keep = build_batch(ops, cache, [StepEntry(slot, pos, [0] * c)])
                out = torch.empty(c, 1, dtype=dtype, device=DEV)
                ops.short_conv(rows[pos:pos + c].contiguous(), w, None,
                               cache.layer_cache(0).states["bx"], out, batch)
                got += out.float().cpu().reshape(-1).tolist()
                pos += c
            if dtype == torch.float32:
                assert got == want
            else:
                assert got[0] == want[0] and abs(got[1] - want[1]) <= 4.0   # far from 1079, 1106, 2112


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("head_dim", [2, 64])
def test_q_and_k_are_normalised_before_they_are_rotated(ops, dtype, head_dim):
    """q = k = {3, 4}, norm weight {1, 2}, eps 0, position 1, one pair of frequency 1: the
    kernel that normalises, rotates and stores gives {-1.44557, 1.93658}
    (src/backend/cpu/kernels/rope.cpp:95-108, worked by hand in test_plain.py); rotating
    before normalising would give {-0.4936, 2.6506}.  With head size 64 the pair lies at
    places 0 and 32, every other place is zero and every other frequency tiny."""
    from celeg_amd.engine import StepEntry
    from test_plain import QK_NORM_THEN_ROPE
    half = head_dim // 2
    cache = make_cache(1, head_dim, 1, dtype, n_pages=2)
    kv = cache.layer_cache(0).kv
    slot = cache.open()
    assert cache.prepare(slot, 0, 2)
    batch, keep = build_batch(ops, cache, [StepEntry(slot, 0, [0, 0])])
    row = torch.zeros(2, head_dim)
    row[1, 0], row[1, half] = 3.0, 4.0
    # (the mean of squares is over head_dim values: scaled by s = sqrt(head_dim / 2), the row's
    # 1/rms is that of {3, 4} alone and the result is s times the hand-worked one)
    s = math.sqrt(head_dim / 2)
    row *= s
    q = row.to(dtype).to(DEV)
    k, v = q.clone(), q.clone()
    weight = torch.ones(head_dim)
    weight[half] = 2.0
    weight = weight.to(DEV)
    inv_freq = torch.zeros(half)
    inv_freq[0] = 1.0
    ops.qk_norm_rope_store(q, k, v, weight, weight, 0.0, inv_freq.to(DEV), head_dim, 1, 1, head_dim,
                           batch, kv)
    torch.cuda.synchronize()
    page = cache.table_host(slot, 0)
    stored_k = kv.k[page, 0, 0, 1].float().cpu()            # [page, layer, head, token, :]
    bound = (1e-5 if dtype == torch.float32 else 2e-2) * s
    for got in (q[1].float().cpu(), stored_k):
        assert abs(float(got[0]) - s * QK_NORM_THEN_ROPE[0]) <= bound
        assert abs(float(got[half]) - s * QK_NORM_THEN_ROPE[1]) <= bound
    # the values are stored as they came (transposed inside the page: [.., head_dim, token])
    assert float(kv.v[page, 0, 0, half, 1]) == float(v[1, half])


def attention_case(ops, dtype, heads, kv_heads, head_dim, lengths, cuts, window=None,
                   qk_norm=True, theta=10000.0, rotary_dim=None, boost=None, page_tokens=16):
    """Runs norm+rope+store and attention for several requests cut into steps (one step
    holds the next cut of every request) and compares with the plain whole-sequence
    functions."""
    from celeg_amd.engine import StepEntry
    rotary_dim = head_dim if rotary_dim is None else rotary_dim
    n_layers, layer = 3, 1
    total = sum(lengths)
    cache = make_cache(kv_heads, head_dim, n_layers, dtype, page_tokens=page_tokens,
                       n_pages=(total + page_tokens * len(lengths)) // page_tokens + 2,
                       max_context=max(lengths) + 16, slots=max(4, len(lengths) + 1))
    kv = cache.layer_cache(layer).kv
    qw = 1 + randn(head_dim, seed=20, scale=0.1) if qk_norm else None
    kw = 1 + randn(head_dim, seed=21, scale=0.1) if qk_norm else None
    inv_freq = torch.tensor(plain.rope_inverse_frequencies(theta, rotary_dim),
                            dtype=torch.float64).float().to(DEV) if rotary_dim else None
    scale = 1 / math.sqrt(head_dim)
    reqs = []
    for i, n in enumerate(lengths):
        q = randn(n, heads * head_dim, seed=30 + i, dtype=dtype)
        k = randn(n, kv_heads * head_dim, seed=40 + i, dtype=dtype)
        v = randn(n, kv_heads * head_dim, seed=50 + i, dtype=dtype)
        if boost is not None and n > boost[1]:   # one far key stands out for one query
            far, row = boost
            k[far] *= 6.0
            q[row] = (k[far].float().reshape(kv_heads, 1, head_dim) *
                      torch.ones(1, heads // kv_heads, 1, device=DEV)).reshape(-1).to(dtype) * 2
        reqs.append((q, k, v, cache.open()))
    got = [[] for _ in lengths]
    pos = [0] * len(lengths)
    step = 0
    while any(p < n for p, n in zip(pos, lengths)):
        entries, parts = [], []
        for i, n in enumerate(lengths):
            if pos[i] >= n:
                continue
            c = min(cuts[(step + i) % len(cuts)], n - pos[i])
            assert cache.prepare(reqs[i][3], pos[i], c)
            entries.append(StepEntry(reqs[i][3], pos[i], [0] * c))
            parts.append((i, pos[i], c))
            pos[i] += c
        batch, keep = build_batch(ops, cache, entries)
        parts = [parts[j] for j in batch.entry_order]     # single tokens lie first in the rows
        q = torch.cat([reqs[i][0][p:p + c] for i, p, c in parts]).contiguous()
        k = torch.cat([reqs[i][1][p:p + c] for i, p, c in parts]).contiguous()
        v = torch.cat([reqs[i][2][p:p + c] for i, p, c in parts]).contiguous()
        ops.qk_norm_rope_store(q, k, v, qw, kw, 1e-5, inv_freq, rotary_dim, heads, kv_heads,
                               head_dim, batch, kv)
        out = torch.empty_like(q)
        ops.paged_attention(q, out, heads, kv_heads, head_dim, scale, window, batch, kv)
        torch.cuda.synchronize()
        row = 0
        for i, p, c in parts:
            got[i].append(out[row:row + c].double().cpu())
            row += c
        step += 1
    for i, n in enumerate(lengths):
        q, k, v, _ = reqs[i]
        qf = q.double().cpu().reshape(n, heads, head_dim)
        kf = k.double().cpu().reshape(n, kv_heads, head_dim)
        vf = v.double().cpu().reshape(n, kv_heads, head_dim)
        if qk_norm:
            qf = plain.head_rmsnorm(qf, qw.cpu(), 1e-5)
            kf = plain.head_rmsnorm(kf, kw.cpu(), 1e-5)
        if rotary_dim:
            cos, sin = plain.rope_cos_sin(range(n), theta, rotary_dim)
            qf, kf = plain.rope_apply(qf, cos, sin), plain.rope_apply(kf, cos, sin)
        if dtype == torch.bfloat16:   # the kernels store q and k rounded
            qf, kf = qf.bfloat16().double(), kf.bfloat16().double()
        ref = plain.causal_attention(qf, kf, vf, window=window).reshape(n, -1)
        torch.testing.assert_close(torch.cat(got[i]), ref, **tol(dtype),
                                   msg=lambda m: f"request {i}: {m}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_tokens", [(16, 8, 64, 16), (4, 2, 128, 16), (10, 5, 32, 16),
                                                                 (16, 8, 64, 2), (10, 5, 32, 6), (4, 2, 128, 1)])
def test_norm_rope_store_of_a_long_step_equals_short_steps(ops, dtype, heads, kv_heads, head_dim, page_tokens):
    """A step of thousands of rows takes four rows a thread (values of four neighbouring rows
    leave as one store); the same rows in steps of a few hundred take one row a thread.  Three
    requests whose portions start at positions 0, 5 and 1, so that runs of four rows start on a
    multiple of four, in the middle of one, and straddle the border between two requests: the
    queries and both caches must come out the same bit for bit.  With pages of 1, 2 and 6 tokens
    four neighbouring rows do not lie side by side in one page (or not at an address that a store
    of four takes): they must go row by row, and what the pages hold is compared with the rows
    themselves."""
    from celeg_amd.engine import StepEntry
    starts, lengths = [0, 5, 1], [2503, 1202, 650]
    n_layers, layer = 2, 1
    qw = 1 + randn(head_dim, seed=20, scale=0.1)
    kw = 1 + randn(head_dim, seed=21, scale=0.1)
    inv_freq = torch.tensor(plain.rope_inverse_frequencies(10000.0, head_dim), dtype=torch.float64).float().to(DEV)
    total = sum(lengths)
    q0 = randn(total, heads * head_dim, seed=1, dtype=dtype)
    k0 = randn(total, kv_heads * head_dim, seed=2, dtype=dtype)
    v0 = randn(total, kv_heads * head_dim, seed=3, dtype=dtype)
    results = []
    for pieces in (1, 17):                       # the whole step, then steps of at most 260 rows
        cache = make_cache(kv_heads, head_dim, n_layers, dtype, page_tokens=page_tokens,
                           n_pages=(total + sum(starts)) // page_tokens + 8, max_context=max(lengths) + 16, slots=4)
        kv = cache.layer_cache(layer).kv
        slots = [cache.open() for _ in lengths]
        for slot, start in zip(slots, starts):   # what lies before the portions is of no interest here
            if start:
                assert cache.prepare(slot, 0, start)
        q_out = torch.empty_like(q0)
        done = [0] * len(lengths)
        for piece in range(pieces):
            entries, rows = [], []
            row0 = 0
            for i, n in enumerate(lengths):
                c = n if pieces == 1 else min((n + pieces - 1) // pieces, n - done[i])
                if c > 0:
                    assert cache.prepare(slots[i], starts[i] + done[i], c)
                    entries.append(StepEntry(slots[i], starts[i] + done[i], [0] * c))
                    rows.append((row0 + done[i], c))
                    done[i] += c
                row0 += n
            if not entries:
                continue
            batch, keep = build_batch(ops, cache, entries)
            rows = [rows[j] for j in batch.entry_order]
            index = torch.cat([torch.arange(r, r + c) for r, c in rows]).to(DEV)
            q, k, v = q0[index].contiguous(), k0[index].contiguous(), v0[index].contiguous()
            ops.qk_norm_rope_store(q, k, v, qw, kw, 1e-5, inv_freq, head_dim, heads, kv_heads, head_dim, batch, kv)
            q_out[index] = q
        torch.cuda.synchronize()
        # the pools page by page in the order of the requests' tables (the page numbers may differ)
        table = kv.table.cpu()
        pages = [int(table[slot, p]) for slot, start, n in zip(slots, starts, lengths)
                 for p in range((start + n + page_tokens - 1) // page_tokens)]
        results.append((q_out.clone(), kv.k[pages].clone(), kv.v[pages].clone(), [int(x) for x in starts]))
        # the values are stored as they came: position p of a request in page p // page_tokens, place p % page_tokens
        row0 = 0
        for slot, start, n in zip(slots, starts, lengths):
            mine = table[slot, :(start + n + page_tokens - 1) // page_tokens].long().to(DEV)
            held = kv.v[mine, layer].permute(1, 2, 0, 3).reshape(kv_heads, head_dim, -1)[:, :, start:start + n]
            assert torch.equal(held.permute(2, 0, 1).reshape(n, -1), v0[row0:row0 + n])
            row0 += n
    (qa, ka, va, _), (qb, kb, vb, _) = results
    assert torch.equal(qa, qb)
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    assert float(ka.float().abs().max()) > 0 and float(va.float().abs().max()) > 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [
    (6, 3, 48), (5, 5, 16), (8, 1, 128), (4, 2, 80), (16, 8, 64), (3, 3, 64), (6, 2, 96),
    (8, 2, 32), (12, 4, 128)])
def test_attention_mixed_steps(ops, dtype, heads, kv_heads, head_dim):
    attention_case(ops, dtype, heads, kv_heads, head_dim, lengths=[70, 33, 150],
                   cuts=[7, 1, 2, 30, 1, 16, 5])


@pytest.mark.parametrize("page_tokens", [16, 32, 64, 128])
@pytest.mark.parametrize("heads,kv_heads,head_dim", [(4, 2, 64), (8, 1, 128), (3, 1, 64)])
def test_attention_long_prompt_then_decode_rows(ops, heads, kv_heads, head_dim, page_tokens):
    """A long portion through the matrix-core kernel, then rows one by one through the
    split-key kernel (64 keys a wavefront), several requests per step, at several page sizes."""
    attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[333, 150, 420],
                   cuts=[300] + [1] * 40, boost=(2, 331), page_tokens=page_tokens)


def test_fast_and_general_attention_agree(ops):
    """The same bfloat16 case through the general kernel."""
    ops.attention_impl = "general"
    try:
        attention_case(ops, torch.bfloat16, 4, 2, 64, lengths=[333, 150], cuts=[300] + [1] * 40)
    finally:
        ops.attention_impl = "auto"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_far_key_stands_out(ops, dtype):
    # query 299 is built to look at key 3, hundreds of keys back and in the first page
    attention_case(ops, dtype, 4, 2, 64, lengths=[300], cuts=[64, 1, 1, 50], boost=(3, 299),
                   qk_norm=False, rotary_dim=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_window_edge(ops, dtype):
    # with a window of 20 the boosted key 3 is visible to row 22 and not to row 23
    attention_case(ops, dtype, 4, 2, 32, lengths=[90], cuts=[5, 1, 13, 2], window=20,
                   boost=(3, 22), qk_norm=False, rotary_dim=0)
    attention_case(ops, dtype, 4, 2, 32, lengths=[90], cuts=[5, 1, 13, 2], window=20,
                   boost=(3, 23), qk_norm=False, rotary_dim=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_partial_rotary_and_other_page_size(ops, dtype):
    attention_case(ops, dtype, 4, 4, 64, lengths=[45, 80], cuts=[9, 1, 3],
                   rotary_dim=32, theta=1e6, page_tokens=32)


def test_attention_window_fast_kernels(ops):
    # head size 64: the matrix-core and split-key kernels, window 70, pages of 32
    attention_case(ops, torch.bfloat16, 4, 2, 64, lengths=[260], cuts=[100, 1, 1, 60, 1],
                   window=70, boost=(31, 100), qk_norm=False, rotary_dim=0, page_tokens=32)
    attention_case(ops, torch.bfloat16, 4, 2, 64, lengths=[260], cuts=[100, 1, 1, 60, 1],
                   window=70, boost=(31, 101), qk_norm=False, rotary_dim=0, page_tokens=32)


@pytest.mark.parametrize("rows_per_tile", [64, 128])
@pytest.mark.parametrize("form", [1, 2, 3, 4])
@pytest.mark.parametrize("heads,kv_heads,head_dim,page_tokens", [
    (4, 2, 64, 16), (2, 1, 128, 32), (3, 3, 96, 16), (4, 1, 32, 64), (2, 2, 64, 128), (6, 2, 64, 16),
    (3, 1, 96, 32)])
def test_attention_rows_tiles_and_forms(ops, rows_per_tile, form, heads, kv_heads, head_dim, page_tokens):
    """Portions of many row tiles (tiles with an odd and an even number of rounds of keys,
    so that the wavefronts that take the rounds in turn get equal and unequal shares),
    continued at a position inside a tile, at either tile size, with the rounds of keys taken
    by one set of wavefronts, shared between two, or by two sets that each take a query head
    of a group (groups of 1, 2, 3 and 4 heads), or shared between four sets (tiles of 64 rows and
    heads up to 64 only: some sets then have no round at all in the first tiles); then the same
    with a window that ends inside a round of keys.  Pages shorter and longer than a round."""
    if form == 4 and (rows_per_tile != 64 or head_dim > 64):
        from kernel_ops import KernelError
        ops.attention_rows_per_tile, ops.attention_rows_form = rows_per_tile, form
        try:
            with pytest.raises(KernelError):
                attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[130], cuts=[130],
                               page_tokens=page_tokens)
        finally:
            ops.attention_rows_per_tile = ops.attention_rows_form = 0
        return
    ops.attention_rows_per_tile = rows_per_tile
    ops.attention_rows_form = form
    try:
        attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[717, 150, 390],
                       cuts=[330, 61, 200], boost=(2, 700), page_tokens=page_tokens)
        attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[500],
                       cuts=[270, 230], window=150, boost=(301, 450), qk_norm=False, rotary_dim=0,
                       page_tokens=page_tokens)
        attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[500],
                       cuts=[270, 230], window=150, boost=(300, 450), qk_norm=False, rotary_dim=0,
                       page_tokens=page_tokens)
    finally:
        ops.attention_rows_per_tile = 0
        ops.attention_rows_form = 0


def test_attention_decode_of_many_requests_and_heads(ops):
    """33 requests x 16 key/value heads decoding together: enough workgroups for the form
    with 8 wavefronts a workgroup (more rounds of keys than wavefronts; a boosted far key)."""
    attention_case(ops, torch.bfloat16, 32, 16, 64, lengths=[600 + 7 * i for i in range(33)],
                   cuts=[590] + [1] * 40, boost=(5, 598))


@pytest.mark.parametrize("heads,kv_heads,head_dim,page_tokens", [
    (8, 2, 64, 16), (3, 1, 64, 64), (6, 1, 128, 32), (16, 1, 64, 16), (40, 2, 64, 32), (4, 4, 64, 16),
    (32, 8, 64, 16), (12, 2, 128, 16), (4, 2, 64, 16), (8, 1, 128, 32)])
@pytest.mark.parametrize("whole", [0, 1, 4, 16])
def test_attention_decode_one_workgroup_per_request(ops, heads, kv_heads, head_dim, page_tokens, whole):
    """(whole 0: the same rounds of keys as workgroups of their own, joined by a second kernel;
    4 and 16: parts of 4 and of 16 rounds a workgroup, a wavefront per round, joined likewise:
    contexts that fill a part, leave its end empty, and need several.)
    The decode kernel that walks a request's whole context in one workgroup, the query
    heads of a key/value head being the rows of its matrix instructions (groups of 1 to 20
    heads; more than 16 take two workgroups): long contexts (more rounds of 64 keys than
    wavefronts), a boosted far key, a window that cuts the first round of keys, the last round
    ending inside a page."""
    ops.attention_decode_whole = min(whole, 1) if whole <= 1 else 0
    if whole > 1:
        ops.decode_part_thresholds = (0, 1 << 30) if whole == 4 else (0, 0)
    try:
        attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[1300, 150, 70],
                       cuts=[1260] + [1] * 40, boost=(2, 1290), page_tokens=page_tokens)
        attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[400],
                       cuts=[300, 1, 1, 60, 1] + [1] * 40, window=150, boost=(231, 380),
                       qk_norm=False, rotary_dim=0, page_tokens=page_tokens)
        attention_case(ops, torch.bfloat16, heads, kv_heads, head_dim, lengths=[400],
                       cuts=[300, 1, 1, 60, 1] + [1] * 40, window=150, boost=(230, 380),
                       qk_norm=False, rotary_dim=0, page_tokens=page_tokens)
    finally:
        ops.attention_decode_whole = -1
        ops.decode_part_thresholds = (64, 256)


def test_attention_rows_with_the_block_table_looked_up_in_memory(ops):
    """A tile whose pages do not fit the room that the kernel keeps for them in LDS (contexts
    of several ten thousand tokens) looks them up in memory instead: forced here at a small
    size by lowering that room to 8 entries, against the same case with the table in LDS."""
    lib = ops._lib("attention_fast")
    lib.celeg_attention_rows_pages_in_lds(8)
    try:
        attention_case(ops, torch.bfloat16, 4, 2, 64, lengths=[717, 150, 390], cuts=[330, 61, 200],
                       boost=(2, 700))
        attention_case(ops, torch.bfloat16, 2, 1, 128, lengths=[500], cuts=[270, 230], window=150,
                       boost=(301, 450), qk_norm=False, rotary_dim=0, page_tokens=32)
    finally:
        lib.celeg_attention_rows_pages_in_lds(0)


@pytest.mark.parametrize("head_dim,page_tokens", [(64, 16), (128, 16), (32, 32)])
def test_window_attention_never_reads_pages_it_has_given_back(ops, head_dim, page_tokens):
    """A window group hands back the pages that the window has passed; the device's block
    table still names them.  Another request takes them and fills them with infinities.  The
    first round of 64 keys of a tile starts at a multiple of 64, before the window's first
    key: the kernel must stay on the request's live pages there (a masked key has probability
    zero, and zero times infinity is not a number)."""
    from celeg_amd.engine import StepEntry
    window, heads, kv_heads = 40, 2, 1
    cache = make_cache(kv_heads, head_dim, 1, torch.bfloat16, n_pages=24, page_tokens=page_tokens, slots=2,
                       max_context=512, window=window)
    kv = cache.layer_cache(0).kv
    n = 330
    q = randn(n, heads * head_dim, seed=70, dtype=torch.bfloat16)
    k = randn(n, kv_heads * head_dim, seed=71, dtype=torch.bfloat16)
    v = randn(n, kv_heads * head_dim, seed=72, dtype=torch.bfloat16)
    slot = cache.open()
    got, pos, before = [], 0, set()
    for c in [150, 100, 1, 1, 78]:
        assert cache.prepare(slot, pos, c)          # gives back what lies before pos - window + 1
        held = set(cache.pages_held(slot)[0])
        free = [p for p in range(24) if p not in held]
        kv.k[free] = float("inf")                   # what another request may be writing there
        kv.v[free] = float("inf")
        fresh = sorted(held - before)               # pages handed out now hold someone's old, finite values
        kv.k[fresh] = randn(len(fresh), *kv.k.shape[1:], seed=73, dtype=torch.bfloat16)
        kv.v[fresh] = randn(len(fresh), *kv.v.shape[1:], seed=74, dtype=torch.bfloat16)
        before = held
        batch, keep = build_batch(ops, cache, [StepEntry(slot, pos, [0] * c)])
        qs, ks, vs = (t[pos:pos + c].contiguous() for t in (q, k, v))
        ops.qk_norm_rope_store(qs, ks, vs, None, None, 1e-5, None, 0, heads, kv_heads, head_dim, batch, kv)
        out = torch.empty_like(qs)
        ops.paged_attention(qs, out, heads, kv_heads, head_dim, 1 / math.sqrt(head_dim), window, batch, kv)
        got.append(out.double().cpu())
        pos += c
    got = torch.cat(got)
    assert torch.isfinite(got).all()
    ref = plain.causal_attention(q.double().cpu().reshape(n, heads, head_dim),
                                 k.double().cpu().reshape(n, kv_heads, head_dim),
                                 v.double().cpu().reshape(n, kv_heads, head_dim), window=window).reshape(n, -1)
    torch.testing.assert_close(got, ref, **tol(torch.bfloat16))


@pytest.mark.parametrize("whole,parts", [(0, (64, 256)), (0, (0, 1 << 30)), (0, (0, 0)), (1, (64, 256))])
@pytest.mark.parametrize("heads,kv_heads,head_dim,rotate,normed", [(16, 8, 64, True, True), (4, 1, 128, True, True),
                                                                   (6, 2, 64, False, True), (40, 2, 64, True, False)])
def test_attention_decode_that_prepares_and_writes_the_new_token_itself(ops, whole, parts, heads, kv_heads, head_dim,
                                                                        rotate, normed):
    """Decode steps whose attention kernel normalises and turns q and the new key, takes the new
    key and value as one more key and writes them into the pages, against qk_norm_rope_store
    followed by the attention: requests at positions 0, 1, 63, 64, 65 and further (a part that
    holds nothing but the new token; the first key of a round), parts of 1, 4 and 16 rounds and
    one workgroup a request, three steps in a row so that later steps read what earlier ones
    wrote; a window of 40 keys too.  Values must be written bit for bit; outputs and keys may
    differ by a rounding."""
    from celeg_amd.engine import StepEntry
    n_layers, layer, page_tokens = 2, 1, 16
    starts = [0, 1, 63, 64, 65, 200, 331]
    n = len(starts)
    qw = (1 + randn(head_dim, seed=40, scale=0.2)) if normed else None
    kw = (1 + randn(head_dim, seed=41, scale=0.2)) if normed else None
    inv_freq = torch.tensor(plain.rope_inverse_frequencies(10000.0, head_dim), dtype=torch.float64).float().to(DEV) if rotate else None
    scale = head_dim ** -0.5
    N = (heads + 2 * kv_heads) * head_dim
    ops.attention_decode_whole = whole
    saved = ops.decode_part_thresholds
    ops.decode_part_thresholds = parts
    try:
        for window in (None, 40):
            results = []
            for fused in (False, True):
                cache = make_cache(kv_heads, head_dim, n_layers, torch.bfloat16, page_tokens=page_tokens, n_pages=n * 24 + 4,
                                   max_context=352, slots=n, window=window)
                kv = cache.layer_cache(layer).kv
                slots = [cache.open() for _ in starts]
                # what lies before the first step: the same keys and values for both runs
                for i, (slot, start) in enumerate(zip(slots, starts)):
                    assert cache.prepare(slot, 0, start + 3)
                batch, keep = build_batch(ops, cache, [StepEntry(s, 0, [0]) for s in slots])      # (applies the tables)
                table = kv.table.cpu()
                g = torch.Generator().manual_seed(50)
                kv.k.copy_((torch.randn(kv.k.shape, generator=g) * 0.5).to(torch.bfloat16))
                kv.v.copy_((torch.randn(kv.v.shape, generator=g) * 0.5).to(torch.bfloat16))
                outs = []
                for step in range(3):
                    batch, keep = build_batch(ops, cache, [StepEntry(s, st + step, [0]) for s, st in zip(slots, starts)])
                    qkv = randn(n, N, seed=60 + step, dtype=torch.bfloat16)
                    q, k, v = qkv[:, :heads * head_dim], qkv[:, heads * head_dim:(heads + kv_heads) * head_dim], qkv[:, (heads + kv_heads) * head_dim:]
                    out = torch.zeros(n, heads * head_dim, dtype=torch.bfloat16, device=DEV)
                    if fused:
                        ops.attention_decode_fresh(q, k, v, out, qw, kw, 1e-6, inv_freq, heads, kv_heads, head_dim, scale,
                                                   window, batch, kv)
                    else:
                        ops.qk_norm_rope_store(q, k, v, qw, kw, 1e-6, inv_freq, head_dim if rotate else 0, heads, kv_heads,
                                               head_dim, batch, kv)
                        ops.paged_attention(q, out, heads, kv_heads, head_dim, scale, window, batch, kv)
                    torch.cuda.synchronize()
                    outs.append(out.float().clone())
                results.append((torch.stack(outs), kv.k.float().clone(), kv.v.clone()))
            (oa, ka, va), (ob, kb, vb) = results
            assert torch.equal(va, vb)
            assert float(oa.abs().max()) > 0 and not torch.isnan(ob).any()
            assert float(((ka - kb).abs() / (ka.abs() + kb.abs() + 1e-3)).max()) <= 2 ** -7
            assert float((ka != kb).float().mean()) < 0.01
            assert float((oa - ob).abs().max()) <= 2e-2 * float(oa.abs().max())
            assert float((oa - ob).abs().mean()) <= 2e-3 * float(oa.abs().max())
    finally:
        ops.attention_decode_whole = -1
        ops.decode_part_thresholds = saved

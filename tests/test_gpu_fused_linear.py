"""The fused skinny matrix products alone, against torch: every prologue and epilogue, at
row counts from 1 to 64 and sizes that are no multiple of the tiles."""
import pytest
import torch

import plain_lfm2 as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF = torch.bfloat16


@pytest.fixture(scope="module")
def ops():
    from kernel_ops import HipOps
    return HipOps(DEV)


def randn(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, ref, rel=1.5e-2):
    got, ref = got.double().cpu(), ref.double().cpu()
    bound = rel * max(1.0, float(ref.abs().max()))
    assert float((got - ref).abs().max()) <= bound, float((got - ref).abs().max())


SHAPES = [(1, 331, 96), (7, 64, 64), (8, 1024, 1024), (16, 130, 200), (17, 48, 4608),
          (33, 1000, 352), (64, 272, 1024)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_plain_rows_store_and_32bit_store_with_bias(ops, M, N, K):
    a = randn(M, K, seed=1, dtype=BF)
    w = randn(N, K, seed=2, scale=0.1, dtype=BF)
    b = randn(N, seed=3)
    ref = a.double() @ w.double().T + b.double()
    out = torch.empty(M, N, dtype=BF, device=DEV)
    ops.fused_linear(a, w, out, bias=b)
    close(out, ref)
    out32 = torch.empty(M, N, device=DEV)
    ops.fused_linear(a, w, out32, epilogue="store_f32", bias=b)
    close(out32, ref, rel=2e-3)
    # a row alone gives the same 32-bit result as inside the batch, up to the order in
    # which the wavefronts' partial sums are added (their number depends on the rows)
    one = torch.empty(1, N, device=DEV)
    ops.fused_linear(a[M // 2:M // 2 + 1], w, one, epilogue="store_f32", bias=b)
    if M <= 4:   # up to four rows share a layout (the same cut of the matrix instruction's tile into k-slices)
        assert torch.equal(one[0], out32[M // 2])
    close(one[0], out32[M // 2], rel=1e-5)


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("with_stats", [False, True])
def test_norm_prologue_with_and_without_partial_sums(ops, M, N, K, with_stats):
    h = randn(M + 3, K, seed=4)
    nw = 1 + randn(K, seed=5, scale=0.1)
    w = randn(N, K, seed=6, scale=0.1, dtype=BF)
    rows = torch.tensor([(3 * i + 1) % (M + 3) for i in range(M)], dtype=torch.int32, device=DEV)
    eps = 1e-5
    x = plain.rmsnorm(h.cpu(), nw.cpu(), eps)[rows.long().cpu()].to(BF)
    ref = x.double() @ w.double().cpu().T
    stats, blocks = None, 0
    if with_stats:   # partial sums over 5 uneven column blocks
        blocks = 5
        cuts = [0, K // 7, K // 3, K // 2, K - 8, K]
        stats = torch.zeros(80, blocks, device=DEV)
        for j in range(blocks):
            stats[:M + 3, j] = (h[:, cuts[j]:cuts[j + 1]] ** 2).sum(dim=1)
    out = torch.empty(M, N, dtype=BF, device=DEV)
    ops.fused_linear(h, w, out, norm_weight=nw, eps=eps, rows=rows, stats=stats, stat_blocks=blocks)
    close(out, ref)


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (8, 1024, 1024), (20, 200, 352), (64, 96, 4608),
                                   (3, 130, 72), (4, 1024, 4608), (7, 77, 352), (8, 1024, 4608),
                                   (13, 50, 1160), (16, 1024, 1024), (2, 36, 8), (5, 24, 40),
                                   (33, 1000, 96), (64, 8192, 64), (17, 14400, 32), (48, 1024, 2048)])
def test_residual_epilogue_adds_in_place_and_leaves_partial_sums(ops, M, N, K):
    a = randn(M, K, seed=7, dtype=BF)
    w = randn(N, K, seed=8, scale=0.1, dtype=BF)
    b = randn(N, seed=9)
    h = randn(M, N, seed=10)
    h0 = h.clone()
    blocks = ops.residual_stat_blocks(M, N, K)
    stats = torch.full((64, blocks), -1.0, device=DEV)
    ops.fused_linear(a, w, h, epilogue="residual", bias=b, stats_out=stats)
    assert ops.last_stat_blocks == blocks
    delta = (a.double() @ w.double().T + b.double())
    close(h, h0.double() + delta)
    # the product enters the sum rounded to bfloat16: what was added is the product rounded
    # (an element whose 32-bit sum lies at a rounding boundary may land one step away, never
    # more, and few do)
    added, rounded = (h - h0).double().cpu(), delta.to(BF).double().cpu()
    step = rounded.abs() * 2.0 ** -7 + 1e-30         # at least one step of bfloat16 at this size
    err = (added - rounded).abs()
    slack = 4e-6 * h0.abs().double().cpu().clamp_min(1.0) + 1e-6 * rounded.abs()   # 32-bit rounding of the sum
    assert bool((err <= step + slack).all()), float((err - step).max())
    assert float((err > slack).double().mean()) < 0.01
    torch.testing.assert_close(stats[:M].sum(dim=1), (h ** 2).sum(dim=1), rtol=1e-5, atol=1e-5)
    assert float(stats[M:].max()) == -1.0 if M < 64 else True


@pytest.mark.parametrize("M,N,K,form", [(1, 4100, 64, "norm"), (8, 65536, 256, "norm"), (16, 333, 96, "norm"), (5, 24, 40, "norm"),
                                        (9, 4100, 64, "rows"), (64, 65536, 64, "rows"), (33, 1000, 96, "rows"),
                                        (17, 20, 32, "rows"), (64, 4608, 1024, "rows"),
                                        (1, 4100, 64, "rows"), (4, 333, 96, "rows"), (8, 16384, 32, "rows"), (16, 1000, 40, "rows")])
def test_the_32bit_store_leaves_the_best_of_every_share_of_a_row(ops, M, N, K, form):
    """An output head's product writes, beside the logits, the best (logit, index) of the columns of
    every workgroup (or wavefront): their maximum over a row is the row's largest logit at its
    lowest index, and the merging kernel gives that token.  Two equal weight rows make equal logits:
    the lower index wins, wherever the two lie."""
    h = randn(M, K, seed=21)
    nw = 1 + randn(K, seed=22, scale=0.1)
    w = randn(N, K, seed=23, scale=0.1, dtype=BF)
    for r, (lo, hi) in enumerate([(N // 3, N - 1), (0, N // 2), (N - 2, N - 1), (1, 17 % N)]):
        boost = randn(K, seed=30 + r, scale=0.5, dtype=BF)      # a direction that some row likes most, twice
        w[lo] = boost
        w[hi] = boost
    room = max((N + 15) // 16, min((N + 3) // 4, 4096))
    best = torch.full((M + 3, room), -1, dtype=torch.int64, device=DEV)
    out = torch.empty(M, N, device=DEV)
    if form == "norm":
        ops.fused_linear(h, w, out, epilogue="store_f32", norm_weight=nw, eps=1e-5, row_best=best)
    else:
        xb = torch.empty(M, K, dtype=BF, device=DEV)
        stats = torch.zeros(64, 1, device=DEV)
        ops.stream_prepare(h, xb, stats)
        ops.fused_linear(xb, ops.fold_weight(w, nw), out, epilogue="store_f32", eps=1e-5, stats=stats, stat_blocks=1,
                         row_best=best)
    parts, part_cols = ops.last_best_parts, ops.last_best_cols
    assert 0 < parts <= room and parts * part_cols >= N > (parts - 1) * part_cols
    assert bool((best[M:] == -1).all()) and bool((best[:, parts:] == -1).all())
    top = best[:M, :parts].cpu().numpy().view("uint64").max(axis=1)
    index = (0xffffffff - (top & 0xffffffff)).astype("int64")
    logits = out.cpu()
    want = [int((logits[m] == logits[m].max()).nonzero()[0]) for m in range(M)]
    assert index.tolist() == want
    tokens = torch.full((M,), -1, dtype=torch.int32, device=DEV)
    last = torch.full((M + 1,), -1, dtype=torch.int32, device=DEV)
    f = torch.tensor([[0.0, 1.0, 1.0, 0.0]] * M, dtype=torch.float32, device=DEV).reshape(-1)
    i = torch.tensor([[1, -1, m + 1 if m % 2 else -1] for m in range(M)], dtype=torch.int32, device=DEV).reshape(-1)
    before = ops.paths().get("argmax_merged", 0)
    ops.sample(out, f, i, None, tokens, last_tokens=last, all_greedy=True, row_best=best, row_best_parts=parts,
               row_best_cols=part_cols)
    assert ops.paths()["argmax_merged"] == before + 1
    assert tokens.tolist() == want
    assert last.tolist() == [-1] + [want[m] if m % 2 else -1 for m in range(M)]
    # the other greedy kernels give the same tokens from the logits
    ops.sample(out, f, i, None, tokens, all_greedy=True)
    assert tokens.tolist() == want


@pytest.mark.parametrize("M,ff,K", [(1, 192, 64), (8, 4608, 1024), (19, 352, 128), (64, 200, 96)])
def test_swiglu_epilogue(ops, M, ff, K):
    h = randn(M, K, seed=11)
    nw = 1 + randn(K, seed=12, scale=0.1)
    w = randn(2 * ff, K, seed=13, scale=0.2, dtype=BF)
    x = plain.rmsnorm(h.cpu(), nw.cpu(), 1e-6).to(BF).double()
    g = (x @ w[:ff].double().cpu().T).to(BF).double()
    u = (x @ w[ff:].double().cpu().T).to(BF).double()
    out = torch.empty(M, ff, dtype=BF, device=DEV)
    ops.fused_linear(h, w, out, epilogue="swiglu", norm_weight=nw, eps=1e-6)
    close(out, plain.silu(g) * u, rel=2e-2)


@pytest.mark.parametrize("M,H,taps,bias", [(1, 64, 3, False), (8, 1024, 3, False), (5, 128, 4, True),
                                           (33, 96, 1, True), (64, 48, 5, False)])
def test_conv_epilogue_token_by_token_equals_the_whole_convolution(ops, M, H, taps, bias):
    """M requests advance one token per call, each in its own slot (in another order than
    the rows); their outputs over 6 calls equal the plain whole-sequence convolution."""
    steps = 6
    nw = 1 + randn(H, seed=14, scale=0.1)
    w_in = randn(3 * H, H, seed=15, scale=0.2, dtype=BF)
    b_in = randn(3 * H, seed=16, scale=0.1) if bias else None
    cw = randn(H, taps, seed=17)
    cb = randn(H, seed=18) if bias else None
    hs = randn(steps, M, H, seed=19)
    state = torch.zeros(M + 2, taps, H, device=DEV)
    slots = torch.tensor([(M + 1 - i) for i in range(M)], dtype=torch.int32, device=DEV)
    outs = []
    for t in range(steps):
        y = torch.empty(M, H, dtype=BF, device=DEV)
        ops.fused_linear(hs[t], w_in, y, epilogue="conv", norm_weight=nw, eps=1e-5, bias=b_in,
                         conv=(cw, cb, state, slots))
        outs.append(y.double().cpu())
    got = torch.stack(outs)              # [steps, M, H]
    for m in range(0, M, max(1, M // 4)):
        x = plain.rmsnorm(hs[:, m].cpu(), nw.cpu(), 1e-5).to(BF).double()
        bcx = x @ w_in.double().cpu().T + (b_in.double().cpu() if bias else 0)
        ref = plain.short_conv(bcx.to(BF), cw.cpu(), cb.cpu() if bias else None)
        close(got[:, m], ref, rel=2e-2)
    assert float(state[0].abs().max()) == 0.0          # a slot nobody uses stays zero


SLICED = [(1, 64, 64), (3, 130, 200), (4, 1024, 1024), (5, 77, 352), (8, 3072, 1024), (8, 96, 4608),
          (13, 50, 1160), (16, 272, 1024)]
# 9 to 64 rows: the kernel that streams the weights (inner sizes in steps of 32), at widths
# that give it one, two and four column tiles a workgroup, and few and many blocks of k
STREAMED = [(17, 64, 64), (20, 130, 352), (32, 1024, 1024), (33, 77, 96), (48, 3072, 1024),
            (64, 272, 4608), (64, 8192, 128), (33, 14400, 64), (50, 1000, 32)]


def scaled_case(M, N, K, streams, seed):
    """A stream h, its bfloat16 copy, uneven partial sums of squares, a norm weight, weights
    and the same weights with the norm weight folded in; rows picked in another order."""
    h = randn(M + 3, K, seed=seed)
    nw = 1 + randn(K, seed=seed + 1, scale=0.1)
    w = randn(streams * N, K, seed=seed + 2, scale=0.2, dtype=BF)
    folded = (w.float() * nw.reshape(1, -1)).to(BF)
    rows = torch.tensor([(3 * i + 1) % (M + 3) for i in range(M)], dtype=torch.int32, device=DEV)
    cuts = [0, K // 7, K // 3, K // 2, K - 8, K]
    stats = torch.zeros(80, 5, device=DEV)
    for j in range(5):
        stats[:M + 3, j] = (h[:, cuts[j]:cuts[j + 1]] ** 2).sum(dim=1)
    x = plain.rmsnorm(h.cpu(), nw.cpu(), 1e-5)[rows.long().cpu()].to(BF).double()
    return h, h.to(BF), stats, nw, w, folded, rows, x


@pytest.mark.parametrize("M,N,K", SLICED + STREAMED)
def test_sliced_products_behind_a_norm(ops, M, N, K):
    """The form for up to 16 rows, and for 9 to 64: bfloat16 copy of the stream, norm weight folded into the
    weights, 1/rms from the partial sums applied at the end; against the plain norm and
    product."""
    h, xb, stats, nw, w, folded, rows, x = scaled_case(M, N, K, 1, 40)
    b = randn(N, seed=44)
    ref = x @ w.double().cpu().T + b.double().cpu()
    out = torch.empty(M, N, dtype=BF, device=DEV)
    ops.fused_linear(xb, folded, out, eps=1e-5, stats=stats, stat_blocks=5, rows=rows, bias=b)
    close(out, ref)
    out32 = torch.empty(M, N, device=DEV)
    ops.fused_linear(xb, folded, out32, epilogue="store_f32", eps=1e-5, stats=stats, stat_blocks=5,
                     rows=rows, bias=b)
    close(out32, ref, rel=8e-3)
    # the older form (32-bit rows normalised on the fly) agrees
    old = torch.empty(M, N, device=DEV)
    ops.fused_linear(h, w, old, epilogue="store_f32", norm_weight=nw, eps=1e-5, rows=rows, bias=b,
                     stats=stats, stat_blocks=5)
    close(out32, old, rel=8e-3)


@pytest.mark.parametrize("M,ff,K", [(1, 192, 64), (8, 4608, 1024), (7, 352, 128), (16, 200, 96), (4, 100, 1160),
                                    (19, 352, 128), (40, 4608, 1024), (64, 200, 96), (33, 7200, 64),
                                    (5, 2300, 352), (6, 5000, 96), (8, 7000, 64)])
def test_sliced_swiglu(ops, M, ff, K):
    h, xb, stats, nw, w, folded, rows, x = scaled_case(M, ff, K, 2, 50)
    g = (x @ w[:ff].double().cpu().T).to(BF).double()
    u = (x @ w[ff:].double().cpu().T).to(BF).double()
    out = torch.empty(M, ff, dtype=BF, device=DEV)
    ops.fused_linear(xb, folded, out, epilogue="swiglu", eps=1e-5, stats=stats, stat_blocks=5, rows=rows)
    close(out, plain.silu(g) * u, rel=2.5e-2)


@pytest.mark.parametrize("M,H,taps,bias", [(1, 64, 3, False), (8, 1024, 3, False), (5, 128, 4, True),
                                           (16, 96, 1, True), (3, 48, 5, False), (12, 200, 8, True),
                                           (17, 64, 3, False), (40, 1024, 3, True), (62, 96, 4, True),
                                           (33, 160, 8, False)])
def test_sliced_conv_token_by_token_equals_the_whole_convolution(ops, M, H, taps, bias):
    """M requests advance one token per call, each in its own slot (in another order than
    the rows); their outputs over 6 calls equal the plain whole-sequence convolution."""
    steps = 6
    nw = 1 + randn(H, seed=14, scale=0.1)
    w_in = randn(3 * H, H, seed=15, scale=0.2, dtype=BF)
    folded = (w_in.float() * nw.reshape(1, -1)).to(BF)
    b_in = randn(3 * H, seed=16, scale=0.1) if bias else None
    cw = randn(H, taps, seed=17)
    cb = randn(H, seed=18) if bias else None
    hs = randn(steps, M, H, seed=19)
    state = torch.zeros(M + 2, taps, H, device=DEV)
    slots = torch.tensor([(M + 1 - i) for i in range(M)], dtype=torch.int32, device=DEV)
    stats = torch.zeros(64, 1, device=DEV)
    outs = []
    for t in range(steps):
        y = torch.empty(M, H, dtype=BF, device=DEV)
        xb = torch.empty(M, H, dtype=BF, device=DEV)
        ops.stream_prepare(hs[t], xb, stats)
        assert torch.equal(xb, hs[t].to(BF))
        torch.testing.assert_close(stats[:M, 0], (hs[t] ** 2).sum(dim=1), rtol=1e-5, atol=1e-5)
        ops.fused_linear(xb, folded, y, epilogue="conv", eps=1e-5, stats=stats, stat_blocks=1,
                         bias=b_in, conv=(cw, cb, state, slots))
        outs.append(y.double().cpu())
    got = torch.stack(outs)              # [steps, M, H]
    for m in range(0, M, max(1, M // 4)):
        x = plain.rmsnorm(hs[:, m].cpu(), nw.cpu(), 1e-5).to(BF).double()
        bcx = x @ w_in.double().cpu().T + (b_in.double().cpu() if bias else 0)
        ref = plain.short_conv(bcx.to(BF), cw.cpu(), cb.cpu() if bias else None)
        close(got[:, m], ref, rel=2.5e-2)
    assert float(state[0].abs().max()) == 0.0          # a slot nobody uses stays zero


@pytest.mark.parametrize("cols", [4, 7, 8, 9, 13, 16, 17, 24])
def test_sliced_swiglu_with_every_share_of_columns(ops, cols):
    """At 5 to 8 rows a workgroup of the SwiGLU product owns up to three tiles of 8 columns of each
    weight stream, as many as make the workgroups a whole number of rounds of the compute units; here
    the number of columns is forced, at widths that leave the last workgroup and its last tile partly
    empty."""
    lib = ops._lib("gemv_slices")
    lib.celeg_gemv_slices_force_cols(cols)
    try:
        test_sliced_swiglu(ops, 8, 1000, 128)
        test_sliced_swiglu(ops, 5, 333, 352)
    finally:
        lib.celeg_gemv_slices_force_cols(0)


@pytest.mark.parametrize("mt", [1, 2, 4])
@pytest.mark.parametrize("ct", [1, 2, 4])
def test_rows_kernel_with_every_share_of_rows_and_columns(ops, mt, ct):
    """The kernel for 9 to 64 rows chooses how many rows (16, 32 or 64) and columns (16, 32 or
    64 of every weight stream) a workgroup takes from the sizes; here every choice is forced in
    turn (a wider share of columns than an epilogue's streams allow falls back to the kernel's
    own), for every epilogue, at sizes that leave a part of a share empty."""
    lib = ops._lib("gemm_rows")
    lib.celeg_gemm_rows_force(ct, 0, mt)
    try:
        test_sliced_products_behind_a_norm(ops, 50, 1000, 352)
        test_sliced_products_behind_a_norm(ops, 64, 272, 4608)
        test_residual_epilogue_adds_in_place_and_leaves_partial_sums(ops, 64, 272, 1024)
        test_residual_epilogue_adds_in_place_and_leaves_partial_sums(ops, 33, 1000, 352)
        test_sliced_swiglu(ops, 40, 352, 128)
        test_sliced_conv_token_by_token_equals_the_whole_convolution(ops, 62, 96, 4, True)
    finally:
        lib.celeg_gemm_rows_force(0, 0, 0)


@pytest.mark.parametrize("M,N,K", [(1, 64, 64), (4, 1024, 1024), (5, 77, 352), (8, 96, 4608), (16, 272, 1024),
                                   (20, 77, 352), (33, 1024, 1024), (64, 272, 1024)])
def test_packed_weights_give_the_same_bits(ops, M, N, K):
    """The layout of blocks of 32 k-values changes where the weights lie, not what is added
    in which order: every epilogue gives identical results from either layout."""
    h, xb, stats, nw, w, folded, rows, x = scaled_case(M, N, K, 1, 70)
    b = randn(N, seed=74)
    packed = ops.pack_weight(folded)
    assert packed.shape == (K // 32, N, 32)
    outs = []
    for wt in (folded, packed):
        out32 = torch.empty(M, N, device=DEV)
        ops.fused_linear(xb, wt, out32, epilogue="store_f32", eps=1e-5, stats=stats, stat_blocks=5,
                         rows=rows, bias=b)
        hh = randn(M, N, seed=75)
        so = torch.zeros(64, ops.residual_stat_blocks(M, N, K), device=DEV)
        ops.fused_linear(xb[:M], wt, hh, epilogue="residual", stats_out=so)
        outs.append((out32, hh, so))
    for got, ref in zip(outs[1], outs[0]):
        assert torch.equal(got, ref)
    if N % 2 == 0:   # two streams from one packed tensor
        act = [torch.empty(M, N // 2, dtype=BF, device=DEV) for _ in range(2)]
        for o, wt in zip(act, (folded, packed)):
            ops.fused_linear(xb, wt, o, epilogue="swiglu", eps=1e-5, stats=stats, stat_blocks=5, rows=rows)
        assert torch.equal(act[0], act[1])


@pytest.mark.parametrize("M,N,K", [(17, 64, 64), (33, 80, 96), (40, 1024, 1024), (64, 272, 4608)])
def test_operands_with_rows_side_by_side_give_the_same_bits(ops, M, N, K):
    """For 9 to 64 rows the bfloat16 operands may lie as [width/8, 64, 8] (the rows side by
    side inside every group of 8 values): inputs and outputs in that layout give the same bits
    as rows that lie one after the other."""
    h, xb, stats, nw, w, folded, rows, x = scaled_case(M, N, K, 1, 90)
    xc = ops.chunked_rows(M + 3, K, DEV, max_rows=80)
    assert xc.shape == (M + 3, K // 8, 8) and xc.stride() == (8, 80 * 8, 1)
    st = torch.zeros(80, 1, device=DEV)
    ops.stream_prepare(h, xc, st)
    assert torch.equal(xc.reshape(M + 3, K), xb)
    torch.testing.assert_close(st[:M + 3, 0], (h ** 2).sum(dim=1), rtol=1e-5, atol=1e-5)
    b = randn(N, seed=94)
    flat, side = torch.empty(M, N, dtype=BF, device=DEV), ops.chunked_rows(M, N, DEV)
    for a_, out in ((xb, flat), (xc, side)):
        ops.fused_linear(a_, folded, out, eps=1e-5, stats=stats, stat_blocks=5, rows=rows, bias=b)
    assert torch.equal(side.reshape(M, N), flat)
    act = [torch.empty(M, N // 2, dtype=BF, device=DEV), ops.chunked_rows(M, N // 2, DEV)]
    for a_, out in zip((xb, xc), act):
        ops.fused_linear(a_, folded, out, epilogue="swiglu", eps=1e-5, stats=stats, stat_blocks=5, rows=rows)
    assert torch.equal(act[1].reshape(M, N // 2), act[0])
    hh = [randn(M, N, seed=95) for _ in range(2)]
    copies = [torch.zeros(M, N, dtype=BF, device=DEV), ops.chunked_rows(M, N, DEV)]
    so = [torch.zeros(64, ops.residual_stat_blocks(M, N, K), device=DEV) for _ in range(2)]
    for a_, h_, c_, s_ in zip((xb[:M], xc[:M]), hh, copies, so):
        ops.fused_linear(a_, folded, h_, epilogue="residual", stats_out=s_, out_bf16=c_)
    assert torch.equal(hh[0], hh[1]) and torch.equal(so[0], so[1])
    assert torch.equal(copies[1].reshape(M, N), copies[0]) and torch.equal(copies[0], hh[0].to(BF))
    # the kernels for up to 16 rows read rows that lie one after the other only
    from kernel_ops import KernelError
    with pytest.raises(KernelError, match="side by side"):
        ops.fused_linear(xc[:8], folded, torch.empty(8, N, dtype=BF, device=DEV))


def test_embed_stream_with_rows_side_by_side(ops):
    table = randn(300, 96, seed=96, dtype=BF)
    ids = torch.tensor([(7 * i) % 300 for i in range(40)], dtype=torch.int32, device=DEV)
    out = torch.empty(40, 96, device=DEV)
    xc = ops.chunked_rows(40, 96, DEV)
    st = torch.zeros(64, 2, device=DEV)
    ops.embed_stream(table, ids, out, xc, st)
    assert torch.equal(out, table[ids.long()].float()) and torch.equal(xc.reshape(40, 96), table[ids.long()])
    torch.testing.assert_close(st[:40, 0], (out ** 2).sum(dim=1), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("M", [6, 40])
def test_residual_refreshes_the_bfloat16_copy(ops, M):
    N, K = 200, 352
    a = randn(M, K, seed=60, dtype=BF)
    w = randn(N, K, seed=61, scale=0.1, dtype=BF)
    h = randn(M, N, seed=62)
    xb = torch.zeros(M + 2, N, dtype=BF, device=DEV)
    stats = torch.zeros(64, ops.residual_stat_blocks(M, N, K), device=DEV)
    ops.fused_linear(a, w, h, epilogue="residual", stats_out=stats, out_bf16=xb)
    assert torch.equal(xb[:M], h.to(BF)) and float(xb[M:].abs().max()) == 0.0


def test_embed_stream(ops):
    table = randn(331, 96, seed=20, dtype=BF)
    ids = torch.tensor([5, 330, 0, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(4, 96, device=DEV)
    xb = torch.empty(4, 96, dtype=BF, device=DEV)
    stats = torch.zeros(64, 6, device=DEV)
    ops.embed_stream(table, ids, out, xb, stats)
    assert torch.equal(out, table[ids.long()].float()) and torch.equal(xb, table[ids.long()])
    torch.testing.assert_close(stats[:4, 0], (out ** 2).sum(dim=1), rtol=1e-6, atol=1e-6)


def test_embed_stats(ops):
    table = randn(331, 96, seed=20, dtype=BF)
    ids = torch.tensor([5, 330, 0, 17], dtype=torch.int32, device=DEV)
    out = torch.empty(4, 96, device=DEV)
    stats = torch.zeros(64, 6, device=DEV)
    ops.embed_stats(table, ids, out, stats)
    assert torch.equal(out, table[ids.long()].float())
    torch.testing.assert_close(stats[:4, 0], (out ** 2).sum(dim=1), rtol=1e-6, atol=1e-6)


def test_unsupported_sizes_are_refused(ops):
    from kernel_ops import KernelError
    w = randn(32, 100, dtype=BF)
    with pytest.raises(KernelError, match="not supported"):
        ops.fused_linear(randn(4, 100, dtype=BF), w, torch.empty(4, 32, dtype=BF, device=DEV))
    w = randn(32, 64, dtype=BF)
    with pytest.raises(KernelError, match="not supported"):
        ops.fused_linear(randn(65, 64, dtype=BF), w, torch.empty(65, 32, dtype=BF, device=DEV))
    assert not ops.fused_linear_ok(8, 100) and ops.fused_linear_ok(64, 96)


@pytest.mark.parametrize("K", [1024, 2048])
@pytest.mark.parametrize("R", [1, 8, 17, 64])
def test_output_head_at_the_real_vocabulary(tmp_path, R, K):
    """Final norm and output product the way the model's head runs them for few wanted rows, at
    65,536 columns: wider than the k-sliced kernels take, so up to 8 rows go to the kernel that
    keeps its rows in LDS and 9 to 64 rows to the one that streams the weights.  Rows picked out
    of a longer step, through a model of one convolution layer of that width."""
    from celeg_amd.engine import StepEntry, load_model
    from celeg_amd.weights import write_random_model
    from helpers import assert_close_bf16, random_tokens
    V = 65536
    cfg = {"architectures": ["Lfm2ForCausalLM"], "vocab_size": V, "hidden_size": K, "num_hidden_layers": 1,
           "layer_types": ["conv"], "num_attention_heads": K // 64, "num_key_value_heads": 8, "head_dim": 64,
           "intermediate_size": 256, "block_auto_adjust_ff_dim": False, "rope_theta": 1e6, "conv_L_cache": 3,
           "conv_bias": False, "tie_word_embeddings": K == 1024, "norm_eps": 1e-5, "max_position_embeddings": 128}
    folder = write_random_model(cfg, str(tmp_path / "head"), seed=R, dtype=BF, std=0.05)
    pcfg, W = plain.load_model_folder(folder)
    T = R + 5 if R < 64 else 64
    tokens = random_tokens(V, T, seed=60 + R)
    picked = sorted({(3 * i + 1) % T for i in range(R)}) if R < 64 else list(range(64))
    lm = load_model(folder, dtype="bfloat16", page_tokens=16, n_pages=8, max_requests=1, max_batched_tokens=64)
    slot = lm.cache.open()
    assert lm.cache.prepare(slot, 0, T)
    got = lm.runner.step([StepEntry(slot, 0, tokens, picked)])
    assert got.shape == (len(picked), V)
    ref = plain.model_logits(pcfg, W, tokens)[picked]
    assert_close_bf16(got, ref, f"head R={R} K={K}")
    # the last columns and rows are there
    assert_close_bf16(got[-1:, -64:], ref[-1:, -64:], "head, last columns")
    lm.close()


@pytest.mark.parametrize("M,N,K,epilogue", [(1, 4100, 64, "store_f32"), (8, 70000, 2048, "store_f32"), (16, 333, 96, "store"),
                                            (5, 24, 160, "store_f32"), (8, 200, 128, "swiglu"), (33, 1000, 96, "store_f32")])
def test_the_staged_kernel_reads_weights_in_blocks_of_32_as_it_reads_rows(ops, M, N, K, epilogue):
    """The kernel that normalises the rows itself takes its weights with the rows one after the other
    or as [K/32, rows, 32] (what a wide model's output head is copied to): the same products in
    the same order, so the same bits."""
    streams = 2 if epilogue == "swiglu" else 1
    h = randn(M, K, seed=41)
    nw = 1 + randn(K, seed=42, scale=0.1)
    w = randn(streams * N, K, seed=43, scale=0.1, dtype=BF)
    dtype = torch.float32 if epilogue == "store_f32" else BF
    a = torch.empty(M, N, dtype=dtype, device=DEV)
    b = torch.empty(M, N, dtype=dtype, device=DEV)
    ops.fused_linear(h, w, a, epilogue=epilogue, norm_weight=nw, eps=1e-5)
    ops.fused_linear(h, ops.pack_weight(w), b, epilogue=epilogue, norm_weight=nw, eps=1e-5)
    assert torch.equal(a, b)
    x = h * torch.rsqrt((h * h).mean(dim=1, keepdim=True) + 1e-5) * nw
    y = x.to(BF).float() @ w.float().T
    want = torch.nn.functional.silu(y[:, :N]) * y[:, N:] if streams == 2 else y
    assert torch.allclose(a.float(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))

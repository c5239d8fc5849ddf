"""The fused bfloat16 products for many rows (gemm_tiles.hip) alone, against torch: every
epilogue, every tile shape, at sizes that are no multiple of the tiles."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF = torch.bfloat16
N_SHAPES = 19


@pytest.fixture(scope="module")
def ops():
    from kernel_ops import HipOps
    ops = HipOps(DEV)
    yield ops
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(-1)


def randn(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def product(a, w, scale=None, bias=None):
    y = a.double() @ w.double().T
    if scale is not None:
        y = y * scale.double()[:, None]
    if bias is not None:
        y = y + bias.double()
    return y


def bf16_round(x):
    return x.to(torch.float32).to(BF).double()


SIZES = [(300, 200, 128), (65, 36, 64), (512, 256, 192), (129, 1024, 1024), (520, 648, 192)]


@pytest.mark.parametrize("shape", list(range(N_SHAPES)) + [-1])
@pytest.mark.parametrize("M,N,K", SIZES)
def test_store_with_row_scale_and_bias(ops, shape, M, N, K):
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(shape)
    a = randn(M, K, seed=1, dtype=BF)
    w = randn(N, K, seed=2, scale=0.05, dtype=BF)
    bias = randn(N, seed=3) if shape % 2 else None
    eps, blocks = 1e-5, 11                       # more partial sums than one round of loads
    g = torch.Generator().manual_seed(4)
    stats = (torch.rand(M, blocks + 2, generator=g) * K / blocks).to(DEV)
    scale = 1.0 / torch.sqrt(stats[:, :blocks].sum(1) / K + eps)
    out = torch.zeros(M + 1, N, dtype=BF, device=DEV)
    ops.tiled_linear(a, w, out[:M], bias=bias, stats=stats, stat_blocks=blocks, eps=eps)
    ref = product(a, w, scale, bias)
    assert float((out[:M].double() - ref).abs().max()) <= 2 ** -7 * float(ref.abs().max())
    assert float(out[M].abs().max()) == 0        # nothing behind the last row is written
    # without statistics the sums are stored as they are
    ops.tiled_linear(a, w, out[:M], bias=bias)
    ref = product(a, w, None, bias)
    assert float((out[:M].double() - ref).abs().max()) <= 2 ** -7 * float(ref.abs().max())


@pytest.mark.parametrize("shape", list(range(N_SHAPES)) + [-1])
@pytest.mark.parametrize("M,ff,K", SIZES)
def test_swiglu(ops, shape, M, ff, K):
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(shape)
    a = randn(M, K, seed=5, dtype=BF)
    w = randn(2 * ff, K, seed=6, scale=0.1, dtype=BF)
    bias = randn(2 * ff, seed=7, scale=0.1) if shape % 2 else None
    y = product(a, w, None, bias)
    gate, up = bf16_round(y[:, :ff]), bf16_round(y[:, ff:])
    ref = gate / (1 + torch.exp(-gate)) * up
    out = torch.zeros(M, ff, dtype=BF, device=DEV)
    ops.tiled_linear(a, w, out, epilogue="swiglu", bias=bias)
    # a flip of the rounding of gate or up moves the result by one bfloat16 step of it
    bound = 2 ** -6 * float(ref.abs().max()) + 2 ** -7 * float((up.abs() * (1 + gate.abs())).max())
    assert float((out.double() - ref).abs().max()) <= bound


@pytest.mark.parametrize("shape", list(range(N_SHAPES)) + [-1])
@pytest.mark.parametrize("M,N,K", SIZES)
def test_residual_adds_in_place_refreshes_the_copy_and_leaves_partial_sums(ops, shape, M, N, K):
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(shape)
    a = randn(M, K, seed=8, dtype=BF)
    w = randn(N, K, seed=9, scale=0.05, dtype=BF)
    bias = randn(N, seed=10) if shape % 2 else None
    h0 = randn(M + 1, N, seed=11)
    h = h0.clone()
    blocks = ops.tiled_stat_blocks(M, N, K)
    copy = torch.zeros(M, N, dtype=BF, device=DEV)
    sums = torch.zeros(M, blocks + 1, device=DEV)
    ops.tiled_linear(a, w, h[:M], epilogue="residual", bias=bias, out_bf16=copy, stats_out=sums)
    assert ops.last_stat_blocks == blocks
    y = product(a, w, None, bias)
    ref = h0[:M].double() + bf16_round(y)
    # the product enters the sum rounded to bfloat16: a flip of that rounding is one step of it
    assert float((h[:M].double() - ref).abs().max()) <= 2 ** -7 * float(y.abs().max())
    assert torch.equal(h[M], h0[M])
    assert torch.equal(copy, h[:M].to(BF))
    squares = (h[:M].double() ** 2).sum(1)
    assert float(((sums[:, :blocks].double().sum(1) - squares).abs() / squares).max()) < 1e-5
    assert float(sums[:, blocks].abs().max()) == 0


@pytest.mark.parametrize("M,N,K,blocks", [(2000, 1024, 2304, 16), (2000, 1024, 1024, 8), (2048, 2048, 1024, 16),
                                          (2048, 3072, 1024, 16), (1024, 3072, 1024, 24)])
def test_the_shapes_chosen_for_a_prefill(ops, M, N, K, blocks):
    """What the choice of shape gives at the sizes of a prefill of some 2,000 rows (few weight
    rows with a long and a short K, q/k/v, in_proj), against torch, with the residual epilogue;
    the number of tile columns says which shape it was."""
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(-1)
    assert ops.tiled_stat_blocks(M, N, K) == blocks
    a = randn(M, K, seed=20, dtype=BF)
    w = randn(N, K, seed=21, scale=0.03, dtype=BF)
    h0 = randn(M, N, seed=22)
    h = h0.clone()
    copy = torch.zeros(M, N, dtype=BF, device=DEV)
    sums = torch.zeros(M, blocks, device=DEV)
    ops.tiled_linear(a, w, h, epilogue="residual", out_bf16=copy, stats_out=sums)
    y = product(a, w)
    ref = h0.double() + bf16_round(y)
    assert float((h.double() - ref).abs().max()) <= 2 ** -7 * float(y.abs().max())
    assert torch.equal(copy, h.to(BF))
    squares = (h.double() ** 2).sum(1)
    assert float(((sums.double().sum(1) - squares).abs() / squares).max()) < 1e-5


def test_a_row_does_not_depend_on_the_other_rows(ops):
    """The same row in a step of 70 rows and in one of 700 gives the same bits where the tile
    shape is the same (the sums of a row are formed in an order that K alone fixes)."""
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(7)
    K, N = 192, 128
    a = randn(700, K, seed=12, dtype=BF)
    w = randn(N, K, seed=13, scale=0.05, dtype=BF)
    big = torch.empty(700, N, dtype=BF, device=DEV)
    small = torch.empty(70, N, dtype=BF, device=DEV)
    ops.tiled_linear(a, w, big)
    ops.tiled_linear(a[330:400], w, small)
    assert torch.equal(big[330:400], small)


def test_unsupported_sizes_are_refused(ops):
    from kernel_ops import KernelError
    ops._lib("gemm_tiles").celeg_gemm_tiles_force(-1)
    a = randn(80, 96, dtype=BF)
    with pytest.raises(KernelError):             # inner size no multiple of 64
        ops.tiled_linear(a, randn(64, 96, dtype=BF), torch.empty(80, 64, dtype=BF, device=DEV))
    a = randn(80, 128, dtype=BF)
    with pytest.raises(KernelError):             # columns no multiple of 4
        ops.tiled_linear(a, randn(66, 128, dtype=BF), torch.empty(80, 66, dtype=BF, device=DEV))
    with pytest.raises(KernelError):             # a 32-bit output goes with the residual epilogue only
        ops.tiled_linear(a, randn(64, 128, dtype=BF), torch.empty(80, 64, device=DEV))
    with pytest.raises(KernelError):
        ops.tiled_linear(a, randn(64, 128, dtype=BF), torch.empty(80, 64, dtype=BF, device=DEV),
                         stats_out=torch.empty(80, 4, device=DEV))
    assert not ops.tiled_linear_ok(80, 64, 96)
    assert ops.tiled_linear_ok(80, 64, 128, 4608)


# ---------------------------------------------------------------- the q/k/v product with its tail
@pytest.mark.parametrize("heads,kv_heads,K,rotate,normed", [(16, 8, 1024, True, True), (6, 2, 192, True, False),
                                                            (4, 4, 128, False, True), (3, 1, 64, True, True)])
def test_qkv_product_with_norm_rotation_and_cache_write(ops, heads, kv_heads, K, rotate, normed):
    """The product of the q, k and v projections that normalises and turns the query and key
    heads and writes keys and values into the pages inside its own kernel, against the product
    followed by qk_norm_rope_store: a step of three requests (portions that start at positions
    0, 5 and 130, so that groups of four rows start on a multiple of four, in the middle of one,
    and straddle the border between two requests; one request brings a single row).  Values must
    come out bit for bit; queries and keys may differ by a rounding (the sums of squares are
    added in another order)."""
    import plain_lfm2 as plain
    from celeg_amd.engine import StepEntry
    from kernel_harness import build_batch, make_cache
    hd, n_layers, layer, page_tokens = 64, 2, 1, 16
    starts, lengths = [0, 5, 130, 77], [203, 131, 1, 66]
    total = sum(lengths)
    N = (heads + 2 * kv_heads) * hd
    a = randn(total, K, seed=30, dtype=BF)
    w = randn(N, K, seed=31, scale=0.05, dtype=BF)
    bias = randn(N, seed=32) if not normed else None
    qw = (1 + randn(hd, seed=33, scale=0.2)) if normed else None
    kw = (1 + randn(hd, seed=34, scale=0.2)) if normed else None
    inv_freq = torch.tensor(plain.rope_inverse_frequencies(10000.0, hd), dtype=torch.float64).float().to(DEV) if rotate else None
    eps, blocks = 1e-5, 5
    g = torch.Generator().manual_seed(35)
    stats = (torch.rand(total, blocks, generator=g) * K / blocks).to(DEV)
    results = []
    for fused in (False, True):
        cache = make_cache(kv_heads, hd, n_layers, BF, page_tokens=page_tokens, n_pages=64, max_context=512, slots=4)
        kv = cache.layer_cache(layer).kv
        slots = [cache.open() for _ in lengths]
        entries = []
        for slot, start, n in zip(slots, starts, lengths):
            assert cache.prepare(slot, 0, start + n)
            entries.append(StepEntry(slot, start, [0] * n))
        batch, keep = build_batch(ops, cache, entries)
        qkv = torch.zeros(total + 1, N, dtype=BF, device=DEV)
        if fused:
            ops.tiled_linear(a, w, qkv[:total], stats=stats, stat_blocks=blocks, eps=eps, bias=bias,
                             qkv=dict(heads=heads, kv_heads=kv_heads, q_weight=qw, k_weight=kw, eps=1e-6, inv_freq=inv_freq,
                                      batch=batch, kv=kv))
        else:
            ops.tiled_linear(a, w, qkv[:total], stats=stats, stat_blocks=blocks, eps=eps, bias=bias)
            q, k, v = qkv[:total, :heads * hd], qkv[:total, heads * hd:(heads + kv_heads) * hd], qkv[:total, (heads + kv_heads) * hd:]
            ops.qk_norm_rope_store(q, k, v, qw, kw, 1e-6, inv_freq, hd, heads, kv_heads, hd, batch, kv)
        torch.cuda.synchronize()
        assert float(qkv[total].abs().max()) == 0
        table = kv.table.cpu()
        pages = [int(table[slot, p]) for slot, start, n in zip(slots, starts, lengths)
                 for p in range((start + n + page_tokens - 1) // page_tokens)]
        others = sorted(set(range(kv.k.shape[0])) - set(pages))
        assert float(kv.k[others].float().abs().max()) == 0 and float(kv.v[others].float().abs().max()) == 0
        assert float(kv.k[:, 0].float().abs().max()) == 0          # the other layer's pages
        results.append((qkv[:total, :heads * hd].float().clone(), kv.k[pages].float().clone(), kv.v[pages].clone()))
    (qa, ka, va), (qb, kb, vb) = results
    assert torch.equal(va, vb) and float(va.float().abs().max()) > 0
    for x, y in ((qa, qb), (ka, kb)):
        assert float(x.abs().max()) > 0
        # a rounding of bfloat16 where the two differ at all
        assert float(((x - y).abs() / (x.abs() + y.abs() + 1e-3)).max()) <= 2 ** -7
        assert float((x != y).float().mean()) < 0.02

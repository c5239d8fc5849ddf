"""The entry point that allocates nothing (``celeg_attention_decode_bf16_no_alloc``), called
through ``ctypes`` as a caller without an allocator would, against the existing entry point
(``celeg_attention_decode_bf16`` with a workspace the caller allocated): two calls in a row on
the same GPU, the second with a smaller input, then a call beyond the scratch array's size."""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(lib, rows, heads, kv_heads, head_dim, context, page_tokens, seed):
    """Both entry points on the same paged keys and values; returns (existing, new)."""
    g = torch.Generator().manual_seed(seed)
    pages_per_row = (context + page_tokens - 1) // page_tokens
    n_pages = rows * pages_per_row
    n_layers, layer = 2, 1
    k_pool = (torch.randn(n_pages, n_layers, kv_heads, page_tokens, head_dim, generator=g)).bfloat16().to(DEV)
    v_pool = (torch.randn(n_pages, n_layers, kv_heads, head_dim, page_tokens, generator=g)).bfloat16().to(DEV)
    q = torch.randn(rows, heads * head_dim, generator=g).bfloat16().to(DEV)
    # every request's pages in a shuffled order, and contexts of different lengths
    table = torch.randperm(n_pages, generator=g).to(torch.int32).reshape(rows, pages_per_row).to(DEV)
    slots = torch.arange(rows, dtype=torch.int32, device=DEV)
    positions = torch.tensor([context - 1 - (7 * i) % (context // 2) for i in range(rows)],
                             dtype=torch.int32, device=DEV)
    split_rounds = 1 if context <= 4096 else 4
    n_parts = (context + 64 * split_rounds - 1) // (64 * split_rounds)
    parts = rows * heads * n_parts
    ws = torch.empty(parts * (head_dim + 2), device=DEV)
    out_a = torch.zeros(rows, heads * head_dim, dtype=torch.bfloat16, device=DEV)
    out_b = torch.zeros_like(out_a)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    scale = ctypes.c_float(1 / math.sqrt(head_dim))
    code = lib.celeg_attention_decode_bf16(
        ptr(q), heads * head_dim, ptr(k_pool), ptr(v_pool), ptr(table), pages_per_row, ptr(slots),
        ptr(positions), ptr(ws), ctypes.c_void_p(ws.data_ptr() + 4 * parts * head_dim), n_parts, ptr(out_a),
        heads * head_dim, rows, heads, kv_heads, head_dim, page_tokens, n_layers, layer, scale, 0, 0,
        split_rounds, n_parts, stream)
    assert code == 0
    code = lib.celeg_attention_decode_bf16_no_alloc(
        ptr(q), heads * head_dim, ptr(k_pool), ptr(v_pool), ptr(table), pages_per_row, ptr(slots),
        ptr(positions), ptr(out_b), heads * head_dim, rows, heads, kv_heads, head_dim, page_tokens,
        n_layers, layer, scale, 0, split_rounds, n_parts, stream)
    assert code == 0
    torch.cuda.synchronize()
    # and a plain reference of one row, so that "equal" is not "equally wrong"
    r = rows - 1
    n = int(positions[r]) + 1
    group = heads // kv_heads
    pages = table[r].long().cpu()
    kk = k_pool[:, layer].float().cpu()[pages].permute(1, 0, 2, 3).reshape(kv_heads, -1, head_dim)[:, :n]
    vv = v_pool[:, layer].float().cpu()[pages].permute(1, 2, 0, 3).reshape(kv_heads, head_dim, -1)[:, :, :n]
    qq = q[r].float().cpu().reshape(heads, head_dim)
    ref = torch.stack([torch.softmax(kk[h // group] @ qq[h] / math.sqrt(head_dim), 0) @ vv[h // group].T
                       for h in range(heads)]).reshape(-1)
    torch.testing.assert_close(out_b[r].float().cpu(), ref, rtol=2e-2, atol=2e-2)
    return out_a, out_b


def test_no_alloc_entry_point_equals_the_one_with_a_workspace():
    from celeg_amd.csrc import build
    lib = ctypes.CDLL(build.ensure_built("attention_fast"))
    torch.cuda.set_device(0)
    torch.zeros(1, device=DEV)                       # the context exists before the first call
    assert lib.celeg_attention_decode_no_alloc_init() == 0
    a, b = _case(lib, rows=8, heads=16, kv_heads=8, head_dim=64, context=2100, page_tokens=16, seed=1)
    assert torch.equal(a, b) and float(b.float().abs().max()) > 0
    # a smaller input right after: the array still holds the first call's parts
    a, b = _case(lib, rows=3, heads=4, kv_heads=1, head_dim=128, context=300, page_tokens=32, seed=2)
    assert torch.equal(a, b) and float(b.float().abs().max()) > 0
    a, b = _case(lib, rows=2, heads=8, kv_heads=2, head_dim=64, context=9000, page_tokens=16, seed=3)
    assert torch.equal(a, b)
    # beyond the array: refused, nothing launched
    null = ctypes.c_void_p(0)
    code = lib.celeg_attention_decode_bf16_no_alloc(
        null, 64, null, null, null, 1, null, null, null, 64, 4096, 64, 8, 64, 16, 1, 0,
        ctypes.c_float(1.0), 0, 1, 64, null)
    assert code == 1                                  # hipErrorInvalidValue
    code = lib.celeg_attention_decode_bf16_no_alloc(
        null, 64, null, null, null, 1, null, null, null, 64, 1, 4, 2, 80, 16, 1, 0,
        ctypes.c_float(1.0), 0, 1, 4, null)
    assert code == 1                                  # a head size the kernels are not built for

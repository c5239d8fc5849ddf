"""The library's plain C++ functions (``celeg_amd/csrc/host/reference.cpp``: what each kernel computes,
as loops over host memory) as Python calls on numpy arrays, through ``celeg_reference_call``.  They need
no GPU."""
from __future__ import annotations

import ctypes
import json

import numpy as np

from celeg_amd import native


class ReferenceError_(RuntimeError):
    pass


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def call(op: str, keep=(), **args):
    lib = native.lib()
    lib.celeg_reference_call.restype = ctypes.c_char_p
    lib.celeg_reference_call.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    packed = {k: (int(v.ctypes.data) if isinstance(v, np.ndarray) else v) for k, v in args.items()}
    answer = lib.celeg_reference_call(op.encode(), json.dumps(packed).encode())
    if answer is None:
        raise ReferenceError_(native.last_error())
    return json.loads(answer.decode())


def embed(table, ids):
    table, ids = _f32(table), _i32(ids)
    out = np.empty((len(ids), table.shape[1]), dtype=np.float32)
    call("embed", table=table, vocab=table.shape[0], width=table.shape[1], ids=ids, rows=len(ids), out=out)
    return out


def rmsnorm(x, weight, eps, delta=None):
    """Returns (normalised rows, x + delta)."""
    x, weight = _f32(x).copy(), _f32(weight)
    delta = _f32(delta) if delta is not None else None
    out = np.empty_like(x)
    call("rmsnorm", x=x, delta=delta, weight=weight, eps=float(eps), rows=x.shape[0], width=x.shape[1], out=out)
    return out, x


def linear(x, w, bias=None):
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    out = np.empty((x.shape[0], w.shape[0]), dtype=np.float32)
    call("linear", x=x, w=w, bias=bias, M=x.shape[0], N=w.shape[0], K=x.shape[1], out=out)
    return out


def swiglu(gate_up):
    gate_up = _f32(gate_up)
    out = np.empty((gate_up.shape[0], gate_up.shape[1] // 2), dtype=np.float32)
    call("swiglu", gate_up=gate_up, rows=gate_up.shape[0], ff=gate_up.shape[1] // 2, out=out)
    return out


def short_conv(bcx, w, bias, state, seq_slot, seq_start, cu_seqlens):
    """``state`` [slots, taps, width] float32 (contiguous) is updated in place."""
    assert state.dtype == np.float32 and state.flags["C_CONTIGUOUS"]
    bcx, w = _f32(bcx), _f32(w)
    bias = _f32(bias) if bias is not None else None
    seq_slot, seq_start, cu_seqlens = _i32(seq_slot), _i32(seq_start), _i32(cu_seqlens)
    width = bcx.shape[1] // 3
    out = np.empty((bcx.shape[0], width), dtype=np.float32)
    call("short_conv", bcx=bcx, w=w, bias=bias, state=state, seq_slot=seq_slot, seq_start=seq_start, cu_seqlens=cu_seqlens,
         n_seqs=len(seq_slot), width=width, taps=w.shape[1], out=out)
    return out


def qk_norm_rope(x, weight, eps, inv_freq, rotary_dim, pairing, positions):
    """x [rows, heads, head_dim]; returns the normalised and rotated copy."""
    x = _f32(x).copy()
    weight = _f32(weight) if weight is not None else None
    inv_freq = _f32(inv_freq) if inv_freq is not None else None
    positions = _i32(positions)
    call("qk_norm_rope", x=x, weight=weight, eps=float(eps), inv_freq=inv_freq, rotary_dim=int(rotary_dim), pairing=int(pairing),
         positions=positions, rows=x.shape[0], heads=x.shape[1], head_dim=x.shape[2])
    return x


class PagedCache:
    """Keys [pages, layers, kv_heads, page_tokens, head_dim] and values [pages, layers, kv_heads, head_dim,
    page_tokens] on the host, with a block table [slots, pages per request]."""

    def __init__(self, n_pages, n_layers, kv_heads, head_dim, page_tokens, slots, pages_per_request):
        self.k = np.zeros((n_pages, n_layers, kv_heads, page_tokens, head_dim), dtype=np.float32)
        self.v = np.zeros((n_pages, n_layers, kv_heads, head_dim, page_tokens), dtype=np.float32)
        self.table = np.full((slots, pages_per_request), -1, dtype=np.int32)
        self.n_layers, self.kv_heads, self.head_dim, self.page_tokens = n_layers, kv_heads, head_dim, page_tokens

    def store(self, k, v, token_slot, positions, layer):
        k, v, token_slot, positions = _f32(k), _f32(v), _i32(token_slot), _i32(positions)
        call("kv_store", k=k, v=v, k_pool=self.k, v_pool=self.v, table=self.table, table_stride=self.table.shape[1],
             token_slot=token_slot, positions=positions, rows=len(positions), kv_heads=self.kv_heads, head_dim=self.head_dim,
             page_tokens=self.page_tokens, n_layers=self.n_layers, layer=layer)

    def attend(self, q, token_slot, positions, layer, heads, scale, window=0):
        q, token_slot, positions = _f32(q), _i32(token_slot), _i32(positions)
        out = np.empty((len(positions), heads * self.head_dim), dtype=np.float32)
        call("paged_attention", q=q, k_pool=self.k, v_pool=self.v, table=self.table, table_stride=self.table.shape[1],
             token_slot=token_slot, positions=positions, rows=len(positions), heads=heads, kv_heads=self.kv_heads,
             head_dim=self.head_dim, page_tokens=self.page_tokens, n_layers=self.n_layers, layer=layer, scale=float(scale),
             window=int(window or 0), out=out)
        return out


def sample(logits, temperature, top_k, top_p, penalty, seen, u):
    logits = _f32(logits)
    seen = np.ascontiguousarray(seen, dtype=np.uint8) if seen is not None else None
    return call("sample", logits=logits, vocab=len(logits), temperature=float(temperature), top_k=int(top_k), top_p=float(top_p),
                penalty=float(penalty), seen=seen, u=float(u))["token"]

"""The kernels as Python calls on torch tensors, for the tests of single kernels.

Every call goes to the library's own dispatcher (``Ops`` in ``celeg_amd/csrc/host/ops.cpp``, the
one the parts call) through ``celeg_ops_call``: the shape checks, the choice of kernel, the
workspaces and the tables of cosines and sines are the library's, and a size it refuses comes
back as a ``KernelError`` with the library's reason.  What is here only turns torch tensors
into addresses, sizes and strides, with torch's current HIP stream (so a stream that records a
graph records the kernels too).  There is no fallback: if the library cannot be built or loaded,
or a tensor is not on the GPU, the call fails loudly.
"""
from __future__ import annotations

import ctypes
import json
from typing import Dict, Optional

import torch

from celeg_amd.csrc import build

_NAMES = {torch.float32: "float32", torch.bfloat16: "bfloat16", torch.int32: "int32", torch.uint8: "uint8"}


class KernelError(RuntimeError):
    pass


def _raw_stream(device_index: int) -> int:
    """The raw handle of torch's current stream on a device."""
    return torch._C._cuda_getCurrentRawStream(device_index)


def _tensor(t: Optional[torch.Tensor], name: str = "tensor"):
    """A tensor as the library reads it: address, dtype, sizes and strides in elements."""
    if t is None:
        return None
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
        raise KernelError(f"{name} must be a GPU tensor")
    if t.dtype not in _NAMES:
        raise KernelError(f"{name}: dtype {t.dtype} is not supported (float32, bfloat16, int32, uint8)")
    if t.dim() > 4:
        raise KernelError(f"{name}: up to four dimensions")
    return {"data": t.data_ptr(), "dtype": _NAMES[t.dtype], "shape": list(t.shape), "stride": list(t.stride())}


def _address(t: Optional[torch.Tensor], name: str, dtype=torch.int32):
    if t is None:
        return None
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda" or t.dtype != dtype or not t.is_contiguous():
        raise KernelError(f"{name} must be a contiguous {dtype} tensor on the GPU")
    return t.data_ptr()


def _batch(b) -> dict:
    """A step's arrays (``kernel_harness.build_batch``) as addresses and counts."""
    out = {name: int(getattr(b, name, 0) or 0) for name in ("n_tokens", "n_seqs", "n_logit_rows", "single_rows",
                                                            "max_context_len", "context_bound")}
    out["decode_only"] = bool(getattr(b, "decode_only", False))
    for name in ("token_ids", "positions", "token_seq", "token_slot", "cu_seqlens", "seq_slot", "seq_start", "logit_rows"):
        t = getattr(b, name, None)
        out[name] = _address(t, name) if t is not None and t.numel() else None
    return out


def _kv(kv) -> dict:
    """One layer's view of a cache group (``kernel_harness.HarnessCache.layer_cache(...).kv``)."""
    for t, name in ((kv.k, "k cache"), (kv.v, "v cache"), (kv.table, "block table")):
        if not t.is_cuda or not t.is_contiguous():
            raise KernelError(f"{name} must be a contiguous GPU tensor")
    if kv.k.dtype != kv.v.dtype or kv.k.dtype not in (torch.float32, torch.bfloat16) or kv.table.dtype != torch.int32:
        raise KernelError("the cache must be float32 or bfloat16 with an int32 block table")
    if tuple(kv.k.shape[1:]) != (kv.n_layers, kv.kv_heads, kv.page_tokens, kv.head_dim) or \
            tuple(kv.v.shape[1:]) != (kv.n_layers, kv.kv_heads, kv.head_dim, kv.page_tokens):
        raise KernelError("attention: unexpected cache shape")
    return {"k": kv.k.data_ptr(), "v": kv.v.data_ptr(), "dtype": _NAMES[kv.k.dtype], "layer": kv.layer,
            "n_layers": kv.n_layers, "table": kv.table.data_ptr(), "table_stride": kv.table.stride(0),
            "table_rows": kv.table.shape[0], "page_tokens": kv.page_tokens, "kv_heads": kv.kv_heads,
            "head_dim": kv.head_dim, "n_pages": kv.k.shape[0] - 1, "group": getattr(kv, "group", 0)}


class HipOps:
    # what the attributes below are called in the library
    _KNOBS = ("attention_decode_whole", "use_blaslt", "attention_rows_per_tile", "attention_rows_form",
              "use_rope_table", "use_argmax_parts", "use_sliced", "use_rows_kernel", "use_tiles", "use_qkv_tail",
              "use_fresh_decode", "rows_kernel_min_rows", "tiles_min_rows", "fused_linear_shape")

    def __init__(self, device="cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError("celeg_amd needs a GPU: torch.cuda.is_available() is False and "
                              "there is no CPU path")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"celeg_amd runs on a GPU only, not on '{device}'")
        self._device_index = self.device.index if self.device.index is not None else torch.cuda.current_device()
        self._library: Optional[ctypes.CDLL] = None
        self.loaded_libraries: Dict[str, str] = {}
        # the dispatcher's knobs, with the library's own defaults; every call carries them
        self.attention_decode_whole = -1     # -1: chosen from the batch; 0 split-key kernels; 1 one workgroup per request and key/value head
        self.use_blaslt = True               # products of many rows: hipBLASLt called directly
        self.attention_rows_per_tile = 0     # 0: the kernel chooses; 64 or 128 to force
        self.attention_rows_form = 0         # 0: the kernel chooses; 1 to 4 to force (see attention_fast.hip)
        self.decode_part_thresholds = (64, 256)
        self.attention_impl = "auto"         # "general": always the general attention kernel
        self.use_rope_table = True
        self.use_argmax_parts = True
        self.use_sliced = True
        self.use_rows_kernel = True
        self.rows_kernel_min_rows = 9
        self.use_tiles = True
        self.tiles_min_rows = 65
        self.use_qkv_tail = True
        self.use_fresh_decode = True
        self.fused_linear_shape = 0
        self.last_stat_blocks = 0
        self.last_best_parts = 0
        handle = ctypes.c_void_p()
        lib = self._lib("host")
        if lib.celeg_ops_create(ctypes.byref(handle)) != 0:
            raise KernelError(lib.celeg_last_error().decode())
        self._handle = handle

    def __del__(self):
        try:
            if self._library is not None and self._handle:
                self._library.celeg_ops_destroy(self._handle)
        except Exception:
            pass

    # ------------------------------------------------------------------ plumbing
    def _lib(self, module: str) -> ctypes.CDLL:
        """The built library (all kernel files and the host code are one library; ``module`` names
        the file a call belongs to, for the record of what ran).  Tests reach the kernels' own
        test hooks (a forced tile shape and the like) through it."""
        if self._library is None:
            path = build.ensure_built()
            try:
                lib = ctypes.CDLL(path)
            except OSError as err:
                raise KernelError(f"cannot load the built library {path}: {err}") from err
            lib.celeg_ops_create.restype = ctypes.c_int
            lib.celeg_ops_create.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
            lib.celeg_ops_destroy.restype = None
            lib.celeg_ops_destroy.argtypes = [ctypes.c_void_p]
            lib.celeg_ops_call.restype = ctypes.c_char_p
            lib.celeg_ops_call.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_void_p]
            lib.celeg_last_error.restype = ctypes.c_char_p
            self._library = lib
        self.loaded_libraries[module] = build.library_path() or ""
        return self._library

    def _knobs(self) -> dict:
        knobs = {name: int(getattr(self, name)) for name in self._KNOBS}
        knobs["decode_parts_few"], knobs["decode_parts_some"] = (int(v) for v in self.decode_part_thresholds)
        knobs["attention_general"] = int(self.attention_impl == "general")
        return knobs

    def _call(self, op: str, **args) -> dict:
        args["knobs"] = self._knobs()
        answer = self._lib(op).celeg_ops_call(self._handle, op.encode(), json.dumps(args).encode(),
                                              ctypes.c_void_p(_raw_stream(self._device_index)))
        if answer is None:
            raise KernelError(self._library.celeg_last_error().decode())
        out = json.loads(answer.decode())
        self.last_stat_blocks = out.get("last_stat_blocks", self.last_stat_blocks)
        self.last_best_parts = out.get("last_best_parts", 0)
        self.last_best_cols = out.get("last_best_cols", 0)
        return out

    def paths(self) -> Dict[str, int]:
        """How many launches each kernel family has taken through this dispatcher."""
        return self._call("state")["paths"]

    @staticmethod
    def chunked_rows(rows: int, width: int, device, max_rows: int = 64) -> torch.Tensor:
        """Room for ``rows`` bfloat16 rows of ``width`` values in the layout that the products
        for 9 to 64 rows read best: [width/8, max_rows, 8], returned as its view
        [rows, width/8, 8] (element (m, k) at [m, k // 8, k % 8])."""
        if width % 8 or rows > max_rows:
            raise KernelError("chunked_rows: the width must be a multiple of 8 and rows <= max_rows")
        return torch.empty(width // 8, max_rows, 8, dtype=torch.bfloat16, device=device).permute(1, 0, 2)[:rows]

    # ------------------------------------------------------------------ row-wise
    def embed(self, table, token_ids, out):
        if token_ids.numel() < out.shape[0]:
            raise KernelError("embed: one token id per output row is needed")
        self._call("embed", table=_tensor(table, "table"), token_ids=_address(token_ids, "token_ids"), out=_tensor(out, "out"))

    def rmsnorm(self, x, weight, eps, out, delta=None, rows=None):
        if rows is not None and rows.numel() != out.shape[0]:
            raise KernelError("rmsnorm: one output row per listed row is needed")
        self._call("rmsnorm", x=_tensor(x, "x"), weight=_tensor(weight, "weight"), eps=float(eps), out=_tensor(out, "out"),
                   delta=_tensor(delta, "delta"), rows=_address(rows, "rows"))

    def swiglu(self, gate_up, out):
        self._call("swiglu", gate_up=_tensor(gate_up, "gate_up"), out=_tensor(out, "out"))

    def add_bias(self, x, bias):
        self._call("add_bias", x=_tensor(x, "x"), bias=_tensor(bias, "bias"))

    def cast(self, src, dst):
        self._call("cast", src=_tensor(src, "src"), dst=_tensor(dst, "dst"))

    def apply_table_updates(self, table, updates, capacity):
        if updates.numel() < 1 + 3 * capacity:
            raise KernelError("apply_table_updates: the update list is shorter than its capacity")
        self._call("apply_table_updates", table=_tensor(table, "table"), updates=_address(updates, "updates"), capacity=int(capacity))

    def step_prologue(self, table, updates, capacity, token_ids, token_slot, last_tokens, n):
        """``apply_table_updates`` (capacity > 0) and ``resolve_tokens`` (``last_tokens`` given)
        in one launch."""
        if updates.numel() < 1 + 3 * capacity or token_ids.numel() < n or token_slot.numel() < n:
            raise KernelError("step_prologue: an array is shorter than its count")
        self._call("step_prologue", table=_tensor(table, "table"), updates=_address(updates, "updates"), capacity=int(capacity),
                   token_ids=_address(token_ids, "token_ids"), token_slot=_address(token_slot, "token_slot"),
                   last_tokens=_address(last_tokens, "last_tokens"), n=int(n))

    def resolve_tokens(self, token_ids, token_slot, last_tokens, n):
        """token_ids[i] = last_tokens[token_slot[i]] where token_ids[i] < 0 (i < n)."""
        if token_ids.numel() < n or token_slot.numel() < n:
            raise KernelError("resolve_tokens: fewer rows than n")
        self._call("resolve_tokens", token_ids=_address(token_ids, "token_ids"), token_slot=_address(token_slot, "token_slot"),
                   last_tokens=_address(last_tokens, "last_tokens"), n=int(n))

    # ------------------------------------------------------------------ matrix products
    def linear(self, x, w, out, bias=None):
        """out = x w^T (+ bias).  x [M,K] (rows may be strided), w [N,K], out [M,N] in the
        dtype of x or in 32-bit.  ``use_blaslt`` False keeps bfloat16 products of many rows away
        from hipBLASLt."""
        self._call("linear", x=_tensor(x, "x"), w=_tensor(w, "w"), out=_tensor(out, "out"), bias=_tensor(bias, "bias"))
        return out

    # ------------------------------------------------------------------ short convolution
    def short_conv(self, bcx, weight, bias, state, out, batch):
        self._call("short_conv", bcx=_tensor(bcx, "bcx"), weight=_tensor(weight, "weight"), bias=_tensor(bias, "bias"),
                   state=_tensor(state, "state"), out=_tensor(out, "out"), batch=_batch(batch))

    # ------------------------------------------------------------------ attention
    def qk_norm_rope_store(self, q, k, v, q_weight, k_weight, eps, inv_freq, rotary_dim,
                           heads, kv_heads, head_dim, batch, kv, pairing=0):
        self._call("qk_norm_rope_store", q=_tensor(q, "q"), k=_tensor(k, "k"), v=_tensor(v, "v"),
                   q_weight=_tensor(q_weight, "q_weight"), k_weight=_tensor(k_weight, "k_weight"), eps=float(eps),
                   inv_freq=_tensor(inv_freq, "inv_freq"), rotary_dim=int(rotary_dim or 0), pairing=int(pairing),
                   heads=int(heads), kv_heads=int(kv_heads), head_dim=int(head_dim), batch=_batch(batch), kv=_kv(kv))

    def paged_attention(self, q, out, heads, kv_heads, head_dim, scale, window, batch, kv, fresh=None):
        self._call("paged_attention", q=_tensor(q, "q"), out=_tensor(out, "out"), heads=int(heads), kv_heads=int(kv_heads),
                   head_dim=int(head_dim), scale=float(scale), window=int(window or 0), batch=_batch(batch), kv=_kv(kv),
                   fresh=fresh)

    def attention_decode_fresh(self, q, k, v, out, q_weight, k_weight, eps, inv_freq, heads, kv_heads, head_dim,
                               scale, window, batch, kv):
        """A decode-only step whose new keys and values are not in the cache yet: q, k and v as
        the q/k/v product left them; the attention kernel normalises and turns q and the new
        key, adds the new key and value as one more key and writes them into the pages."""
        fresh = {"k": _tensor(k, "k"), "v": _tensor(v, "v"), "q_weight": _tensor(q_weight, "q_weight"),
                 "k_weight": _tensor(k_weight, "k_weight"), "eps": float(eps), "inv_freq": _tensor(inv_freq, "inv_freq")}
        self.paged_attention(q, out, heads, kv_heads, head_dim, scale, window, batch, kv, fresh=fresh)

    def attention_fresh_ok(self, heads, head_dim, inv_freq, batch, kv, dtype=torch.bfloat16) -> bool:
        """Whether a decode-only step's attention would prepare and write the new keys itself."""
        return bool(self._call("attention_fresh_ok", heads=int(heads), head_dim=int(head_dim), batch=_batch(batch), kv=_kv(kv),
                               fresh={"inv_freq": _tensor(inv_freq, "inv_freq")}, dtype=_NAMES[dtype])["ok"])

    # ------------------------------------------------------------------ sampling
    def sample(self, logits, fparams, iparams, seen, out_tokens, last_tokens=None, all_greedy=False, row_best=None,
               row_best_parts=0, row_best_cols=0, penalised=False):
        """One token per row.  ``all_greedy``: the caller knows that every row takes its
        (penalised) largest logit; the rows are then cut into parts over many workgroups.
        ``row_best`` [>= rows, >= row_best_parts] (int64): what the head's product left beside these
        logits (``fused_linear(..., row_best=...)``, ``row_best_cols`` columns a part: ``last_best_cols``); greedy
        rows without a penalty (``penalised`` false) then take their token from it, and sampled rows look for
        their candidates in the columns of the parts it names instead of reading the row."""
        R, V = logits.shape
        if out_tokens.numel() != R or fparams.numel() < 4 * R or iparams.numel() < 3 * R:
            raise KernelError("sample: parameter arrays do not fit the rows")
        if seen is not None and seen.shape[1] != V:
            raise KernelError("sample: the seen table must be [slots, vocab]")
        self._call("sample", logits=_tensor(logits, "logits"), fparams=_address(fparams, "fparams", torch.float32),
                   iparams=_address(iparams, "iparams"), seen=_address(seen, "seen", torch.uint8),
                   seen_stride=int(seen.stride(0)) if seen is not None else 0, out_tokens=_address(out_tokens, "out_tokens"),
                   last_tokens=_address(last_tokens, "last_tokens"), all_greedy=bool(all_greedy),
                   row_best=_address(row_best, "row_best", torch.int64),
                   row_best_ld=int(row_best.stride(0)) if row_best is not None else 0, row_best_parts=int(row_best_parts),
                   row_best_cols=int(row_best_cols), penalised=bool(penalised))

    def mark_seen(self, seen, token_ids, token_slot, n):
        if token_ids.numel() < n or token_slot.numel() < n:
            raise KernelError("mark_seen: fewer rows than n")
        self._call("mark_seen", seen=_tensor(seen, "seen"), token_ids=_address(token_ids, "token_ids"),
                   token_slot=_address(token_slot, "token_slot"), n=int(n))

    # ------------------------------------------------------------------ fused skinny products
    has_fused_linear = True

    def fused_linear_ok(self, rows: int, *inner_sizes: int) -> bool:
        """Whether the fused skinny product takes ``rows`` rows and these inner sizes."""
        return bool(self._call("fused_linear_ok", rows=int(rows), inner=[int(k) for k in inner_sizes])["ok"])

    def rows_kernel_ok(self, rows: int, *inner_sizes: int) -> bool:
        """Whether bfloat16 products of ``rows`` rows with these inner sizes go to the kernel
        for 9 to 64 rows."""
        return bool(self._call("rows_kernel_ok", rows=int(rows), inner=[int(k) for k in inner_sizes])["ok"])

    def residual_stat_blocks(self, rows: int, n: int, k: int) -> int:
        """How many partial sums of squares per row the "residual" epilogue of
        ``fused_linear`` leaves for these sizes (the rows ``stats_out`` needs)."""
        return int(self._call("residual_stat_blocks", rows=int(rows), n=int(n), k=int(k))["blocks"])

    def pack_weight(self, w: torch.Tensor) -> torch.Tensor:
        """``w`` [rows, K] as [K/32, rows, 32]: blocks of 32 k-values with the rows side by
        side inside a block, the layout in which the k-sliced products read whole runs of
        memory per load (made by the library's own ``fold_weight``)."""
        return self.fold_weight(w, None, packed=True)

    def fold_weight(self, w, scale=None, packed=False) -> torch.Tensor:
        """``w`` [rows, K] with column k multiplied by ``scale[k]`` (rounded to bfloat16 again), as
        it is or, ``packed``, as [K/32, rows, 32]."""
        rows, K = w.shape
        if packed and K % 32:
            raise KernelError("pack_weight: the inner size must be a multiple of 32")
        out = torch.empty((K // 32, rows, 32) if packed else (rows, K), dtype=torch.bfloat16, device=w.device)
        self._call("fold_weight", w=_tensor(w, "w"), scale=_tensor(scale, "scale"), packed=bool(packed), out=_tensor(out, "out"))
        return out

    def stream_prepare(self, h, xb, stats):
        """The bfloat16 copy ``xb`` of the 32-bit stream ``h`` and its rows' sums of squares
        (``stats[:rows, 0]``)."""
        self._call("stream_prepare", h=_tensor(h, "h"), xb=_tensor(xb, "xb"), stats=_tensor(stats, "stats"))

    def embed_stream(self, table, token_ids, out, xb, stats):
        """Embedding gather into the 32-bit stream ``out``, its bfloat16 copy ``xb`` and the
        rows' sums of squares (``stats[:rows, 0]``)."""
        if token_ids.numel() < out.shape[0]:
            raise KernelError("embed_stream: shapes do not fit")
        self._call("embed_stream", table=_tensor(table, "table"), token_ids=_address(token_ids, "token_ids"),
                   out=_tensor(out, "out"), xb=_tensor(xb, "xb"), stats=_tensor(stats, "stats"))

    def embed_stats(self, table, token_ids, out, stats):
        """Embedding gather that also leaves every row's sum of squares in ``stats[:rows, 0]``."""
        if token_ids.numel() < out.shape[0]:
            raise KernelError("embed_stats: shapes do not fit")
        self._call("embed_stats", table=_tensor(table, "table"), token_ids=_address(token_ids, "token_ids"),
                   out=_tensor(out, "out"), stats=_tensor(stats, "stats"))

    def fused_linear(self, a, w, out, *, epilogue="store", norm_weight=None, eps=0.0, stats=None,
                     stat_blocks=0, rows=None, bias=None, stats_out=None, conv=None, n_rows=None,
                     out_bf16=None, row_best=None):
        """out = epilogue(prologue(a) w^T) for up to 64 rows, bfloat16 weights (``Ops::fused_linear``).
        ``row_best`` (int64 [>= rows, >= parts], with "store_f32"): receives the best (logit, index) of every
        share of a row's columns; ``last_best_parts`` says how many parts were written.

        ``a``: bfloat16 rows [M, K], or, with ``norm_weight``, the 32-bit residual stream,
        normalised on the fly (``stats[row, :stat_blocks]`` holding partial sums of squares
        of its rows if ``stat_blocks`` > 0).  ``rows`` picks rows of ``a``.  Epilogues: "store"
        (bfloat16 [M, N]), "store_f32", "residual" (``out`` is the stream, [M, N] 32-bit,
        added to in place; ``stats_out`` [>= M, ``residual_stat_blocks``] receives partial
        sums of squares of the new rows, ``last_stat_blocks`` says how many a row), "swiglu"
        (``w`` is [2N, K]: gate rows then up rows), "conv" (``w`` is [3N, K]: B, C, x rows;
        ``conv`` = (taps [N, L], bias or None, state [slots, L, N], seq_slot [M]); one new token
        per request).  ``w`` with three dimensions is in the layout of ``pack_weight``."""
        if n_rows is None and rows is not None:
            n_rows = rows.numel()
        conv_json = None
        if conv is not None:
            taps, conv_bias, state, seq_slot = conv
            conv_json = {"taps": _tensor(taps, "conv taps"), "bias": _tensor(conv_bias, "conv bias"),
                         "state": _tensor(state, "state"), "seq_slot": _address(seq_slot, "seq_slot")}
        self._call("fused_linear", a=_tensor(a, "a"), w=_tensor(w, "w"), out=_tensor(out, "out"), epilogue=epilogue,
                   norm_weight=_tensor(norm_weight, "norm_weight"), eps=float(eps), stats=_tensor(stats, "stats"),
                   stat_blocks=int(stat_blocks), rows=_address(rows, "rows"), n_rows=-1 if n_rows is None else int(n_rows),
                   bias=_tensor(bias, "bias"), stats_out=_tensor(stats_out, "stats_out"), conv=conv_json,
                   out_bf16=_tensor(out_bf16, "out_bf16"), packed=w.dim() == 3,
                   row_best=_address(row_best, "row_best", torch.int64),
                   row_best_ld=int(row_best.stride(0)) if row_best is not None else 0,
                   row_best_rows=int(row_best.shape[0]) if row_best is not None else 0)
        return out

    # ------------------------------------------------------------------ fused products of many rows
    def tiled_linear_ok(self, rows: int, n: int, *inner_sizes: int) -> bool:
        """Whether the fused bfloat16 product for many rows takes these sizes."""
        return bool(self._call("tiled_linear_ok", rows=int(rows), n=int(n), inner=[int(k) for k in inner_sizes])["ok"])

    def tiled_stat_blocks(self, rows: int, n: int, k: int) -> int:
        """Partial sums of squares per row that the "residual" epilogue of ``tiled_linear``
        leaves for these sizes."""
        return int(self._call("tiled_stat_blocks", rows=int(rows), n=int(n), k=int(k))["blocks"])

    def tiled_linear(self, a, w, out, *, epilogue="store", eps=0.0, stats=None, stat_blocks=0,
                     bias=None, stats_out=None, out_bf16=None, qkv=None):
        """out = epilogue(scale * (a w^T) + bias) for many bfloat16 rows (``Ops::tiled_linear``).

        ``qkv`` (with "store"): a dict ``heads, kv_heads, q_weight, k_weight, eps, inv_freq
        ([32] 32-bit or None), batch, kv``: the columns are heads of 64; query heads are
        normalised, turned and stored to ``out``, key heads likewise and stored to their rows'
        pages, value heads stored to the pages (what ``qk_norm_rope_store`` does behind a product)."""
        tail = None
        if qkv is not None:
            tail = {"heads": int(qkv["heads"]), "kv_heads": int(qkv["kv_heads"]), "head_dim": int(qkv.get("head_dim", 64)),
                    "q_weight": _tensor(qkv.get("q_weight"), "q_weight"), "k_weight": _tensor(qkv.get("k_weight"), "k_weight"),
                    "eps": float(qkv.get("eps", 0.0)), "inv_freq": _tensor(qkv.get("inv_freq"), "inv_freq"),
                    "batch": _batch(qkv["batch"]), "kv": _kv(qkv["kv"])}
        self._call("tiled_linear", a=_tensor(a, "a"), w=_tensor(w, "w"), out=_tensor(out, "out"), epilogue=epilogue,
                   eps=float(eps), stats=_tensor(stats, "stats"), stat_blocks=int(stat_blocks), bias=_tensor(bias, "bias"),
                   stats_out=_tensor(stats_out, "stats_out"), out_bf16=_tensor(out_bf16, "out_bf16"), qkv=tail)
        return out

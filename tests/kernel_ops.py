"""The kernels as Python calls on torch tensors, for the tests of single kernels.  (The
engine does not come through here: its host code, ``celeg_amd/csrc/host/ops.cpp``, makes the
same checks and calls in C++.)  Shapes are checked on the host, then the extern "C" entry
points of the built library are called through ``ctypes`` with raw device pointers and the
current HIP stream (so a stream that is capturing a graph captures them too).  There is no
fallback: if the library cannot be built or loaded, or a tensor is not on the GPU, the call
fails loudly.  ``linear`` goes through the library's own dispatch (``celeg_ops_linear``).
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional

import torch

from celeg_amd.csrc import build

_DT = {torch.float32: 0, torch.bfloat16: 1}
_c_int, _c_float, _c_void_p, _c_size_t = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t


class KernelError(RuntimeError):
    pass


def _raw_stream(device_index: int) -> int:
    """The raw handle of torch's current stream on a device."""
    return torch._C._cuda_getCurrentRawStream(device_index)


def _ptr(t: Optional[torch.Tensor]):
    return _c_void_p(0 if t is None else t.data_ptr())


class HipOps:
    def __init__(self, device="cuda:0"):
        if not torch.cuda.is_available():
            raise KernelError("celeg_amd needs a GPU: torch.cuda.is_available() is False and "
                              "there is no CPU path")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise KernelError(f"celeg_amd runs on a GPU only, not on '{device}'")
        self._libs: Dict[str, ctypes.CDLL] = {}
        self.loaded_libraries: Dict[str, str] = {}
        # "auto": the matrix-core and split-key kernels where they apply; "general": always
        # the general kernel (tests compare the two)
        self.attention_decode_whole = -1     # -1: chosen from the batch; 0 split-key kernels; 1 one workgroup per request and key/value head
        self.use_blaslt = True               # products of many rows: hipBLASLt called directly
        self._device_index = torch.device(device).index if torch.device(device).index is not None \
            else torch.cuda.current_device()
        self.attention_rows_per_tile = 0     # 0: the kernel chooses; 64 or 128 to force
        self.attention_rows_form = 0         # 0: the kernel chooses; 1 to 4 to force (see attention_fast.hip)
        # decode attention over few requests: contexts of up to this many rounds of 64 keys are
        # cut into parts of 1 round, up to that many into parts of 4, longer ones into parts of 16
        self.decode_part_thresholds = (64, 256)
        self.attention_impl = "auto"
        self._decode_ws = None
        self._retired = []
        self._rope_tables = {}
        self.use_rope_table = True         # cos/sin of every position from a table made once
        self.use_argmax_parts = True       # up to 16 greedy rows: many workgroups a row (1 row 6.9 against 11.8 us, 8 rows 8.2 against 11.4)
        self._argmax_state = None
        self.use_sliced = True             # up to 16 bfloat16 rows: the k-sliced kernels
        self.use_rows_kernel = True        # 9 to 64 bfloat16 rows: the kernel that streams the weights
        # fewest rows it is used for (it takes any number up to 64).  Measured per decode step: at 16
        # rows it equals the k-sliced kernels on 1,024-wide layers and is 20 % faster on 2,048-wide
        # ones (1.55 against 1.94 ms at the 2.6B shape); at 8 rows it loses 19 % on the former
        self.rows_kernel_min_rows = 9
        self.use_tiles = True              # fused bfloat16 products of many rows (gemm_tiles.hip)
        self.tiles_min_rows = 65
        self.last_stat_blocks = 0
        self.fused_linear_shape = 0        # 0: chosen from the sizes; 1..4 force a workgroup shape

    # ------------------------------------------------------------------ plumbing
    def _lib(self, module: str) -> ctypes.CDLL:
        """The built library (all kernel files are in the one library; ``module`` names the file
        a call belongs to, for the record of what ran)."""
        lib = self._libs.get("library")
        if lib is None:
            path = build.ensure_built()
            try:
                lib = ctypes.CDLL(path)
            except OSError as err:
                raise KernelError(f"cannot load the built library {path}: {err}") from err
            if lib.celeg_gemv_params_size() != ctypes.sizeof(_GemvParams):
                raise KernelError("the argument block of the skinny products does not match the built kernels")
            if lib.celeg_gemm_tiles_params_size() != ctypes.sizeof(_TileParams):
                raise KernelError("the argument block of the tiled products does not match the built kernels")
            self._libs["library"] = lib
        self.loaded_libraries[module] = build.library_path() or ""
        return lib

    def _stream(self):
        # (the raw handle of torch's current stream, without building a stream object per launch)
        return _c_void_p(_raw_stream(self._device_index))

    def _check(self, code: int, what: str) -> None:
        if code != 0:
            raise KernelError(f"{what}: HIP error {code}")

    def _dev(self, t: torch.Tensor, name: str, dtype=None, contiguous=True):
        if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
            raise KernelError(f"{name} must be a GPU tensor")
        if dtype is not None and t.dtype != dtype:
            raise KernelError(f"{name} must be {dtype}, got {t.dtype}")
        if contiguous and not t.is_contiguous():
            raise KernelError(f"{name} must be contiguous")
        return t

    @staticmethod
    def _rows(t: torch.Tensor, name: str) -> int:
        """Row stride of a 2-D tensor whose rows are dense."""
        if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
            raise KernelError(f"{name} must be 2-D with dense rows")
        return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])

    def _operand(self, t: torch.Tensor, name: str):
        """(rows, width, row stride, stride of a group of 8 values) of a bfloat16 operand:
        [rows, width] with dense rows, or [rows, width/8, 8], a view of a buffer in which the
        rows lie side by side inside every group of 8 values (``chunked_rows``)."""
        if t.dim() == 2:
            return t.shape[0], t.shape[1], self._rows(t, name), 8
        if t.dim() != 3 or t.shape[2] != 8 or t.stride(2) != 1:
            raise KernelError(f"{name} must be [rows, width] or [rows, width/8, 8]")
        return t.shape[0], t.shape[1] * 8, t.stride(0), t.stride(1)

    @staticmethod
    def chunked_rows(rows: int, width: int, device, max_rows: int = 64) -> torch.Tensor:
        """Room for ``rows`` bfloat16 rows of ``width`` values in the layout that the products
        for 9 to 64 rows read best: [width/8, max_rows, 8], returned as its view
        [rows, width/8, 8] (element (m, k) at [m, k // 8, k % 8])."""
        if width % 8 or rows > max_rows:
            raise KernelError("chunked_rows: the width must be a multiple of 8 and rows <= max_rows")
        return torch.empty(width // 8, max_rows, 8, dtype=torch.bfloat16, device=device).permute(1, 0, 2)[:rows]

    def _dtype(self, t: torch.Tensor, name: str) -> int:
        if t.dtype not in _DT:
            raise KernelError(f"{name}: dtype {t.dtype} is not supported (float32, bfloat16)")
        return _DT[t.dtype]

    # ------------------------------------------------------------------ row-wise
    def embed(self, table, token_ids, out):
        self._dev(table, "table"); self._dev(token_ids, "token_ids", torch.int32)
        self._dev(out, "out", torch.float32)
        rows, width = out.shape
        if table.dim() != 2 or table.shape[1] != width or token_ids.numel() != rows:
            raise KernelError("embed: shapes do not fit")
        code = self._lib("elementwise").celeg_embed(
            _ptr(table), _c_int(self._dtype(table, "table")), _ptr(token_ids), _ptr(out),
            _c_int(rows), _c_int(width), _c_int(table.shape[0]), self._stream())
        self._check(code, "embed")

    def rmsnorm(self, x, weight, eps, out, delta=None, rows=None):
        self._dev(x, "x"); self._dev(weight, "weight", torch.float32); self._dev(out, "out")
        width = x.shape[-1]
        n_rows = out.shape[0]
        if x.dim() != 2 or out.dim() != 2 or out.shape[1] != width or weight.numel() != width:
            raise KernelError("rmsnorm: shapes do not fit")
        if delta is not None:
            self._dev(delta, "delta")
            if delta.shape != x.shape:
                raise KernelError("rmsnorm: delta must have the shape of x")
        if rows is not None:
            self._dev(rows, "rows", torch.int32)
            if rows.numel() != n_rows:
                raise KernelError("rmsnorm: one output row per listed row is needed")
        elif n_rows != x.shape[0]:
            raise KernelError("rmsnorm: out must have the rows of x")
        write_back = 1 if (delta is not None and rows is None) else 0
        if write_back and x.dtype != torch.float32:
            raise KernelError("rmsnorm: the sum can only be written back to a 32-bit x")
        code = self._lib("elementwise").celeg_rmsnorm(
            _ptr(x), _c_int(self._dtype(x, "x")), _ptr(delta),
            _c_int(self._dtype(delta, "delta") if delta is not None else 0), _ptr(weight),
            _ptr(out), _c_int(self._dtype(out, "out")), _ptr(rows), _c_int(n_rows),
            _c_int(width), _c_float(eps), _c_int(write_back), self._stream())
        self._check(code, "rmsnorm")

    def swiglu(self, gate_up, out):
        self._dev(gate_up, "gate_up"); self._dev(out, "out", gate_up.dtype)
        rows, ff = out.shape
        if gate_up.shape != (rows, 2 * ff):
            raise KernelError("swiglu: gate_up must be [rows, 2*ff]")
        code = self._lib("elementwise").celeg_swiglu(
            _ptr(gate_up), _ptr(out), _c_int(self._dtype(out, "out")), _c_int(rows), _c_int(ff),
            self._stream())
        self._check(code, "swiglu")

    def add_bias(self, x, bias):
        self._dev(x, "x"); self._dev(bias, "bias", torch.float32)
        rows, width = x.shape
        if bias.numel() != width:
            raise KernelError("add_bias: bias must have the width of x")
        code = self._lib("elementwise").celeg_add_bias(
            _ptr(x), _c_int(self._dtype(x, "x")), _ptr(bias), _c_int(rows), _c_int(width),
            self._stream())
        self._check(code, "add_bias")

    def cast(self, src, dst):
        self._dev(src, "src"); self._dev(dst, "dst")
        if src.numel() != dst.numel():
            raise KernelError("cast: sizes differ")
        code = self._lib("elementwise").celeg_cast(
            _ptr(src), _c_int(self._dtype(src, "src")), _ptr(dst),
            _c_int(self._dtype(dst, "dst")), _c_size_t(src.numel()), self._stream())
        self._check(code, "cast")

    def apply_table_updates(self, table, updates, capacity):
        self._dev(table, "table", torch.int32); self._dev(updates, "updates", torch.int32)
        if updates.numel() < 1 + 3 * capacity:
            raise KernelError("apply_table_updates: the update list is shorter than its capacity")
        code = self._lib("elementwise").celeg_table_update(
            _ptr(table), _c_int(table.shape[1]), _c_int(table.shape[0]), _ptr(updates),
            _c_int(capacity), self._stream())
        self._check(code, "apply_table_updates")

    def step_prologue(self, table, updates, capacity, token_ids, token_slot, last_tokens, n):
        """``apply_table_updates`` (capacity > 0) and ``resolve_tokens`` (``last_tokens`` given)
        in one launch."""
        self._dev(table, "table", torch.int32); self._dev(updates, "updates", torch.int32)
        if capacity <= 0 or updates.numel() < 1 + 3 * capacity:
            raise KernelError("step_prologue: the update list is shorter than its capacity")
        for t, name in ((token_ids, "token_ids"), (token_slot, "token_slot")):
            self._dev(t, name, torch.int32)
        if last_tokens is not None:
            self._dev(last_tokens, "last_tokens", torch.int32)
            if token_ids.numel() < n or token_slot.numel() < n:
                raise KernelError("step_prologue: fewer rows than n")
        code = self._lib("elementwise").celeg_step_prologue(
            _ptr(table), _c_int(table.shape[1]), _c_int(table.shape[0]), _ptr(updates), _c_int(capacity),
            _ptr(token_ids), _ptr(token_slot), _ptr(last_tokens), _c_int(n), self._stream())
        self._check(code, "step_prologue")

    # ------------------------------------------------------------------ matrix products
    def linear(self, x, w, out, bias=None):
        """out = x w^T (+ bias).  x [M,K] (rows may be strided), w [N,K], out [M,N] in the
        dtype of x or in 32-bit: the library's own dispatch (``Ops::linear``), the one the parts
        call.  ``use_blaslt`` False keeps bfloat16 products of many rows away from hipBLASLt."""
        from celeg_amd import native
        for t, name in ((x, "x"), (w, "w"), (out, "out")):
            if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
                raise KernelError(f"linear: {name} must be a matrix on the GPU with dense rows")
        codes = {torch.float32: 0, torch.bfloat16: 1}
        if x.dtype not in codes or w.dtype not in codes or out.dtype not in codes:
            raise KernelError(f"linear: unsupported dtypes {x.dtype} x {w.dtype} -> {out.dtype}")
        if not w.is_contiguous():
            raise KernelError("linear: w must be contiguous")
        if bias is not None:
            self._dev(bias, "bias", torch.float32)
        M, K = x.shape
        if w.shape[1] != K or out.shape != (M, w.shape[0]):
            raise KernelError(f"linear: shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
        lib = native.lib()
        lib.celeg_ops_linear.restype = ctypes.c_int
        lib.celeg_ops_linear.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int32,
                                         ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p] + \
            [ctypes.c_int32] * 4 + [ctypes.c_void_p]
        try:
            native.check(lib.celeg_ops_linear(
                x.data_ptr(), codes[x.dtype], x.stride(0) if M > 1 else max(x.stride(0), K), w.data_ptr(), codes[w.dtype],
                out.data_ptr(), codes[out.dtype], out.stride(0) if M > 1 else max(out.stride(0), out.shape[1]),
                bias.data_ptr() if bias is not None else None, M, w.shape[0], K, int(self.use_blaslt), _raw_stream(self._device_index)))
        except (native.NativeError, native.NativeArgumentError) as err:
            raise KernelError(str(err)) from None
        return out

    # ------------------------------------------------------------------ short convolution
    def short_conv(self, bcx, weight, bias, state, out, batch):
        self._dev(bcx, "bcx"); self._dev(weight, "weight", torch.float32)
        self._dev(state, "state", torch.float32, contiguous=False); self._dev(out, "out", bcx.dtype)
        T, width = out.shape
        taps = weight.shape[1]
        if bcx.shape != (T, 3 * width) or weight.shape[0] != width or T != batch.n_tokens:
            raise KernelError("short_conv: shapes do not fit")
        if state.dim() != 3 or state.shape[1:] != (taps, width) or state.stride(2) != 1 \
                or state.stride(1) != width:
            raise KernelError("short_conv: state must be [slots, taps, width] with dense slots")
        if bias is not None:
            self._dev(bias, "bias", torch.float32)
        code = self._lib("short_conv").celeg_short_conv(
            _ptr(bcx), _c_int(3 * width), _c_int(self._dtype(bcx, "bcx")), _ptr(weight), _ptr(bias),
            _ptr(state), _c_size_t(state.stride(0)), _ptr(out), _ptr(batch.positions),
            _ptr(batch.token_seq), _ptr(batch.seq_start), _ptr(batch.seq_slot),
            _ptr(batch.cu_seqlens), _c_int(batch.n_tokens), _c_int(batch.n_seqs), _c_int(width),
            _c_int(taps), self._stream())
        self._check(code, "short_conv")

    # ------------------------------------------------------------------ attention
    def _check_kv(self, kv, kv_heads, head_dim, dtype):
        if kv.kv_heads != kv_heads or kv.head_dim != head_dim:
            raise KernelError("attention: the cache has other head sizes than the mixer")
        self._dev(kv.k, "k cache", dtype); self._dev(kv.v, "v cache", dtype)
        if kv.k.shape[1:] != (kv.n_layers, kv_heads, kv.page_tokens, head_dim) or \
                kv.v.shape[1:] != (kv.n_layers, kv_heads, head_dim, kv.page_tokens):
            raise KernelError("attention: unexpected cache shape")
        self._dev(kv.table, "block table", torch.int32)
        if not 0 <= kv.layer < kv.n_layers:
            raise KernelError("attention: layer index outside the cache")

    def _rope_table(self, inv_freq, n_positions: int) -> torch.Tensor:
        """cos and sin of position * frequency for every position a request can reach
        ([n_positions, rotary_dim/2, 2], 32-bit), made once per frequency table."""
        key = (inv_freq.data_ptr(), n_positions)
        table = self._rope_tables.get(key)
        if table is None:
            table = torch.empty((n_positions, inv_freq.numel(), 2), dtype=torch.float32,
                                device=inv_freq.device)
            code = self._lib("attention").celeg_rope_table(
                _ptr(inv_freq), _c_int(inv_freq.numel()), _c_int(n_positions), _ptr(table),
                self._stream())
            self._check(code, "rope_table")
            self._rope_tables[key] = (table, inv_freq)   # the key's tensor is kept alive with it
            return table
        return table[0]

    def qk_norm_rope_store(self, q, k, v, q_weight, k_weight, eps, inv_freq, rotary_dim,
                           heads, kv_heads, head_dim, batch, kv, pairing=0):
        self._dev(q, "q", contiguous=False)
        T = q.shape[0]
        dtype = q.dtype
        if T != batch.n_tokens or q.shape[1] != heads * head_dim:
            raise KernelError("qk_norm_rope_store: q must be [rows, heads*head_dim]")
        if head_dim % 2 or head_dim > 1024:
            raise KernelError(f"qk_norm_rope_store: head_dim {head_dim} must be even and <= 1024")
        self._check_kv(kv, kv_heads, head_dim, dtype)
        store = k is not None
        if store:
            self._dev(k, "k", dtype, contiguous=False); self._dev(v, "v", dtype, contiguous=False)
            if k.shape != (T, kv_heads * head_dim) or v.shape != k.shape:
                raise KernelError("qk_norm_rope_store: k and v must be [rows, kv_heads*head_dim]")
        for name, wt in (("q_weight", q_weight), ("k_weight", k_weight)):
            if wt is not None:
                self._dev(wt, name, torch.float32)
                if wt.numel() != head_dim:
                    raise KernelError(f"qk_norm_rope_store: {name} must have head_dim entries")
        if inv_freq is not None:
            self._dev(inv_freq, "inv_freq", torch.float32)
            if rotary_dim % 2 or rotary_dim > head_dim or inv_freq.numel() != rotary_dim // 2:
                raise KernelError("qk_norm_rope_store: rotary_dim and the frequency table disagree")
        cos_sin = None
        if inv_freq is not None and rotary_dim > 0 and self.use_rope_table:
            cos_sin = self._rope_table(inv_freq, kv.table.shape[1] * kv.page_tokens)
        code = self._lib("attention").celeg_qk_norm_rope_store(
            _ptr(q), _c_int(self._rows(q, "q")), _ptr(k), _c_int(self._rows(k, "k") if store else 0),
            _ptr(v), _c_int(self._rows(v, "v") if store else 0), _c_int(self._dtype(q, "q")),
            _ptr(q_weight), _ptr(k_weight if store else None), _c_float(eps), _ptr(inv_freq),
            _ptr(cos_sin), _c_int(rotary_dim), _c_int(pairing), _ptr(batch.positions), _ptr(batch.token_slot), _ptr(kv.table),
            _c_int(kv.table.shape[1]), _ptr(kv.k), _ptr(kv.v), _c_int(kv.n_layers),
            _c_int(kv.layer), _c_int(kv.page_tokens), _c_int(T), _c_int(heads), _c_int(kv_heads),
            _c_int(head_dim), _c_int(1 if store else 0), self._stream())
        self._check(code, "qk_norm_rope_store")

    def paged_attention(self, q, out, heads, kv_heads, head_dim, scale, window, batch, kv):
        self._dev(q, "q", contiguous=False); self._dev(out, "out", q.dtype)
        T = q.shape[0]
        if T != batch.n_tokens or q.shape[1] != heads * head_dim or out.shape != (T, heads * head_dim):
            raise KernelError("paged_attention: q and out must be [rows, heads*head_dim]")
        if head_dim > 256:
            raise KernelError(f"paged_attention: head_dim {head_dim} exceeds 256")
        if heads % kv_heads:
            raise KernelError("paged_attention: heads must be a multiple of kv_heads")
        self._check_kv(kv, kv_heads, head_dim, q.dtype)
        if q.dtype == torch.bfloat16 and self.attention_impl != "general" \
                and kv.page_tokens >= 16 and kv.page_tokens & (kv.page_tokens - 1) == 0 \
                and self._rows(q, "q") % 8 == 0:
            if batch.decode_only and head_dim in (64, 128) and batch.n_seqs == T:
                return self._attention_decode(q, out, heads, kv_heads, head_dim, scale, window,
                                              batch, kv, T)
            if head_dim in (32, 64, 96, 128):
                # entries of one token lie first: they go to the kernel for single rows (a
                # tile of the rows kernel would hold one row), the portions to the rows kernel
                single = batch.single_rows if head_dim in (64, 128) else 0
                if single:
                    self._attention_decode(q, out, heads, kv_heads, head_dim, scale, window,
                                           batch, kv, single)
                if single < batch.n_seqs:
                    code = self._lib("attention_fast").celeg_attention_rows_bf16(
                        _ptr(q), _c_int(self._rows(q, "q")), _ptr(kv.k), _ptr(kv.v), _ptr(kv.table),
                        _c_int(kv.table.shape[1]), _ptr(batch.cu_seqlens[single:]),
                        _ptr(batch.seq_slot[single:]), _ptr(batch.seq_start[single:]),
                        _c_int(batch.n_seqs - single), _c_int(T - single), _ptr(out),
                        _c_int(heads * head_dim), _c_int(heads), _c_int(kv_heads), _c_int(head_dim),
                        _c_int(kv.page_tokens), _c_int(kv.n_layers), _c_int(kv.layer), _c_float(scale),
                        _c_int(window if window else 0), _c_int(self.attention_rows_per_tile),
                        _c_int(self.attention_rows_form),
                        _c_int(getattr(batch, "context_bound", 0) or getattr(batch, "max_context_len", 0) or 0),
                        self._stream())
                    self._check(code, "attention over rows (bfloat16)")
                return
        code = self._lib("attention").celeg_paged_attention(
            _ptr(q), _c_int(self._rows(q, "q")), _ptr(kv.k), _ptr(kv.v),
            _c_int(self._dtype(q, "q")), _ptr(kv.table), _c_int(kv.table.shape[1]),
            _ptr(batch.token_slot), _ptr(batch.positions), _ptr(out), _c_int(heads * head_dim),
            _c_int(T), _c_int(heads), _c_int(kv_heads), _c_int(head_dim), _c_int(kv.page_tokens),
            _c_int(kv.n_layers), _c_int(kv.layer), _c_float(scale),
            _c_int(window if window else 0), self._stream())
        self._check(code, "paged_attention")

    def attention_decode_fresh(self, q, k, v, out, q_weight, k_weight, eps, inv_freq, heads, kv_heads, head_dim,
                               scale, window, batch, kv):
        """A decode-only step whose new keys and values are not in the cache yet: q, k and v as
        the q/k/v product left them; the attention kernel normalises and turns q and the new
        key, adds the new key and value as one more key and writes them into the pages."""
        cos_sin = self._rope_table(inv_freq, kv.table.shape[1] * kv.page_tokens) if inv_freq is not None else None
        self._attention_decode(q, out, heads, kv_heads, head_dim, scale, window, batch, kv, q.shape[0],
                               fresh=(k, v, q_weight, k_weight, eps, cos_sin))

    def _attention_decode(self, q, out, heads, kv_heads, head_dim, scale, window, batch, kv, T, fresh=None):
        """The first ``T`` rows of the step, each the one new token of its request."""
        max_context = kv.table.shape[1] * kv.page_tokens
        n_splits = (max_context + 63) // 64          # the kernel takes 64 keys a wavefront
        need = T * heads * n_splits * (head_dim + 2)
        if self._decode_ws is None or self._decode_ws.numel() < need:
            if self._decode_ws is not None:
                self._retired.append(self._decode_ws)   # recorded graphs may still point at it
            self._decode_ws = torch.empty(need, dtype=torch.float32, device=q.device)
        # where the context is cut into parts (few requests): parts of 1, 4 or 16 rounds of 64
        # keys, so that a long context gets longer parts rather than hundreds of them; the
        # bound is the step's longest context, or what the step's recorded graph is good for
        bound = getattr(batch, "context_bound", 0) or getattr(batch, "max_context_len", 0) or max_context
        rounds = (min(bound, max_context) + 63) // 64
        few, some = self.decode_part_thresholds
        split_rounds = 1 if rounds <= few else (4 if rounds <= some else 16)
        n_parts = (rounds + split_rounds - 1) // split_rounds
        ws_o = self._decode_ws[:T * heads * n_splits * head_dim]
        ws_ml = self._decode_ws[T * heads * n_splits * head_dim:need]
        if fresh is not None:
            k, v, q_weight, k_weight, eps, cos_sin = fresh
            code = self._lib("attention_fast").celeg_attention_decode_fresh_bf16(
                _ptr(q), _c_int(self._rows(q, "q")), _ptr(k), _c_int(self._rows(k, "k")), _ptr(v), _c_int(self._rows(v, "v")),
                _ptr(q_weight), _ptr(k_weight), _c_float(eps), _ptr(cos_sin), _ptr(kv.k), _ptr(kv.v), _ptr(kv.table),
                _c_int(kv.table.shape[1]), _ptr(batch.token_slot), _ptr(batch.positions), _ptr(ws_o),
                _ptr(ws_ml), _c_int(n_splits), _ptr(out), _c_int(heads * head_dim),
                _c_int(T), _c_int(heads), _c_int(kv_heads), _c_int(head_dim), _c_int(kv.page_tokens),
                _c_int(kv.n_layers), _c_int(kv.layer), _c_float(scale),
                _c_int(window if window else 0), _c_int(self.attention_decode_whole),
                _c_int(split_rounds), _c_int(n_parts), self._stream())
            self._check(code, "attention for decode rows with fresh keys (bfloat16)")
            return
        code = self._lib("attention_fast").celeg_attention_decode_bf16(
            _ptr(q), _c_int(self._rows(q, "q")), _ptr(kv.k), _ptr(kv.v), _ptr(kv.table),
            _c_int(kv.table.shape[1]), _ptr(batch.token_slot), _ptr(batch.positions), _ptr(ws_o),
            _ptr(ws_ml), _c_int(n_splits), _ptr(out), _c_int(heads * head_dim),
            _c_int(T), _c_int(heads), _c_int(kv_heads), _c_int(head_dim), _c_int(kv.page_tokens),
            _c_int(kv.n_layers), _c_int(kv.layer), _c_float(scale),
            _c_int(window if window else 0), _c_int(self.attention_decode_whole),
            _c_int(split_rounds), _c_int(n_parts), self._stream())
        self._check(code, "attention for decode rows (bfloat16)")

    # ------------------------------------------------------------------ sampling
    def resolve_tokens(self, token_ids, token_slot, last_tokens, n):
        """token_ids[i] = last_tokens[token_slot[i]] where token_ids[i] < 0 (i < n)."""
        for t, name in ((token_ids, "token_ids"), (token_slot, "token_slot"), (last_tokens, "last_tokens")):
            self._dev(t, name, torch.int32)
        if token_ids.numel() < n or token_slot.numel() < n:
            raise KernelError("resolve_tokens: fewer rows than n")
        code = self._lib("elementwise").celeg_resolve_tokens(
            _ptr(token_ids), _ptr(token_slot), _ptr(last_tokens), _c_int(n), self._stream())
        self._check(code, "resolve_tokens")

    def sample(self, logits, fparams, iparams, seen, out_tokens, last_tokens=None, all_greedy=False):
        """One token per row.  ``all_greedy``: the caller knows that every row takes its
        (penalised) largest logit; the rows are then cut into parts over many workgroups."""
        self._dev(logits, "logits", torch.float32, contiguous=False)
        self._dev(fparams, "fparams", torch.float32); self._dev(iparams, "iparams", torch.int32)
        self._dev(out_tokens, "out_tokens", torch.int32)
        R, V = logits.shape
        if out_tokens.numel() != R or fparams.numel() < 4 * R or iparams.numel() < 3 * R:
            raise KernelError("sample: parameter arrays do not fit the rows")
        if last_tokens is not None:
            self._dev(last_tokens, "last_tokens", torch.int32)
        if seen is not None:
            self._dev(seen, "seen", torch.uint8)
            if seen.shape[1] != V:
                raise KernelError("sample: the seen table must be [slots, vocab]")
        if all_greedy and self.use_argmax_parts and R <= 16:    # (64 rows: 23 us against 12 us, one workgroup a row)
            if self._argmax_state is None or self._argmax_state[0].numel() < R:
                if self._argmax_state is not None:
                    self._retired.append(self._argmax_state)      # recorded graphs may still point at it
                self._argmax_state = (torch.zeros(max(R, 64), dtype=torch.int64, device=logits.device),
                                      torch.zeros(max(R, 64), dtype=torch.int32, device=logits.device))
            best, arrived = self._argmax_state
            code = self._lib("sampling").celeg_argmax_rows(
                _ptr(logits), _c_int(self._rows(logits, "logits")), _c_int(R), _c_int(V),
                _ptr(fparams), _ptr(iparams), _ptr(seen),
                _c_size_t(seen.stride(0) if seen is not None else 0), _ptr(out_tokens),
                _ptr(last_tokens), _ptr(best), _ptr(arrived), self._stream())
            self._check(code, "argmax of rows")
            return
        code = self._lib("sampling").celeg_sample(
            _ptr(logits), _c_int(self._rows(logits, "logits")), _c_int(R), _c_int(V),
            _ptr(fparams), _ptr(iparams), _ptr(seen),
            _c_size_t(seen.stride(0) if seen is not None else 0), _ptr(out_tokens),
            _ptr(last_tokens), self._stream())
        self._check(code, "sample")

    def mark_seen(self, seen, token_ids, token_slot, n):
        self._dev(seen, "seen", torch.uint8); self._dev(token_ids, "token_ids", torch.int32)
        self._dev(token_slot, "token_slot", torch.int32)
        if token_ids.numel() < n or token_slot.numel() < n:
            raise KernelError("mark_seen: fewer rows than n")
        code = self._lib("sampling").celeg_mark_seen(
            _ptr(seen), _c_size_t(seen.stride(0)), _c_int(seen.shape[0]), _c_int(seen.shape[1]),
            _ptr(token_ids), _ptr(token_slot), _c_int(n), self._stream())
        self._check(code, "mark_seen")

    # ------------------------------------------------------------------ fused skinny products
    has_fused_linear = True
    _EPILOGUES = {"store": 0, "store_f32": 1, "residual": 2, "swiglu": 3, "conv": 4}

    def fused_linear_ok(self, rows: int, *inner_sizes: int) -> bool:
        """Whether the fused skinny product takes ``rows`` rows and these inner sizes."""
        return 0 < rows <= 64 and all(k > 0 and k % 8 == 0 for k in inner_sizes)

    def residual_stat_blocks(self, rows: int, n: int, k: int) -> int:
        """How many partial sums of squares per row the "residual" epilogue of
        ``fused_linear`` leaves for these sizes (the rows ``stats_out`` needs)."""
        if self.rows_kernel_ok(rows, k):
            return int(self._lib("gemm_rows").celeg_gemm_rows_blocks(
                _c_int(rows), _c_int(n), _c_int(k), _c_int(self._EPILOGUES["residual"])))
        if rows <= 16 and self.use_sliced:
            return int(self._lib("gemv_slices").celeg_gemv_slices_blocks(
                _c_int(rows), _c_int(n), _c_int(k)))
        return (n + 15) // 16

    def rows_kernel_ok(self, rows: int, *inner_sizes: int) -> bool:
        """Whether bfloat16 products of ``rows`` rows with these inner sizes go to the kernel
        for 9 to 64 rows."""
        return self.use_rows_kernel and self.rows_kernel_min_rows <= rows <= 64 \
            and all(k % 32 == 0 for k in inner_sizes)

    @staticmethod
    def pack_weight(w: torch.Tensor) -> torch.Tensor:
        """``w`` [rows, K] as [K/32, rows, 32]: blocks of 32 k-values with the rows side by
        side inside a block, the layout in which the k-sliced products read whole runs of
        memory per load.  K must be a multiple of 32."""
        rows, K = w.shape
        if K % 32:
            raise KernelError("pack_weight: the inner size must be a multiple of 32")
        return w.reshape(rows, K // 32, 32).permute(1, 0, 2).contiguous()

    def stream_prepare(self, h, xb, stats):
        """The bfloat16 copy ``xb`` of the 32-bit stream ``h`` and its rows' sums of squares
        (``stats[:rows, 0]``)."""
        self._dev(h, "h", torch.float32, contiguous=False); self._dev(xb, "xb", torch.bfloat16, contiguous=False)
        self._dev(stats, "stats", torch.float32)
        rows, width = h.shape
        xb_rows, xb_width, ldx, xb_k8 = self._operand(xb, "xb")
        if xb_rows < rows or xb_width != width or stats.shape[0] < rows:
            raise KernelError("stream_prepare: shapes do not fit")
        code = self._lib("gemv_slices").celeg_stream_prepare(
            _ptr(h), _c_int(self._rows(h, "h")), _ptr(xb), _c_int(ldx), ctypes.c_longlong(xb_k8),
            _ptr(stats), _c_int(stats.stride(0)), _c_int(rows), _c_int(width), self._stream())
        self._check(code, "stream_prepare")

    def embed_stream(self, table, token_ids, out, xb, stats):
        """Embedding gather into the 32-bit stream ``out``, its bfloat16 copy ``xb`` and the
        rows' sums of squares (``stats[:rows, 0]``)."""
        self._dev(table, "table", torch.bfloat16); self._dev(token_ids, "token_ids", torch.int32)
        self._dev(out, "out", torch.float32); self._dev(xb, "xb", torch.bfloat16, contiguous=False)
        self._dev(stats, "stats", torch.float32)
        rows, width = out.shape
        xb_rows, xb_width, ldx, xb_k8 = self._operand(xb, "xb")
        if table.shape[1] != width or token_ids.numel() != rows or stats.shape[0] < rows \
                or (xb_rows, xb_width) != (rows, width):
            raise KernelError("embed_stream: shapes do not fit")
        code = self._lib("gemv_slices").celeg_embed_stream(
            _ptr(table), _ptr(token_ids), _ptr(out), _ptr(xb), _c_int(ldx), ctypes.c_longlong(xb_k8),
            _ptr(stats), _c_int(stats.stride(0)),
            _c_int(rows), _c_int(width), _c_int(table.shape[0]), self._stream())
        self._check(code, "embed_stream")

    def embed_stats(self, table, token_ids, out, stats):
        """Embedding gather that also leaves every row's sum of squares in ``stats[:rows, 0]``."""
        self._dev(table, "table", torch.bfloat16); self._dev(token_ids, "token_ids", torch.int32)
        self._dev(out, "out", torch.float32); self._dev(stats, "stats", torch.float32)
        rows, width = out.shape
        if table.shape[1] != width or token_ids.numel() != rows or stats.shape[0] < rows:
            raise KernelError("embed_stats: shapes do not fit")
        code = self._lib("gemv_fused").celeg_embed_stats(
            _ptr(table), _ptr(token_ids), _ptr(out), _ptr(stats), _c_int(stats.stride(0)),
            _c_int(rows), _c_int(width),
            _c_int(table.shape[0]), self._stream())
        self._check(code, "embed_stats")

    def fused_linear(self, a, w, out, *, epilogue="store", norm_weight=None, eps=0.0, stats=None,
                     stat_blocks=0, rows=None, bias=None, stats_out=None, conv=None, n_rows=None,
                     out_bf16=None):
        """out = epilogue(prologue(a) w^T) for up to 64 rows, bfloat16 weights.

        ``a``: bfloat16 rows [M, K], or, with ``norm_weight``, the 32-bit residual stream,
        normalised on the fly (``stats[row, :stat_blocks]`` holding partial sums of squares
        of its rows if ``stat_blocks`` > 0).  ``rows`` picks rows of ``a``.  Epilogues: "store"
        (bfloat16 [M, N]), "store_f32", "residual" (``out`` is the stream, [M, N] 32-bit,
        added to in place; ``stats_out`` [>= M, ``residual_stat_blocks``] receives partial
        sums of squares of the new rows, ``last_stat_blocks`` says how many a row), "swiglu" (``w`` is [2N, K]: gate rows then up rows), "conv"
        (``w`` is [3N, K]: B, C, x rows; ``conv`` = (taps [N, L], bias or None, state
        [slots, L, N], seq_slot [M]); one new token per request).

        Up to 16 bfloat16 rows go to the k-sliced kernels, and 9 to 64 rows with an inner size
        that is a multiple of 32 to the kernel that streams the weights.  Both also take the form behind a
        norm whose weight the caller has folded into ``w``: ``a`` is then the bfloat16 copy
        of the stream and ``stats[row, :stat_blocks]`` its partial sums of squares, from which
        the rows' 1/rms (with ``eps``) scales the sums; their "residual" epilogue refreshes
        ``out_bf16``, the bfloat16 copy of the stream, if given.  They also take ``w`` in the
        layout of ``pack_weight``."""
        if epilogue not in self._EPILOGUES:
            raise KernelError(f"fused_linear: unknown epilogue '{epilogue}'")
        self._dev(w, "w", torch.bfloat16)
        streams = {"swiglu": 2, "conv": 3}.get(epilogue, 1)
        packed = w.dim() == 3                  # [K/32, rows, 32], see pack_weight
        if packed and w.shape[2] != 32:
            raise KernelError("fused_linear: a packed weight is [K/32, rows, 32]")
        w_rows, K = (w.shape[1], w.shape[0] * 32) if packed else (w.shape[0], w.shape[1])
        if w_rows % streams:
            raise KernelError("fused_linear: weight rows do not split into the epilogue's streams")
        N = w_rows // streams
        M = n_rows if n_rows is not None else (rows.numel() if rows is not None else a.shape[0])
        if not self.fused_linear_ok(M, K):
            raise KernelError(f"fused_linear: {M} rows with inner size {K} are not supported "
                              "(1..64 rows, inner size a multiple of 8)")
        self._dev(a, "a", contiguous=False)
        a_rows, a_width, lda, a_k8 = self._operand(a, "a")
        if a_width != K or (rows is None and a_rows < M):
            raise KernelError("fused_linear: a does not fit the weights")
        if norm_weight is not None:
            if a.dtype != torch.float32:
                raise KernelError("fused_linear: the normalising prologue reads a 32-bit stream")
            self._dev(norm_weight, "norm_weight", torch.float32)
            if norm_weight.numel() != K:
                raise KernelError("fused_linear: norm weight must have the inner size")
            if epilogue == "residual":
                raise KernelError("fused_linear: this combination is not built")
        else:
            if a.dtype != torch.bfloat16:
                raise KernelError("fused_linear: rows must be bfloat16 (or 32-bit with a norm weight)")
            if (epilogue in ("swiglu", "conv") or stat_blocks > 0) \
                    and not (M <= 16 and self.use_sliced) and not self.rows_kernel_ok(M, K):
                raise KernelError("fused_linear: this combination is not built")
        if lda % 8:
            raise KernelError("fused_linear: the row stride of a must be a multiple of 8")
        if rows is not None:
            self._dev(rows, "rows", torch.int32)
        out_dtype = torch.float32 if epilogue in ("store_f32", "residual") else torch.bfloat16
        self._dev(out, "out", out_dtype, contiguous=False)
        out_rows, out_width, ldo, out_k8 = self._operand(out, "out")
        if out_rows < M or out_width != N:
            raise KernelError(f"fused_linear: out must be [{M}, {N}], got {tuple(out.shape)}")
        if bias is not None:
            self._dev(bias, "bias", torch.float32)
            if bias.numel() != streams * N:
                raise KernelError("fused_linear: bias does not fit")
        prm = _GemvParams()
        prm.a, prm.lda = a.data_ptr(), lda
        prm.rows = rows.data_ptr() if rows is not None else None
        prm.norm_w = norm_weight.data_ptr() if norm_weight is not None else None
        prm.eps = eps
        if stat_blocks > 0:
            self._dev(stats, "stats", torch.float32)
            if stats.shape[1] < stat_blocks:
                raise KernelError("fused_linear: fewer partial sums than stat_blocks")
            prm.stats, prm.n_stat_blocks, prm.stats_ld = stats.data_ptr(), stat_blocks, stats.stride(0)
        prm.w, prm.stream_rows = w.data_ptr(), N
        prm.bias = bias.data_ptr() if bias is not None else None
        prm.M, prm.N, prm.K = M, N, K
        prm.out, prm.ldo = out.data_ptr(), ldo
        streamed = norm_weight is None and self.rows_kernel_ok(M, K)
        sliced = norm_weight is None and not streamed and M <= 16 and self.use_sliced
        prm.a_k8_stride, prm.out_k8_stride, prm.w_q_stride = a_k8, out_k8, 8
        if (a.dim() == 3 or out.dim() == 3 or (out_bf16 is not None and out_bf16.dim() == 3)) \
                and not streamed:
            raise KernelError("fused_linear: operands with the rows side by side go with the kernel for 9 to 64 rows")
        if out.dim() == 3 and out_dtype != torch.bfloat16:
            raise KernelError("fused_linear: a 32-bit output has its rows one after the other")
        if packed and not (sliced or streamed):
            raise KernelError("fused_linear: packed weights go with bfloat16 rows")
        prm.w_row_stride, prm.w_kb_stride = (32, w_rows * 32) if packed else (K, 32)
        if out_bf16 is not None:
            if not ((sliced or streamed) and epilogue == "residual"):
                raise KernelError("fused_linear: out_bf16 goes with the residual epilogue of bfloat16 rows")
            self._dev(out_bf16, "out_bf16", torch.bfloat16, contiguous=False)
            b_rows, b_width, ld_bf16, bf16_k8 = self._operand(out_bf16, "out_bf16")
            if b_rows < M or b_width != N:
                raise KernelError("fused_linear: out_bf16 does not fit")
            prm.out_bf16, prm.ld_bf16, prm.bf16_k8_stride = out_bf16.data_ptr(), ld_bf16, bf16_k8
        if epilogue == "residual":
            # partial sums of squares: one per workgroup and row
            self.last_stat_blocks = self.residual_stat_blocks(M, N, K) if sliced or streamed \
                else (N + 15) // 16
        if epilogue == "residual" and stats_out is not None:
            self._dev(stats_out, "stats_out", torch.float32)
            if stats_out.shape[1] < self.last_stat_blocks or stats_out.shape[0] < M:
                raise KernelError(f"fused_linear: stats_out must be [>= rows, >= {self.last_stat_blocks}]")
            prm.stats_out, prm.stats_ld_out = stats_out.data_ptr(), stats_out.stride(0)
        if epilogue == "conv":
            taps_w, conv_bias, state, seq_slot = conv
            self._dev(taps_w, "conv taps", torch.float32); self._dev(seq_slot, "seq_slot", torch.int32)
            self._dev(state, "state", torch.float32, contiguous=False)
            L = taps_w.shape[1]
            if L > 8:
                raise KernelError(f"fused_linear: the convolution epilogue holds up to 8 taps, not {L}")
            if taps_w.shape[0] != N or state.shape[1:] != (L, N) or state.stride(1) != N \
                    or state.stride(2) != 1 or seq_slot.numel() < M:
                raise KernelError("fused_linear: convolution operands do not fit")
            prm.conv_w = taps_w.data_ptr()
            prm.conv_b = conv_bias.data_ptr() if conv_bias is not None else None
            prm.state, prm.state_slot_stride = state.data_ptr(), state.stride(0)
            prm.seq_slot, prm.taps = seq_slot.data_ptr(), L
        if sliced:
            code = self._lib("gemv_slices").celeg_gemv_slices(
                ctypes.byref(prm), _c_int(self._EPILOGUES[epilogue]), self._stream())
            self._check(code, f"fused_linear ({epilogue}, k-sliced)")
            return out
        if streamed:
            code = self._lib("gemm_rows").celeg_gemm_rows(
                ctypes.byref(prm), _c_int(self._EPILOGUES[epilogue]), self._stream())
            self._check(code, f"fused_linear ({epilogue}, 9 to 64 rows)")
            return out
        code = self._lib("gemv_fused").celeg_gemv_fused(
            ctypes.byref(prm), _c_int(1 if norm_weight is not None else 0),
            _c_int(self._EPILOGUES[epilogue]), _c_int(self.fused_linear_shape), self._stream())
        self._check(code, f"fused_linear ({epilogue})")
        return out

    # ------------------------------------------------------------------ fused products of many rows
    def tiled_linear_ok(self, rows: int, n: int, *inner_sizes: int) -> bool:
        """Whether the fused bfloat16 product for many rows takes these sizes."""
        return self.use_tiles and rows >= self.tiles_min_rows and n % 4 == 0 \
            and all(k > 0 and k % 64 == 0 for k in inner_sizes)

    def tiled_stat_blocks(self, rows: int, n: int, k: int) -> int:
        """Partial sums of squares per row that the "residual" epilogue of ``tiled_linear``
        leaves for these sizes."""
        return int(self._lib("gemm_tiles").celeg_gemm_tiles_blocks(_c_int(rows), _c_int(n), _c_int(k)))

    def tiled_linear(self, a, w, out, *, epilogue="store", eps=0.0, stats=None, stat_blocks=0,
                     bias=None, stats_out=None, out_bf16=None, qkv=None):
        """out = epilogue(scale * (a w^T) + bias) for many bfloat16 rows (any number; made for
        more than 64), inner size a multiple of 64, columns a multiple of 4.

        ``a`` [M, K] bfloat16 with dense rows.  With ``stat_blocks`` > 0, ``a`` is the bfloat16
        copy of the residual stream behind a norm whose weight the caller has folded into
        ``w``, and ``stats[row, :stat_blocks]`` are partial sums of squares of its rows, from
        which the rows' 1/rms (with ``eps``) scales the sums.  Epilogues: "store" (bfloat16
        [M, N]), "residual" (``out`` is the 32-bit stream, added to in place; ``out_bf16``
        receives its bfloat16 copy and ``stats_out`` [>= M, ``tiled_stat_blocks``] the partial
        sums of squares of the new rows; ``last_stat_blocks`` says how many a row), "swiglu"
        (``w`` is [2N, K]: gate rows then up rows).

        ``qkv`` (with "store"): a dict ``heads, kv_heads, q_weight, k_weight, eps, cos_sin
        ([positions, 32, 2] 32-bit or None), batch, kv``: the columns are heads of 64; query heads
        are normalised, turned and stored to ``out``, key heads likewise and stored to their rows'
        pages, value heads stored to the pages (what ``qk_norm_rope_store`` does behind a product)."""
        if epilogue not in ("store", "residual", "swiglu"):
            raise KernelError(f"tiled_linear: unknown epilogue '{epilogue}'")
        self._dev(a, "a", torch.bfloat16, contiguous=False); self._dev(w, "w", torch.bfloat16)
        streams = 2 if epilogue == "swiglu" else 1
        if a.dim() != 2 or w.dim() != 2:
            raise KernelError("tiled_linear: a and w must be 2-D")
        M, K = a.shape
        if w.shape[1] != K or w.shape[0] % streams:
            raise KernelError(f"tiled_linear: a {tuple(a.shape)} and w {tuple(w.shape)} do not fit")
        N = w.shape[0] // streams
        if K % 64 or N % 4:
            raise KernelError(f"tiled_linear: inner size {K} must be a multiple of 64 and {N} columns "
                              "a multiple of 4")
        lda = self._rows(a, "a")
        out_dtype = torch.float32 if epilogue == "residual" else torch.bfloat16
        self._dev(out, "out", out_dtype, contiguous=False)
        ldo = self._rows(out, "out")
        if out.shape != (M, N) or lda % 8 or ldo % 4 or a.data_ptr() % 16 or w.data_ptr() % 16 \
                or out.data_ptr() % 16:
            raise KernelError(f"tiled_linear: out must be [{M}, {N}] and the rows aligned")
        prm = _TileParams()
        prm.a, prm.lda, prm.w, prm.ldw, prm.stream_rows = a.data_ptr(), lda, w.data_ptr(), K, N
        if bias is not None:
            self._dev(bias, "bias", torch.float32)
            if bias.numel() != streams * N:
                raise KernelError("tiled_linear: bias does not fit")
            prm.bias = bias.data_ptr()
        if stat_blocks > 0:
            self._dev(stats, "stats", torch.float32)
            if stats.dim() != 2 or stats.shape[0] < M or stats.shape[1] < stat_blocks or stats.stride(1) != 1:
                raise KernelError("tiled_linear: stats must be [>= rows, >= stat_blocks]")
            prm.stats, prm.n_stat_blocks, prm.stats_ld = stats.data_ptr(), stat_blocks, stats.stride(0)
        prm.eps = eps
        prm.M, prm.N, prm.K = M, N, K
        prm.out, prm.ldo = out.data_ptr(), ldo
        code = {"store": 0, "residual": 2, "swiglu": 3}[epilogue]
        if qkv is not None:
            if epilogue != "store":
                raise KernelError("tiled_linear: the q/k/v tail goes with the store epilogue")
            kv, batch = qkv["kv"], qkv["batch"]
            self._check_kv(kv, qkv["kv_heads"], 64, torch.bfloat16)
            if N != (qkv["heads"] + 2 * qkv["kv_heads"]) * 64 or M != batch.n_tokens:
                raise KernelError("tiled_linear: the q/k/v tail needs all heads of every row of the step")
            prm.positions, prm.token_slot = _ptr(batch.positions).value, _ptr(batch.token_slot).value
            prm.table, prm.table_stride = kv.table.data_ptr(), kv.table.stride(0)
            prm.k_pool, prm.v_pool = kv.k.data_ptr(), kv.v.data_ptr()
            prm.n_layers, prm.layer, prm.page_tokens = kv.n_layers, kv.layer, kv.page_tokens
            prm.q_heads, prm.kv_heads = qkv["heads"], qkv["kv_heads"]
            for name in ("q_weight", "k_weight", "cos_sin"):
                t = qkv.get(name)
                if t is not None:
                    self._dev(t, name, torch.float32)
                    setattr(prm, name, t.data_ptr())
            prm.qk_eps = qkv.get("eps", 0.0)
            code = 5
        if epilogue == "residual":
            self.last_stat_blocks = self.tiled_stat_blocks(M, N, K)
            if out_bf16 is not None:
                self._dev(out_bf16, "out_bf16", torch.bfloat16, contiguous=False)
                ldb = self._rows(out_bf16, "out_bf16")
                if out_bf16.shape != (M, N) or ldb % 4 or out_bf16.data_ptr() % 8:
                    raise KernelError("tiled_linear: out_bf16 does not fit")
                prm.out_bf16, prm.ld_bf16 = out_bf16.data_ptr(), ldb
            if stats_out is not None:
                self._dev(stats_out, "stats_out", torch.float32)
                if stats_out.dim() != 2 or stats_out.shape[0] < M or stats_out.shape[1] < self.last_stat_blocks \
                        or stats_out.stride(1) != 1:
                    raise KernelError(f"tiled_linear: stats_out must be [>= rows, >= {self.last_stat_blocks}]")
                prm.stats_out, prm.stats_ld_out = stats_out.data_ptr(), stats_out.stride(0)
        elif out_bf16 is not None or stats_out is not None:
            raise KernelError("tiled_linear: out_bf16 and stats_out go with the residual epilogue")
        status = self._lib("gemm_tiles").celeg_gemm_tiles(ctypes.byref(prm), _c_int(code), self._stream())
        self._check(status, f"tiled_linear ({epilogue})")
        return out


class _TileParams(ctypes.Structure):
    """Mirror of ``TileParams`` in gemm_tiles.hip (its size is checked when the library loads)."""
    _fields_ = [
        ("a", ctypes.c_void_p), ("lda", ctypes.c_int), ("w", ctypes.c_void_p), ("ldw", ctypes.c_int),
        ("stream_rows", ctypes.c_int), ("bias", ctypes.c_void_p), ("stats", ctypes.c_void_p),
        ("n_stat_blocks", ctypes.c_int), ("stats_ld", ctypes.c_int), ("eps", ctypes.c_float),
        ("M", ctypes.c_int), ("N", ctypes.c_int), ("K", ctypes.c_int),
        ("out", ctypes.c_void_p), ("ldo", ctypes.c_int), ("out_bf16", ctypes.c_void_p),
        ("ld_bf16", ctypes.c_int), ("stats_out", ctypes.c_void_p), ("stats_ld_out", ctypes.c_int),
        ("positions", ctypes.c_void_p), ("token_slot", ctypes.c_void_p), ("table", ctypes.c_void_p),
        ("table_stride", ctypes.c_int), ("k_pool", ctypes.c_void_p), ("v_pool", ctypes.c_void_p),
        ("n_layers", ctypes.c_int), ("layer", ctypes.c_int), ("page_tokens", ctypes.c_int),
        ("q_heads", ctypes.c_int), ("kv_heads", ctypes.c_int), ("q_weight", ctypes.c_void_p),
        ("k_weight", ctypes.c_void_p), ("qk_eps", ctypes.c_float), ("cos_sin", ctypes.c_void_p),
    ]


class _GemvParams(ctypes.Structure):
    """Mirror of ``GemvParams`` in gemv_params.h (its size is checked when the library loads)."""
    _fields_ = [
        ("a", ctypes.c_void_p), ("lda", ctypes.c_int), ("rows", ctypes.c_void_p),
        ("norm_w", ctypes.c_void_p), ("eps", ctypes.c_float), ("stats", ctypes.c_void_p),
        ("n_stat_blocks", ctypes.c_int), ("stats_ld", ctypes.c_int),
        ("w", ctypes.c_void_p), ("stream_rows", ctypes.c_int), ("bias", ctypes.c_void_p),
        ("M", ctypes.c_int), ("N", ctypes.c_int), ("K", ctypes.c_int),
        ("out", ctypes.c_void_p), ("ldo", ctypes.c_int), ("stats_out", ctypes.c_void_p),
        ("stats_ld_out", ctypes.c_int),
        ("conv_w", ctypes.c_void_p), ("conv_b", ctypes.c_void_p), ("state", ctypes.c_void_p),
        ("state_slot_stride", ctypes.c_size_t), ("seq_slot", ctypes.c_void_p), ("taps", ctypes.c_int),
        ("out_bf16", ctypes.c_void_p), ("ld_bf16", ctypes.c_int),
        ("w_row_stride", ctypes.c_longlong), ("w_kb_stride", ctypes.c_longlong),
        ("a_k8_stride", ctypes.c_longlong), ("out_k8_stride", ctypes.c_longlong),
        ("bf16_k8_stride", ctypes.c_longlong), ("w_q_stride", ctypes.c_longlong),
    ]

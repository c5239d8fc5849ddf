"""The library, loaded: ``ctypes`` signatures of the C interface (``csrc/include/celeg_amd.h``)
and thin Python objects over its handles.

Everything between a request's tokens and its next token happens inside the library; Python
packs arguments and unpacks results.  The library is built at first need (``csrc/build.py``);
if it cannot be built or loaded, importing this module fails loudly: there is no other path.
"""
from __future__ import annotations

import ctypes
import json
from typing import Any, Dict, List, Optional, Sequence

import numpy as np

from .csrc import build

c_int, c_int32, c_int64, c_float = ctypes.c_int, ctypes.c_int32, ctypes.c_int64, ctypes.c_float
c_char_p, c_void_p, c_size_t = ctypes.c_char_p, ctypes.c_void_p, ctypes.c_size_t
P = ctypes.POINTER

STATUS_NAMES = ["queued", "prefill", "decoding", "finished", "cancelled", "failed"]
OK, ERROR, INVALID_ARGUMENT, NOT_FOUND = 0, 1, 2, 3


class NativeError(RuntimeError):
    """A failure inside the library (a kernel, a page, a step)."""


class NativeArgumentError(ValueError):
    """The library refused an argument or a configuration."""


class GenerationOptions(ctypes.Structure):
    _fields_ = [("struct_size", c_size_t), ("temperature", c_float), ("top_k", c_int32), ("top_p", c_float),
                ("repetition_penalty", c_float), ("seed", ctypes.c_uint64),
                ("forced_prefix", P(c_int32)), ("n_forced_prefix", c_int32)]


class SessionMetrics(ctypes.Structure):
    _fields_ = [("struct_size", c_size_t), ("prefill_ms", ctypes.c_double), ("prefill_tokens", ctypes.c_uint64),
                ("decode_ms", ctypes.c_double), ("decode_tokens", ctypes.c_uint64)]


class EngineOptions(ctypes.Structure):
    _fields_ = [("struct_size", c_size_t), ("dtype", c_char_p), ("device", c_int32),
                ("max_active_requests", c_int32), ("max_batched_tokens", c_int32),
                ("prefill_chunk_tokens", c_int32), ("page_tokens", c_int32), ("logical_kv_pages", c_int32),
                ("scheduler_policy", c_int32), ("context", c_int32), ("gemm_backend", c_int32),
                ("use_graphs", c_int32), ("run_ahead", c_int32), ("portion_granule", c_int32),
                ("strict_weights", c_int32)]


class RequestOptionsStruct(ctypes.Structure):
    _fields_ = [("struct_size", c_size_t), ("max_new_tokens", c_int32), ("eos_token_ids", P(c_int32)),
                ("n_eos_token_ids", c_int32), ("priority", c_int32), ("generation", GenerationOptions)]


class TensorView(ctypes.Structure):
    _fields_ = [("data", c_void_p), ("dtype", c_int32), ("ndim", c_int32), ("shape", c_int64 * 4),
                ("stride", c_int64 * 4)]


class StepView(ctypes.Structure):
    _fields_ = [("n_tokens", c_int32), ("n_seqs", c_int32), ("n_logit_rows", c_int32), ("decode_only", c_int32),
                ("single_rows", c_int32)] + \
               [(name, c_void_p) for name in ("token_ids", "positions", "token_seq", "token_slot", "cu_seqlens",
                                              "seq_slot", "seq_start", "logit_rows")] + \
               [(name, P(c_int32)) for name in ("host_seq_slot", "host_seq_start", "host_cu_seqlens")]


class CacheView(ctypes.Structure):
    _fields_ = [("has_kv", c_int32), ("writes_kv", c_int32), ("k", c_void_p), ("v", c_void_p), ("kv_dtype", c_int32),
                ("layer", c_int32), ("n_layers", c_int32), ("page_tokens", c_int32), ("kv_heads", c_int32),
                ("head_dim", c_int32), ("table_stride", c_int32), ("table", c_void_p), ("n_states", c_int32),
                ("state_names", P(c_char_p)), ("states", P(TensorView)), ("v_head_dim", c_int32), ("n_pages", c_int32)]


class ForwardArgs(ctypes.Structure):
    _fields_ = [("x", TensorView), ("out", TensorView), ("delta", TensorView), ("rows", c_void_p),
                ("token_ids", c_void_p), ("step", StepView), ("cache", CacheView), ("stream", c_void_p),
                ("dtype", c_int32)]


DESCRIBE_FN = ctypes.CFUNCTYPE(c_void_p, c_void_p)
LOAD_FN = ctypes.CFUNCTYPE(c_int32, c_void_p, c_int32, P(c_char_p), P(TensorView))
FORWARD_FN = ctypes.CFUNCTYPE(c_int32, c_void_p, P(ForwardArgs))
DESTROY_FN = ctypes.CFUNCTYPE(None, c_void_p)


class PartFunctions(ctypes.Structure):
    _fields_ = [("self", c_void_p), ("describe", DESCRIBE_FN), ("load", LOAD_FN), ("forward", FORWARD_FN),
                ("destroy", DESTROY_FN)]


PART_FACTORY_FN = ctypes.CFUNCTYPE(c_int32, c_char_p, c_void_p, P(PartFunctions))
ARCH_DESCRIBE_FN = ctypes.CFUNCTYPE(c_void_p, c_char_p, c_char_p, c_void_p)

_lib: Optional[ctypes.CDLL] = None


def library_path() -> str:
    return build.ensure_built()


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    try:
        L = ctypes.CDLL(path)
    except OSError as err:
        raise NativeError(f"cannot load the built library {path}: {err}") from err

    def sig(name, restype, *argtypes):
        fn = getattr(L, name)
        fn.restype, fn.argtypes = restype, list(argtypes)

    sig("celeg_last_error", c_char_p)
    sig("celeg_version", c_char_p)
    sig("celeg_backend_capabilities", c_char_p)
    sig("celeg_generation_options_init", None, P(GenerationOptions), c_size_t)
    sig("celeg_engine_options_init", None, P(EngineOptions), c_size_t)
    sig("celeg_request_options_init", None, P(RequestOptionsStruct), c_size_t)
    sig("celeg_engine_create", c_int, c_char_p, P(EngineOptions), P(c_void_p))
    sig("celeg_engine_destroy", None, c_void_p)
    sig("celeg_engine_submit", c_int, c_void_p, P(c_int32), c_int32, P(RequestOptionsStruct), P(c_int64))
    sig("celeg_engine_step", c_int, c_void_p, P(c_int32))
    sig("celeg_engine_run", c_int, c_void_p)
    sig("celeg_engine_run_steps", c_int, c_void_p, c_int64, P(c_int64))
    sig("celeg_engine_has_work", c_int, c_void_p, P(c_int32))
    sig("celeg_engine_poll", c_int, c_void_p, c_int64, P(c_int32), c_int32, P(c_int32), P(c_int32))
    sig("celeg_engine_status", c_int, c_void_p, c_int64, P(c_int32))
    sig("celeg_engine_cancel", c_int, c_void_p, c_int64)
    sig("celeg_engine_release", c_int, c_void_p, c_int64)
    sig("celeg_engine_request_error", c_char_p, c_void_p, c_int64)
    sig("celeg_engine_last_error", c_char_p, c_void_p)
    sig("celeg_engine_metrics", c_char_p, c_void_p)
    sig("celeg_engine_request_metrics", c_char_p, c_void_p, c_int64)
    sig("celeg_engine_last_logits", c_int, c_void_p, P(c_float), c_size_t, P(c_int32), P(c_int32))
    sig("celeg_engine_model", c_void_p, c_void_p)
    sig("celeg_model_create", c_int, c_char_p, P(EngineOptions), P(c_void_p))
    sig("celeg_model_destroy", None, c_void_p)
    sig("celeg_model_describe", c_char_p, c_void_p)
    sig("celeg_model_open_slot", c_int, c_void_p, P(c_int32))
    sig("celeg_model_close_slot", c_int, c_void_p, c_int32)
    sig("celeg_model_prepare", c_int, c_void_p, c_int32, c_int32, c_int32, P(c_int32))
    sig("celeg_model_check_cache", c_int, c_void_p)
    sig("celeg_model_cache_state", c_char_p, c_void_p)
    sig("celeg_model_step", c_int, c_void_p, c_int32, P(c_int32), P(c_int32), P(c_int32), P(c_int32), P(c_int32),
        P(c_int32), c_void_p, c_size_t)
    sig("celeg_model_set_knob", c_int, c_void_p, c_char_p, c_int32)
    sig("celeg_model_knobs", c_char_p, c_void_p)
    sig("celeg_model_stream", c_void_p, c_void_p)
    sig("celeg_model_synchronize", c_int, c_void_p)
    sig("celeg_model_set_generation", c_int, c_void_p, P(GenerationOptions))
    sig("celeg_model_prefill", c_int, c_void_p, P(c_int32), c_size_t)
    sig("celeg_model_decode", c_int, c_void_p, P(c_int32))
    sig("celeg_model_copy_logits", c_int, c_void_p, P(c_float), c_size_t, P(c_size_t))
    sig("celeg_model_get_metrics", c_int, c_void_p, P(SessionMetrics))
    sig("celeg_model_time_phases", c_int, c_void_p, c_int32)
    sig("celeg_model_phase_times", c_char_p, c_void_p)
    sig("celeg_describe_folder", c_char_p, c_char_p)
    sig("celeg_describe_config", c_char_p, c_char_p, c_char_p)
    sig("celeg_check_folder", c_int, c_char_p)
    sig("celeg_check_folder_strict", c_int, c_char_p, c_int32)
    sig("celeg_registered", c_char_p, c_char_p)
    sig("celeg_host_new", ctypes.c_longlong, c_char_p, c_char_p)
    sig("celeg_host_call", c_char_p, ctypes.c_longlong, c_char_p, c_char_p)
    sig("celeg_host_delete", None, ctypes.c_longlong)
    sig("celeg_register_part", c_int, c_char_p, c_char_p, PART_FACTORY_FN, c_void_p)
    sig("celeg_register_architecture", c_int, c_char_p, ARCH_DESCRIBE_FN, c_void_p)
    _lib = L
    return L


def last_error() -> str:
    return (lib().celeg_last_error() or b"").decode("utf-8", "replace")


def check(status: int) -> None:
    if status == OK:
        return
    message = last_error()
    if status in (INVALID_ARGUMENT, NOT_FOUND):
        raise NativeArgumentError(message)
    raise NativeError(message)


def _text(raw) -> str:
    if raw is None:
        message = last_error()
        raise NativeArgumentError(message)
    return raw.decode("utf-8")


def _ints(values: Sequence[int]):
    array = (c_int32 * max(len(values), 1))(*values)
    return array


# ------------------------------------------------------------------ descriptions
def backend_capabilities() -> str:
    """What this build can run and on what, in a sentence."""
    return _text(lib().celeg_backend_capabilities())


def describe_folder(model_dir: str) -> Dict[str, Any]:
    return json.loads(_text(lib().celeg_describe_folder(model_dir.encode())))


def describe_config(config: Dict[str, Any], tensor_shapes: Optional[Dict[str, Sequence[int]]] = None) -> Dict[str, Any]:
    shapes = None if tensor_shapes is None else json.dumps({k: list(v) for k, v in tensor_shapes.items()}).encode()
    return json.loads(_text(lib().celeg_describe_config(json.dumps(config).encode(), shapes)))


def check_folder(model_dir: str, strict: bool = False) -> None:
    check(lib().celeg_check_folder_strict(model_dir.encode(), int(bool(strict))))


def registered(what: str) -> List[str]:
    return json.loads(_text(lib().celeg_registered(what.encode())))


# ------------------------------------------------------------------ options
def engine_options(*, dtype="bfloat16", device=0, max_active_requests=8, max_batched_tokens=2048,
                   prefill_chunk_tokens=1024, page_tokens=16, n_pages=None, policy="max_utilization",
                   context=None, gemm_backend="auto", use_graphs=True, run_ahead=True,
                   portion_granule=1, strict_weights=False) -> EngineOptions:
    if policy not in ("max_utilization", "guaranteed_no_evict"):
        raise NativeArgumentError("policy must be max_utilization or guaranteed_no_evict")
    if gemm_backend not in ("library", "tiles", "auto"):
        raise NativeArgumentError(f"gemm_backend must be 'library', 'tiles' or 'auto', not '{gemm_backend}'")
    o = EngineOptions()
    lib().celeg_engine_options_init(ctypes.byref(o), ctypes.sizeof(o))
    o.dtype = str(dtype).replace("torch.", "").encode()
    o.device = int(device)
    o.max_active_requests, o.max_batched_tokens = int(max_active_requests), int(max_batched_tokens)
    o.prefill_chunk_tokens, o.page_tokens = int(prefill_chunk_tokens), int(page_tokens)
    o.logical_kv_pages = int(n_pages) if n_pages else 0
    o.scheduler_policy = 1 if policy == "guaranteed_no_evict" else 0
    o.context = int(context) if context else 0
    o.gemm_backend = {"library": 0, "tiles": 1, "auto": 2}[gemm_backend]
    o.use_graphs, o.run_ahead, o.portion_granule = int(bool(use_graphs)), int(bool(run_ahead)), int(portion_granule)
    o.strict_weights = int(bool(strict_weights))
    return o


def device_index(device) -> int:
    text = str(device)
    if text in ("cuda", "gpu"):
        return 0
    if text.startswith("cuda:"):
        return int(text[5:])
    if text.isdigit():
        return int(text)
    raise NativeArgumentError(f"celeg_amd runs on a GPU only, not on '{device}'")


# ------------------------------------------------------------------ the step function alone
class NativeModel:
    """A loaded model with its cache manager and runner (``celeg_model``)."""

    def __init__(self, handle: int, owner=None):
        self.handle = c_void_p(handle)
        self._owner = owner          # an engine that owns the handle, kept alive
        self._owned = owner is None
        self.info = json.loads(_text(lib().celeg_model_describe(self.handle)))
        self.logit_width = int(self.info["logit_width"])

    @classmethod
    def load(cls, model_dir: str, options: EngineOptions) -> "NativeModel":
        handle = c_void_p()
        check(lib().celeg_model_create(model_dir.encode(), ctypes.byref(options), ctypes.byref(handle)))
        return cls(handle.value)

    def close(self) -> None:
        if self._owned and self.handle:
            lib().celeg_model_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def open_slot(self) -> Optional[int]:
        slot = c_int32()
        check(lib().celeg_model_open_slot(self.handle, ctypes.byref(slot)))
        return None if slot.value < 0 else slot.value

    def close_slot(self, slot: int) -> None:
        check(lib().celeg_model_close_slot(self.handle, slot))

    def prepare(self, slot: int, start: int, n: int) -> bool:
        ok = c_int32()
        check(lib().celeg_model_prepare(self.handle, slot, start, n, ctypes.byref(ok)))
        return bool(ok.value)

    def check_cache(self) -> None:
        check(lib().celeg_model_check_cache(self.handle))

    def cache_state(self) -> Dict[str, Any]:
        return json.loads(_text(lib().celeg_model_cache_state(self.handle)))

    def step(self, entries) -> np.ndarray:
        """``entries``: objects with slot, start_pos, tokens, want.  Returns float32
        [wanted, logit width]."""
        slots = _ints([int(e.slot) for e in entries])
        starts = _ints([int(e.start_pos) for e in entries])
        counts = _ints([len(e.tokens) for e in entries])
        tokens = _ints([int(t) for e in entries for t in e.tokens])
        n_want = _ints([len(e.want) for e in entries])
        want = _ints([int(w) for e in entries for w in e.want])
        wanted = sum(len(e.want) for e in entries)
        out = np.empty((wanted, self.logit_width), dtype=np.float32)
        check(lib().celeg_model_step(self.handle, len(entries), slots, starts, counts, tokens, n_want, want,
                                     out.ctypes.data_as(c_void_p), out.size))
        return out

    def set_knob(self, name: str, value) -> None:
        check(lib().celeg_model_set_knob(self.handle, name.encode(), int(value)))

    def knobs(self) -> Dict[str, int]:
        return json.loads(_text(lib().celeg_model_knobs(self.handle)))

    def synchronize(self) -> None:
        check(lib().celeg_model_synchronize(self.handle))

    # ---- one request at a time (celeg_model_prefill / decode / copy_logits / get_metrics)
    def set_generation(self, *, temperature=0.1, top_k=50, top_p=1.0, repetition_penalty=1.05, seed=1,
                       forced_prefix=()) -> None:
        g = GenerationOptions()
        lib().celeg_generation_options_init(ctypes.byref(g), ctypes.sizeof(g))
        g.temperature, g.top_k, g.top_p = float(temperature), int(top_k), float(top_p)
        g.repetition_penalty, g.seed = float(repetition_penalty), int(seed)
        forced = None
        if forced_prefix:
            forced = _ints([int(t) for t in forced_prefix])        # (kept alive until the call has copied it)
            g.forced_prefix = ctypes.cast(forced, P(c_int32))
            g.n_forced_prefix = len(forced_prefix)
        check(lib().celeg_model_set_generation(self.handle, ctypes.byref(g)))

    def prefill(self, tokens: Sequence[int]) -> None:
        """Starts a new sequence with this prompt (the model's earlier one is given back)."""
        toks = [int(t) for t in tokens]
        check(lib().celeg_model_prefill(self.handle, _ints(toks), len(toks)))

    def decode(self) -> int:
        """Chooses the next token from the last step's logits, feeds it, returns it."""
        token = c_int32()
        check(lib().celeg_model_decode(self.handle, ctypes.byref(token)))
        return token.value

    def copy_logits(self) -> np.ndarray:
        """The logits the next ``decode`` chooses from."""
        out = np.empty(self.logit_width, dtype=np.float32)
        required = c_size_t()
        check(lib().celeg_model_copy_logits(self.handle, out.ctypes.data_as(P(c_float)), out.size, ctypes.byref(required)))
        return out[:required.value]

    def session_metrics(self) -> Dict[str, float]:
        m = SessionMetrics()
        m.struct_size = ctypes.sizeof(m)
        check(lib().celeg_model_get_metrics(self.handle, ctypes.byref(m)))
        return {"prefill_ms": m.prefill_ms, "prefill_tokens": int(m.prefill_tokens), "decode_ms": m.decode_ms,
                "decode_tokens": int(m.decode_tokens)}

    def time_phases(self, on: bool = True) -> None:
        """Time every step's phases with events (such steps are not replayed from graphs)."""
        check(lib().celeg_model_time_phases(self.handle, int(bool(on))))

    def phase_times(self):
        """{"steps", "tokens", "phases": {name: {"ms", "calls"}}}, or None when nothing is timed."""
        return json.loads(_text(lib().celeg_model_phase_times(self.handle)))

    @property
    def stream(self) -> int:
        return lib().celeg_model_stream(self.handle) or 0


# ------------------------------------------------------------------ the engine
class NativeEngine:
    def __init__(self, model_dir: str, options: EngineOptions):
        handle = c_void_p()
        check(lib().celeg_engine_create(model_dir.encode(), ctypes.byref(options), ctypes.byref(handle)))
        self.handle = handle
        self.model = NativeModel(lib().celeg_engine_model(self.handle), owner=self)

    def close(self) -> None:
        if self.handle:
            self.model.handle = None
            lib().celeg_engine_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def submit(self, tokens: Sequence[int], *, max_new_tokens=128, eos_token_ids=None, priority=0,
               temperature=0.1, top_k=50, top_p=1.0, repetition_penalty=1.05, seed=1, forced_prefix=()) -> int:
        o = RequestOptionsStruct()
        lib().celeg_request_options_init(ctypes.byref(o), ctypes.sizeof(o))
        o.max_new_tokens, o.priority = int(max_new_tokens), int(priority)
        keep = None
        if eos_token_ids is not None:
            keep = _ints([int(t) for t in eos_token_ids])
            o.eos_token_ids = ctypes.cast(keep, P(c_int32))
            o.n_eos_token_ids = len(eos_token_ids)
        g = o.generation
        g.temperature, g.top_k, g.top_p = float(temperature), int(top_k), float(top_p)
        g.repetition_penalty = float(repetition_penalty)
        if not 0 <= int(seed) < (1 << 64):
            raise NativeArgumentError("seed must be non-zero")
        g.seed = int(seed)
        forced = None
        if forced_prefix:
            forced = _ints([int(t) for t in forced_prefix])        # (kept alive until the call has copied it)
            g.forced_prefix = ctypes.cast(forced, P(c_int32))
            g.n_forced_prefix = len(forced_prefix)
        request_id = c_int64()
        toks = [int(t) for t in tokens]
        check(lib().celeg_engine_submit(self.handle, _ints(toks), len(toks), ctypes.byref(o), ctypes.byref(request_id)))
        return request_id.value

    def step(self) -> int:
        fed = c_int32()
        check(lib().celeg_engine_step(self.handle, ctypes.byref(fed)))
        return fed.value

    def run(self) -> None:
        check(lib().celeg_engine_run(self.handle))

    def run_steps(self, limit: int) -> int:
        done = c_int64()
        check(lib().celeg_engine_run_steps(self.handle, int(limit), ctypes.byref(done)))
        return done.value

    def has_work(self) -> bool:
        flag = c_int32()
        check(lib().celeg_engine_has_work(self.handle, ctypes.byref(flag)))
        return bool(flag.value)

    def poll(self, request_id: int, capacity: int = 4096):
        """(status name, tokens generated since the last poll, error message)."""
        buf = (c_int32 * capacity)()
        tokens: List[int] = []
        while True:
            n, status = c_int32(), c_int32()
            check(lib().celeg_engine_poll(self.handle, request_id, buf, capacity, ctypes.byref(n), ctypes.byref(status)))
            tokens.extend(buf[:n.value])
            if n.value < capacity:
                break
        error = (lib().celeg_engine_request_error(self.handle, request_id) or b"").decode("utf-8", "replace")
        return STATUS_NAMES[status.value], tokens, error

    def status(self, request_id: int) -> str:
        status = c_int32()
        check(lib().celeg_engine_status(self.handle, request_id, ctypes.byref(status)))
        return STATUS_NAMES[status.value]

    def cancel(self, request_id: int) -> None:
        check(lib().celeg_engine_cancel(self.handle, request_id))

    def release(self, request_id: int) -> None:
        check(lib().celeg_engine_release(self.handle, request_id))

    def metrics(self) -> Dict[str, Any]:
        return json.loads(_text(lib().celeg_engine_metrics(self.handle)))

    def request_metrics(self, request_id: int) -> Dict[str, Any]:
        return json.loads(_text(lib().celeg_engine_request_metrics(self.handle, request_id)))

    def last_logits(self) -> np.ndarray:
        rows, vocab = c_int32(), c_int32()
        check(lib().celeg_engine_last_logits(self.handle, None, 0, ctypes.byref(rows), ctypes.byref(vocab)))
        out = np.empty((rows.value, vocab.value), dtype=np.float32)
        if out.size:
            check(lib().celeg_engine_last_logits(self.handle, out.ctypes.data_as(P(c_float)), out.size,
                                                 ctypes.byref(rows), ctypes.byref(vocab)))
        return out


# ------------------------------------------------------------------ host-side objects, without a GPU
class HostError(RuntimeError):
    """``kind`` is the library's kind of error: PageError, ConfigError, StepError, Error."""

    def __init__(self, message: str):
        kind, _, text = message.partition(": ")
        super().__init__(text if text else message)
        self.kind = kind if text else "Error"


class HostObject:
    def __init__(self, kind: str, **args):
        self.kind = kind
        self.handle = lib().celeg_host_new(kind.encode(), json.dumps(args).encode())
        if not self.handle:
            raise HostError(last_error())

    def call(self, method: str, *args):
        raw = lib().celeg_host_call(self.handle, method.encode(), json.dumps(list(args)).encode())
        if raw is None:
            raise HostError(last_error())
        return json.loads(raw.decode("utf-8"))

    def __del__(self):
        try:
            if self.handle:
                lib().celeg_host_delete(self.handle)
        except Exception:
            pass


# ------------------------------------------------------------------ parts and architectures from Python
_keep_alive: List[Any] = []      # callbacks the library holds pointers to


def register_architecture(name: str, describe) -> None:
    """``describe(config: dict, tensor_shapes: dict or None) -> {"config": dict, "spec": dict}``."""
    holder: Dict[str, Any] = {}

    def call(config_json, shapes_json, _user):
        try:
            shapes = json.loads(shapes_json.decode())
            result = describe(json.loads(config_json.decode()), shapes)
        except Exception as err:            # handed to the library as the refusal's reason
            result = {"error": f"{type(err).__name__}: {err}"}
        holder["text"] = ctypes.create_string_buffer(json.dumps(result).encode())
        return ctypes.addressof(holder["text"])

    fn = ARCH_DESCRIBE_FN(call)
    _keep_alive.extend([fn, holder])
    check(lib().celeg_register_architecture(name.encode(), fn, None))


def register_part(role: str, kind: str, factory) -> None:
    """``factory(spec: dict)`` builds an object with ``describe() -> dict`` (see
    ``celeg_part_functions`` in the header), optionally ``load(tensors: {role: TensorView})``, and
    ``forward(args: ForwardArgs)``.  Exceptions inside them are reported as failures of the step."""
    parts: Dict[int, Any] = {}

    def make(spec_json, _user, out):
        try:
            part = factory(json.loads(spec_json.decode()))
        except Exception as err:
            import traceback
            traceback.print_exc()
            return 1
        key = len(parts) + 1
        state = {"part": part}
        parts[key] = state

        def describe(_self):
            state["text"] = ctypes.create_string_buffer(json.dumps(part.describe()).encode())
            return ctypes.addressof(state["text"])

        def load(_self, n, roles, tensors):
            try:
                if hasattr(part, "load"):
                    part.load({roles[i].decode(): _copy_view(tensors[i]) for i in range(n)})
                return 0
            except Exception:
                import traceback
                traceback.print_exc()
                return 1

        def forward(_self, args):
            try:
                part.forward(args.contents)
                return 0
            except Exception:
                import traceback
                traceback.print_exc()
                return 1

        def destroy(_self):
            parts.pop(key, None)

        fns = (DESCRIBE_FN(describe), LOAD_FN(load), FORWARD_FN(forward), DESTROY_FN(destroy))
        state["fns"] = fns
        out.contents.self = key
        out.contents.describe, out.contents.load, out.contents.forward, out.contents.destroy = fns
        return 0

    fn = PART_FACTORY_FN(make)
    _keep_alive.extend([fn, parts])
    check(lib().celeg_register_part(role.encode(), kind.encode(), fn, None))


def _copy_view(view: TensorView) -> TensorView:
    out = TensorView()
    ctypes.memmove(ctypes.byref(out), ctypes.byref(view), ctypes.sizeof(TensorView))
    return out

"""The Python entry point: ``Engine`` (submit / step / poll / cancel / generate), and the step
function alone (``load_model``), both thin callers of the library's C interface.

Shaped after the reference's concurrent engine and its C API
(include/celeg/backend/cuda/concurrency.hpp:36-70; include/celeg/api.h:19-183:
``celeg_engine_create/submit/poll/status/cancel/step``): one ``step()`` admits, runs ONE batch
through the step function, samples on the returned logits and frees what finished.  All of that
happens inside the library (``csrc/host/engine.cpp``).
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Sequence, Tuple

import torch

from .. import native
from ..config.registry import ConfigError, read_model_folder as _read_model_folder
from ..sampling import GenerationConfig
from ..weights.checks import translate

TOKEN_FROM_DEVICE = -1


def parse_dtype(name) -> str:
    text = str(name).replace("torch.", "")
    table = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32", "f32": "float32"}
    if text not in table:
        raise ValueError(f"unknown dtype '{name}': bfloat16 or float32")
    return table[text]


def read_model_folder(model_dir: str):
    """(typed configuration, ModelSpec) of a model folder: config.json (with
    generation_config.json merged) and, for what it leaves out, the tensors' names and shapes."""
    try:
        config, spec, _ = _read_model_folder(model_dir)
    except native.NativeError as err:
        raise translate(err) from None
    return config, spec


@dataclass
class StepEntry:
    slot: int                 # the request's slot in the cache manager
    start_pos: int            # position of tokens[0] in the request's sequence
    tokens: Sequence[int]
    want: Sequence[int] = ()  # indices into ``tokens`` whose logits are wanted


class RequestStatus(enum.Enum):
    QUEUED = "queued"
    PREFILL = "prefill"
    DECODING = "decoding"
    FINISHED = "finished"
    CANCELLED = "cancelled"
    FAILED = "failed"

    @property
    def done(self) -> bool:
        return self in (RequestStatus.FINISHED, RequestStatus.CANCELLED, RequestStatus.FAILED)


@dataclass
class RequestOptions:
    """Defaults as include/celeg/runtime/request_types.hpp:16-26, except that the end tokens
    default to the model's own (None here)."""
    max_new_tokens: int = 128
    eos_token_ids: Optional[Sequence[int]] = None
    priority: int = 0
    generation: GenerationConfig = field(default_factory=GenerationConfig)


@dataclass
class SchedulerOptions:
    """Defaults as include/celeg/backend/cuda/concurrency.hpp:18-32."""
    max_active_requests: int = 8
    max_batched_tokens: int = 512
    prefill_chunk_tokens: int = 256
    policy: str = "max_utilization"      # or "guaranteed_no_evict"
    portion_granule: int = 1


def _load_error(err: Exception) -> Exception:
    translated = translate(err)
    if translated is err and isinstance(err, native.NativeArgumentError):
        return ConfigError(str(err))
    return translated


class _CacheFacade:
    """The loaded model's cache manager (inside the library)."""

    def __init__(self, model: native.NativeModel):
        self._m = model
        info = model.info
        self.page_tokens, self.max_requests = info["page_tokens"], info["max_requests"]
        self.max_context = info["max_context"]
        self.layout = info["cache_layout"]

    def open(self) -> Optional[int]:
        return self._m.open_slot()

    def close(self, slot: int) -> None:
        self._m.close_slot(slot)

    def prepare(self, slot: int, start_pos: int, n_new: int) -> bool:
        return self._m.prepare(slot, start_pos, n_new)

    def check(self) -> None:
        self._m.check_cache()

    @property
    def n_free_slots(self) -> int:
        return self._m.cache_state()["free_slots"]

    def free_pages(self) -> List[int]:
        return self._m.cache_state()["free_pages"]

    def pages_held(self, slot: int) -> List[List[int]]:
        return self._m.cache_state()["pages_held"].get(str(slot), [])

    def memory_bytes(self) -> Dict[str, int]:
        return self._m.cache_state()["memory"]


class _RunnerFacade:
    def __init__(self, model: native.NativeModel):
        self._m = model
        self.max_batched_tokens = model.info["max_batched_tokens"]

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Logits, 32-bit [number of wanted places, vocab] (on the host), in the order of the
        entries and of each entry's ``want``."""
        try:
            return torch.from_numpy(self._m.step(entries))
        except native.NativeError as err:
            raise ValueError(str(err)) from None

    @property
    def use_graphs(self) -> bool:
        return bool(self._m.knobs()["use_graphs"])

    @use_graphs.setter
    def use_graphs(self, value: bool) -> None:
        self._m.set_knob("use_graphs", int(bool(value)))

    def counters(self) -> Dict[str, int]:
        k = self._m.knobs()
        return {name: k[name] for name in ("steps_run", "graph_replays", "captures")}


class LoadedModel:
    """A model folder loaded into the library: configuration, description, cache manager and
    step function."""

    def __init__(self, model: native.NativeModel):
        from ..config.spec import ModelSpec
        from ..config.registry import typed_config
        self.native = model
        info = model.info
        self.spec = ModelSpec.from_json(info["spec"])
        self.config = typed_config(self.spec.architecture, info["config"])
        self.cache = _CacheFacade(model)
        self.runner = _RunnerFacade(model)
        self.dtype = info["dtype"]
        self.graph_safe = info["graph_safe"]

    def set_knob(self, name: str, value) -> None:
        self.native.set_knob(name, value)

    def knobs(self) -> Dict[str, int]:
        return self.native.knobs()

    def paths(self) -> Dict[str, int]:
        """How many launches each kernel family has taken so far (attention_decode,
        attention_decode_fresh, attention_rows, attention_general, linear_f32, linear_library,
        fused_sliced, fused_rows, fused_staged, tiled, tiled_qkv ...), counted when the host
        launches (also while a graph records; a replay counts nothing)."""
        return dict(self.native.knobs()["paths"])

    def close(self) -> None:
        self.native.close()


def load_model(model_dir: str, *, dtype="bfloat16", device="cuda:0", page_tokens: int = 16,
               n_pages: Optional[int] = None, max_requests: int = 8, max_context: Optional[int] = None,
               max_batched_tokens: int = 2048, gemm_backend: str = "auto", use_graphs: bool = True,
               strict_weights: bool = False) -> LoadedModel:
    """``n_pages``: pages of the cache pool (per group); by default enough for ``max_requests``
    requests of ``max_context`` tokens.  ``max_context`` defaults to the model's own maximum and
    may not exceed it.  ``gemm_backend``: how bfloat16 steps of more than 64 rows multiply:
    "library" (hipBLASLt, with separate norm and activation kernels), "tiles" (the library's own
    tiled products with the norm, SwiGLU and the residual sum folded in, where the sizes allow) or
    "auto" (the one that was measured faster at the model's width; ``describe()`` says which).
    ``strict_weights``: tensors of the checkpoint that the model has no use for are an error
    instead of a warning (``describe()["unused_tensors"]`` names them)."""
    options = native.engine_options(dtype=parse_dtype(dtype), device=native.device_index(device),
                                    max_active_requests=max_requests, max_batched_tokens=max_batched_tokens,
                                    page_tokens=page_tokens, n_pages=n_pages, context=max_context,
                                    gemm_backend=gemm_backend, use_graphs=use_graphs, strict_weights=strict_weights)
    try:
        return LoadedModel(native.NativeModel.load(model_dir, options))
    except (native.NativeError, native.NativeArgumentError) as err:
        raise _load_error(err) from None


class Engine:
    def __init__(self, handle: native.NativeEngine):
        self.native = handle
        self.loaded = LoadedModel(handle.model)

    @classmethod
    def from_folder(cls, model_dir: str, *, dtype="bfloat16", device="cuda:0", page_tokens: int = 16,
                    n_pages: Optional[int] = None, max_active_requests: int = 8,
                    max_batched_tokens: int = 2048, prefill_chunk_tokens: int = 1024,
                    context: Optional[int] = None, policy: str = "max_utilization",
                    gemm_backend: str = "auto", portion_granule: int = 1, use_graphs: bool = True,
                    run_ahead: bool = True, strict_weights: bool = False) -> "Engine":
        # (Steps of 2,048 tokens and portions of 1,024: on an MI355X a step of a few hundred rows
        # leaves most of the chip idle; the reference's 512 / 256 are ``SchedulerOptions``'.)
        options = native.engine_options(dtype=parse_dtype(dtype), device=native.device_index(device),
                                        max_active_requests=max_active_requests,
                                        max_batched_tokens=max_batched_tokens,
                                        prefill_chunk_tokens=prefill_chunk_tokens, page_tokens=page_tokens,
                                        n_pages=n_pages, policy=policy, context=context,
                                        gemm_backend=gemm_backend, use_graphs=use_graphs, run_ahead=run_ahead,
                                        portion_granule=portion_granule, strict_weights=strict_weights)
        try:
            return cls(native.NativeEngine(model_dir, options))
        except (native.NativeError, native.NativeArgumentError) as err:
            raise _load_error(err) from None

    # ------------------------------------------------------------------ requests
    def submit(self, prompt: Sequence[int], options: Optional[RequestOptions] = None) -> int:
        o = options or RequestOptions()
        g = o.generation
        try:
            return self.native.submit(prompt, max_new_tokens=o.max_new_tokens, eos_token_ids=o.eos_token_ids,
                                      priority=o.priority, temperature=g.temperature, top_k=g.top_k, top_p=g.top_p,
                                      repetition_penalty=g.repetition_penalty, seed=g.seed,
                                      forced_prefix=g.forced_prefix)
        except native.NativeArgumentError as err:
            raise ValueError(str(err)) from None

    def cancel(self, request_id: int) -> None:
        self.native.cancel(request_id)

    def release(self, request_id: int) -> None:
        """Forgets a request that has ended; the engine keeps every request's record until then.
        ValueError while it is queued or running, KeyError-like ValueError for an unknown id."""
        try:
            self.native.release(request_id)
        except native.NativeArgumentError as err:
            raise ValueError(str(err)) from None

    def status(self, request_id: int) -> RequestStatus:
        return RequestStatus(self.native.status(request_id))

    def poll(self, request_id: int) -> Tuple[RequestStatus, List[int], str]:
        status, tokens, error = self.native.poll(request_id)
        return RequestStatus(status), tokens, error

    def has_work(self) -> bool:
        return self.native.has_work()

    def step(self) -> int:
        """Runs one batch; returns the number of tokens it fed (0 if there was nothing)."""
        return self.native.step()

    def run(self) -> None:
        """Steps until nothing is queued or active, decode steps launched one ahead of their tokens."""
        self.native.run()

    @property
    def metrics(self) -> Dict[str, Any]:
        return self.native.metrics()

    def request_metrics(self, request_id: int) -> Dict[str, Any]:
        return self.native.request_metrics(request_id)

    @property
    def last_logits(self) -> torch.Tensor:
        return torch.from_numpy(self.native.last_logits())

    # ------------------------------------------------------------------ convenience
    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 128,
                 generation: Optional[GenerationConfig] = None,
                 eos_token_ids: Optional[Sequence[int]] = None,
                 generations: Optional[Sequence[GenerationConfig]] = None) -> List[List[int]]:
        """Generate for every prompt (all submitted at once, batched by the scheduler) and return
        the generated tokens, the end token included if one was met."""
        ids = []
        for i, prompt in enumerate(prompts):
            g = generations[i] if generations is not None else (generation or GenerationConfig())
            ids.append(self.submit(prompt, RequestOptions(max_new_tokens=max_new_tokens,
                                                          eos_token_ids=eos_token_ids, generation=g)))
        self.run()
        out = []
        for rid in ids:
            status, tokens, error = self.poll(rid)
            out.append((status, tokens, error))
        for rid in ids:
            self.release(rid)
        for rid, (status, tokens, error) in zip(ids, out):
            if status == RequestStatus.FAILED:
                raise RuntimeError(f"request {rid} failed: {error}")
        return [tokens for _, tokens, _ in out]

    def close(self) -> None:
        self.native.close()


class Scheduler:
    """The library's scheduler over a cache manager's bookkeeping, without a GPU: what the tests
    of its decisions drive (``plan`` -> entries, ``accept`` <- the tokens a step sampled)."""

    def __init__(self, cache, options: SchedulerOptions, *, max_context: int, default_eos: Sequence[int] = ()):
        from ..cache import _Host
        self.cache = cache
        self.options = options
        self._host = _Host("scheduler", cache=cache.handle, options=vars(options), max_context=max_context,
                           default_eos=list(default_eos))

    def submit(self, prompt: Sequence[int], options: Optional[RequestOptions] = None) -> int:
        o = options or RequestOptions()
        return self._host._call("submit", [int(t) for t in prompt],
                                {"max_new_tokens": o.max_new_tokens, "priority": o.priority,
                                 "eos_token_ids": None if o.eos_token_ids is None else list(o.eos_token_ids),
                                 "generation": dict(vars(o.generation), forced_prefix=list(o.generation.forced_prefix))})

    def cancel(self, request_id: int) -> None:
        self._host._call("cancel", request_id)

    def release(self, request_id: int) -> bool:
        """Forgets a request that has ended; False (and nothing happens) while it has not."""
        return self._host._call("release", request_id)

    def has_work(self) -> bool:
        return self._host._call("has_work")

    def plan(self) -> List[Dict[str, Any]]:
        """This step's entries: {"id", "slot", "start", "count", "samples", "tokens"} each."""
        return self._host._call("plan")

    def accept(self, sampled: Sequence[int]) -> None:
        self._host._call("accept", [int(t) for t in sampled])

    def fail(self, message: str) -> None:
        self._host._call("fail", message)

    def poll(self, request_id: int):
        r = self._host._call("poll", request_id)
        return RequestStatus(r["status"]), r["tokens"], r["error"]

    def request(self, request_id: int) -> Dict[str, Any]:
        return self._host._call("request", request_id)

    def slot_events(self) -> Dict[str, Any]:
        return self._host._call("slot_events")

    @property
    def stats(self) -> Dict[str, int]:
        return self._host._call("stats")

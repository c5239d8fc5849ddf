"""Parts written in Python, for a model that the library runs.

The library's parts (RMS norm, rotary encoding, grouped-query attention, short convolution,
SwiGLU, embedding, heads, the pre-norm block) are C++ classes in ``csrc/host/parts.cpp``,
registered by kind.  A part defined elsewhere registers through the C interface's
``celeg_register_part`` as a set of functions; this module is the Python side of that: a part is
an object with

* ``describe() -> dict``: ``{"weights": {role: {"shape", "kind": "matrix"|"vector", "init":
  "normal"|"around_one"}}, "kv_need": {"kv_heads", "head_dim", "window"} or None, "states":
  [{"name", "shape", "dtype"}], "graph_safe": False, "out_width": columns of the output}``; a
  position encoding gives ``{"inv_freq": [...], "rotary_dim": n}`` instead;
* optionally ``load(tensors: {role: TensorView})``;
* ``forward(args: ForwardArgs)``: device pointers in, result written to ``args.out``.

``as_tensor`` turns a view of device memory into a torch tensor that shares it, ``on_stream``
makes torch work on the model's stream, so that such a part can be written with torch.
"""
from __future__ import annotations

import contextlib
from typing import Any, Dict

from ..native import ForwardArgs, TensorView, register_part, registered  # noqa: F401

_TYPES = {0: ("<f4", 4), 1: ("<u2", 2), 2: ("<i4", 4), 3: ("|u1", 1)}


class _Exposed:
    def __init__(self, interface: Dict[str, Any]):
        self.__cuda_array_interface__ = interface


def as_tensor(view: TensorView):
    """A torch tensor over the device memory a view names (bfloat16 comes as bfloat16)."""
    import torch
    typestr, size = _TYPES[view.dtype]
    shape = tuple(int(view.shape[i]) for i in range(view.ndim))
    strides = tuple(int(view.stride[i]) * size for i in range(view.ndim))
    if 0 in shape:
        dtype = {0: torch.float32, 1: torch.bfloat16, 2: torch.int32, 3: torch.uint8}[view.dtype]
        return torch.empty(shape, dtype=dtype, device="cuda")
    t = torch.as_tensor(_Exposed({"shape": shape, "typestr": typestr, "data": (int(view.data), False),
                                  "version": 2, "strides": strides}), device="cuda")
    return t.view(torch.bfloat16) if view.dtype == 1 else t


def int_array(pointer, count: int):
    """int32 device array (a field of ``args.step``) as a torch tensor."""
    view = TensorView()
    view.data, view.dtype, view.ndim = pointer, 2, 1
    view.shape[0], view.stride[0] = count, 1
    return as_tensor(view)


@contextlib.contextmanager
def on_stream(args: ForwardArgs):
    """torch's current stream is the model's for the duration."""
    import torch
    with torch.cuda.stream(torch.cuda.ExternalStream(int(args.stream))):
        yield


def registered_parts(role: str):
    return registered(role)


__all__ = ["ForwardArgs", "TensorView", "register_part", "registered_parts", "as_tensor", "int_array", "on_stream"]

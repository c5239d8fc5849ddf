"""Reading and writing the safetensors container.

Layout: an 8-byte little-endian header length, a JSON header
``{name: {dtype, shape, data_offsets}}`` and the data section
(the reference's reader: src/checkpoint/formats/safetensors.cpp:93-239, dtype
table 28-38, ``tensor(name)`` 283-297).  Tensors are memory-mapped and only the
bytes that are asked for are touched.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, Iterable, List, Mapping, Tuple

import numpy as np
import torch


class SafetensorsError(ValueError):
    pass


# name -> (bytes per element, numpy dtype to view the bytes with, torch dtype)
_DTYPES = {
    "F32": (4, np.dtype("<f4"), torch.float32),
    "F16": (2, np.dtype("<f2"), torch.float16),
    "BF16": (2, np.dtype("<u2"), torch.bfloat16),
    "I64": (8, np.dtype("<i8"), torch.int64),
    "I32": (4, np.dtype("<i4"), torch.int32),
    "I16": (2, np.dtype("<i2"), torch.int16),
    "I8": (1, np.dtype("i1"), torch.int8),
    "U8": (1, np.dtype("u1"), torch.uint8),
}
_TORCH_TO_NAME = {torch.float32: "F32", torch.float16: "F16", torch.bfloat16: "BF16",
                  torch.int64: "I64", torch.int32: "I32", torch.int16: "I16",
                  torch.int8: "I8", torch.uint8: "U8"}


class TensorInfo:
    __slots__ = ("name", "dtype", "shape", "begin", "end")

    def __init__(self, name, dtype, shape, begin, end):
        self.name, self.dtype, self.shape, self.begin, self.end = name, dtype, shape, begin, end

    @property
    def is_float(self) -> bool:
        return self.dtype in ("F32", "F16", "BF16")


class SafetensorsFile:
    """One .safetensors file, validated on opening."""

    def __init__(self, path: str):
        self.path = path
        size = os.path.getsize(path)
        if size < 8:
            raise SafetensorsError(f"invalid safetensors file: too small: {path}")
        self._fh = open(path, "rb")
        (header_len,) = struct.unpack("<Q", self._fh.read(8))
        if header_len == 0 or 8 + header_len > size:
            raise SafetensorsError(f"invalid safetensors header length {header_len} in {path}")
        try:
            header = json.loads(self._fh.read(header_len).decode("utf-8"),
                                object_pairs_hook=self._no_duplicates)
        except (UnicodeDecodeError, json.JSONDecodeError) as err:
            raise SafetensorsError(f"invalid safetensors header in {path}: {err}") from err
        if not isinstance(header, dict):
            raise SafetensorsError(f"invalid safetensors header in {path}: not an object")
        self._data_start = 8 + header_len
        data_size = size - self._data_start
        self.metadata = header.pop("__metadata__", {})
        self.tensors: Dict[str, TensorInfo] = {}
        spans: List[Tuple[int, int, str]] = []
        for name, entry in header.items():
            try:
                dtype, shape = entry["dtype"], [int(s) for s in entry["shape"]]
                begin, end = (int(o) for o in entry["data_offsets"])
            except (KeyError, TypeError, ValueError) as err:
                raise SafetensorsError(f"malformed header entry for tensor {name} in {path}") from err
            if dtype not in _DTYPES:
                raise SafetensorsError(f"unsupported dtype {dtype} for tensor {name} in {path}")
            if begin < 0 or end < begin or end > data_size:
                raise SafetensorsError(f"out-of-range tensor {name} in {path}")
            count = 1
            for s in shape:
                if s < 0:
                    raise SafetensorsError(f"negative dimension in tensor {name} in {path}")
                count *= s
            if count * _DTYPES[dtype][0] != end - begin:
                raise SafetensorsError(f"byte count does not match shape for tensor {name} in {path}")
            self.tensors[name] = TensorInfo(name, dtype, tuple(shape), begin, end)
            if end > begin:
                spans.append((begin, end, name))
        spans.sort()
        for (b0, e0, n0), (b1, e1, n1) in zip(spans, spans[1:]):
            if b1 < e0:
                raise SafetensorsError(f"overlapping tensor ranges: {n0} and {n1} in {path}")
        self._map = None

    @staticmethod
    def _no_duplicates(pairs):
        out = {}
        for key, value in pairs:
            if key in out:
                raise SafetensorsError(f"duplicate tensor name: {key}")
            out[key] = value
        return out

    def names(self) -> List[str]:
        return list(self.tensors)

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor of the stored dtype, backed by the mapping (read-only: clone or
        convert before writing)."""
        if name not in self.tensors:
            raise SafetensorsError(f"missing tensor: {name}")
        info = self.tensors[name]
        if self._map is None:
            self._map = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_READ)
        _, np_dtype, torch_dtype = _DTYPES[info.dtype]
        count = (info.end - info.begin) // np_dtype.itemsize
        array = np.frombuffer(self._map, dtype=np_dtype, count=count,
                              offset=self._data_start + info.begin)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # the mapping is read-only; callers copy
            t = torch.from_numpy(array)
        if info.dtype == "BF16":
            t = t.view(torch.bfloat16)
        return t.reshape(info.shape)

    def close(self) -> None:
        if self._map is not None:
            try:
                self._map.close()
            except BufferError:
                pass  # tensors that still view the mapping keep it alive
            self._map = None
        self._fh.close()


def write_safetensors(path: str, tensors: Mapping[str, torch.Tensor],
                      metadata: Mapping[str, str] = None) -> None:
    """Write CPU tensors, in the given order, 8-byte aligned header."""
    header = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    offset = 0
    blobs = []
    for name, t in tensors.items():
        t = t.detach().cpu().contiguous()
        if t.dtype not in _TORCH_TO_NAME:
            raise SafetensorsError(f"cannot store dtype {t.dtype} of tensor {name}")
        raw = t.reshape(-1).view(torch.uint8).numpy()
        header[name] = {"dtype": _TORCH_TO_NAME[t.dtype], "shape": list(t.shape),
                        "data_offsets": [offset, offset + len(raw)]}
        offset += len(raw)
        blobs.append(raw)
    text = json.dumps(header, separators=(",", ":")).encode("utf-8")
    text += b" " * ((8 - len(text) % 8) % 8)
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(text)))
        fh.write(text)
        for raw in blobs:
            fh.write(raw)

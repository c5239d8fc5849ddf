"""The library's check of a model folder's checkpoint against what the model's parts expect.

Opening the container (one file or a sharded index), its validation, the check and the way to
the device are the library's (``csrc/host/weights.cpp``).  ALL problems of a checkpoint come as
one error: missing tensors, tensors nobody asked for, and wrong shapes.  Tensors nobody asked
for are no problem by themselves (the reference binds tensors by name and leaves the rest alone,
include/celeg/checkpoint/weight_repository.hpp:14-20): loading warns about them, and ``strict``
makes them an error.
"""
from __future__ import annotations

from .. import native
from .safetensors_io import SafetensorsError


class WeightError(ValueError):
    """The checkpoint does not fit the model.  ``missing``, ``unexpected`` and ``wrong_shape``
    hold the details that the message lists."""

    def __init__(self, message: str):
        super().__init__(message)
        self.missing, self.unexpected, self.wrong_shape = [], [], []
        for line in message.splitlines():
            line = line.strip()
            if line.startswith("missing tensors"):
                self.missing = line.split(": ", 1)[1].split(", ")
            elif line.startswith("unexpected tensors"):
                self.unexpected = line.split(": ", 1)[1].split(", ")
            elif line.startswith("wrong shape: "):
                self.wrong_shape.append(line[len("wrong shape: "):])


def translate(err: Exception) -> Exception:
    """A failure of the library while it read a model folder, as the Python error it stands for."""
    text = str(err)
    if "does not fit the model" in text:
        return WeightError(text)
    if "config.json not found" in text or "no model.safetensors" in text:
        return FileNotFoundError(text)
    if "safetensors" in text or "tensor" in text:
        return SafetensorsError(text)
    return err


def check_folder(model_dir: str, strict: bool = False) -> None:
    """Raises ``WeightError`` (the checkpoint does not fit), ``SafetensorsError`` (a malformed
    container), ``FileNotFoundError`` or ``ConfigError``; returns None if the folder loads."""
    from ..config.registry import ConfigError
    try:
        native.check_folder(model_dir, strict)
    except native.NativeArgumentError as err:
        translated = translate(err)
        raise (translated if translated is not err else ConfigError(str(err))) from None
    except native.NativeError as err:
        raise translate(err) from None

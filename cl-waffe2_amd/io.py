"""Weights between ``.npy`` files and device tensors.

``load_npy`` is the GPT-2 example's loader (``examples/gpt-2/utils.lisp:6-9``:
``numpy-file-format:load-array`` + ``change-facet``) with the array going to the
device in one bulk transfer.  ``save_weights`` / ``load_weights`` read and write
the ``:wf2model`` layout (``source/backends/lisp/wf2model.lisp:5-54``): a
directory holding ``parameters.json``, which maps every key of the state
dictionary either to a plain value or to the path of a ``<key>.npy`` file with
the tensor's storage vector (flat, as ``tensor-vec`` is).
"""
from __future__ import annotations

import json
import os

import numpy as np

from .tensor import HIPTensor


def _as_float32(a: np.ndarray, what: str) -> np.ndarray:
    if a.dtype.kind != "f":
        raise TypeError(f"{what}: HIPTensor holds :float, the file has dtype {a.dtype}")
    return np.ascontiguousarray(a, dtype=np.float32)


def load_npy(path: str) -> HIPTensor:
    """A ``.npy`` array as a device tensor of the same shape (executes nothing
    from the file: ``allow_pickle`` stays off)."""
    return HIPTensor.from_numpy(_as_float32(np.load(path, allow_pickle=False), path))


def save_npy(tensor: HIPTensor, path: str) -> None:
    """The visible tensor (views applied) as a ``.npy`` file."""
    np.save(path, tensor.numpy(), allow_pickle=False)


def save_weights(path: str, state_dict: dict) -> None:
    """``(save-weights model path :wf2model)``: tensors go to ``<path>/<key>.npy``
    as their flat storage vector, everything else into ``parameters.json``."""
    os.makedirs(path, exist_ok=True)
    table = {}
    for key, value in state_dict.items():
        if isinstance(value, HIPTensor):
            file = f"{path}/{key}.npy"
            os.makedirs(os.path.dirname(file), exist_ok=True)
            np.save(file, value.storage_numpy(), allow_pickle=False)
            table[key] = file
        elif isinstance(value, str):
            raise TypeError(f"{key}: a string value would be read back as a tensor path")
        else:
            table[key] = value
    with open(os.path.join(path, "parameters.json"), "w") as f:
        json.dump(table, f)


def load_weights(path: str, shapes: dict | None = None) -> dict:
    """``(load-weights model path :wf2model)``: every string entry of
    ``parameters.json`` names a ``.npy`` file that becomes a device tensor.  The
    files hold flat storage vectors; ``shapes`` gives the shape a key is viewed
    with (``from-state-dict`` takes it from the model's parameters)."""
    with open(os.path.join(path, "parameters.json")) as f:
        table = json.load(f)
    out = {}
    for key, value in table.items():
        if isinstance(value, str):
            a = _as_float32(np.load(value, allow_pickle=False), value)
            if shapes and key in shapes:
                a = a.reshape(shapes[key])
            out[key] = HIPTensor.from_numpy(a)
        else:
            out[key] = value
    return out

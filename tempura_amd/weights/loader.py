"""Weights by tensor name from the ``*.safetensors`` files of a model folder.

Every ``*.safetensors`` file in the folder is read in path order; a later file's
tensor replaces an earlier one of the same name; an empty folder is an error
(/root/reference/engine/src/loader.rs:119-145).  bfloat16 stays bfloat16, float16
is widened exactly to float32, a tensor stored in 32-bit stays 32-bit, integer
tables become int32.  All faults of a checkpoint
(missing and unexpected tensors, wrong shapes) are reported in ONE error; the
reference stops at the first (/root/reference/engine/src/weights.rs:28-42,150-195)
and checks element counts only (weights.rs:230-238).
"""
from __future__ import annotations

import glob
import os
from typing import Callable, Dict, List, Optional

import torch

from ..parts.base import WeightInfo
from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightsError(ValueError):
    """A checkpoint that does not fit the model.  ``missing``, ``unexpected`` and
    ``wrong_shape`` (name -> (expected, found)) carry the details."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=None):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = dict(wrong_shape or {})


class Checkpoint:
    """All tensors of a model folder, by name."""

    def __init__(self, model_dir: str):
        self.model_dir = model_dir
        paths = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
        if not paths:
            raise WeightsError(f"no .safetensors files in {model_dir}")
        self.files = [SafetensorsFile(p) for p in paths]
        self._where: Dict[str, SafetensorsFile] = {}
        for f in self.files:                # later files overwrite earlier names
            for n in f.names():
                self._where[n] = f

    def names(self) -> List[str]:
        return list(self._where)

    def shape(self, name: str):
        return self._where[name].shape(name)

    def dtype_tag(self, name: str) -> str:
        return self._where[name].dtype_tag(name)

    def tensor(self, name: str) -> torch.Tensor:
        """The tensor on the host in its kept dtype."""
        t = self._where[name].tensor(name)
        if t.dtype == torch.float16:
            return t.to(torch.float32)      # exact widening
        if t.dtype == torch.float64:
            return t.to(torch.float32)
        if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8, torch.bool):
            return t.to(torch.int32)
        return t                            # bfloat16, float32, int32 as stored

    def close(self) -> None:
        for f in self.files:
            f.close()


def check_checkpoint(ckpt: Checkpoint, expected: Dict[str, WeightInfo]) -> None:
    """Raise one ``WeightsError`` that lists every missing, unexpected and mis-shaped tensor."""
    have = set(ckpt.names())
    missing = sorted(n for n, info in expected.items() if n not in have and not info.optional)
    unexpected = sorted(n for n in have if n not in expected)
    wrong = {}
    for n, info in expected.items():
        if n in have and tuple(ckpt.shape(n)) != tuple(info.shape):
            wrong[n] = (tuple(info.shape), tuple(ckpt.shape(n)))
    if missing or unexpected or wrong:
        lines = [f"checkpoint in {ckpt.model_dir} does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes ({len(wrong)}): " + ", ".join(
                f"{n} expected {list(e)} found {list(f)}" for n, (e, f) in sorted(wrong.items())))
        raise WeightsError("\n".join(lines), missing, unexpected, wrong)


def load_into(model, model_dir: str) -> None:
    """Check the folder's tensors against ``model`` and load them, tensor by tensor."""
    try:
        ckpt = Checkpoint(model_dir)
    except SafetensorsError as e:
        raise WeightsError(str(e)) from e
    expected = model.expected_weights()
    check_checkpoint(ckpt, expected)
    have = set(ckpt.names())

    def get(name: str, optional: bool = False) -> Optional[torch.Tensor]:
        if name not in have:
            if optional:
                return None
            raise WeightsError(f"missing tensor {name}", [name])
        return ckpt.tensor(name)

    model.load_weights(get)
    ckpt.close()

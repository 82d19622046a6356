"""Weights by tensor name from the ``*.safetensors`` files of a model folder.

Every ``*.safetensors`` file in the folder is read in path order; a later file's
tensor replaces an earlier one of the same name; an empty folder is an error
(/root/reference/engine/src/loader.rs:119-145).  bfloat16 stays bfloat16, float16
is widened exactly to float32, a tensor stored in 32-bit stays 32-bit, integer
tables become int32.  A weight must be stored as F32, BF16 or F16 and an integer table
as an integer type; anything else is refused by name (the reference reads the bytes of
any other type as if they were float32, /root/reference/engine/src/loader.rs:191-208).
All faults of a checkpoint (missing and unexpected tensors, wrong shapes, wrong element
types) are reported in ONE error; the reference stops at the first
(/root/reference/engine/src/weights.rs:28-42,150-195) and checks element counts only
(weights.rs:230-238).

A folder may hold ``integrity.json``, ``{"tensor_hashes": {name: sha256 of the stored
bytes}}``; every tensor it names is then verified while it is loaded
(/root/reference/engine/src/loader.rs:147-182 hashes the widened float32 values; here
the bytes as stored, so that a bfloat16 checkpoint is never widened just to be hashed;
a digest that fits neither the stored bytes of a BF16 or F16 tensor is tried against the
widened values before the tensor is refused, so that a manifest made the reference's way
verifies here too).
"""
from __future__ import annotations

import glob
import hashlib
import json
import os
import warnings
from typing import Callable, Dict, List, Optional

import torch

from ..parts.base import WeightInfo
from .safetensors_io import SafetensorsError, SafetensorsFile


class WeightsError(ValueError):
    """A checkpoint that does not fit the model.  ``missing``, ``unexpected`` and
    ``wrong_shape`` (name -> (expected, found)) carry the details."""

    def __init__(self, message, missing=(), unexpected=(), wrong_shape=None, wrong_dtype=None):
        super().__init__(message)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = dict(wrong_shape or {})
        self.wrong_dtype = dict(wrong_dtype or {})      # name -> (accepted tags, found tag)


#: element types a checkpoint may store a tensor of each kind in
ACCEPTED_TAGS = {"float": ("F32", "BF16", "F16"), "int": ("I64", "I32", "I16", "I8", "U8")}
MANIFEST_NAME = "integrity.json"


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
        """The tensor on the host in its kept dtype: bfloat16, float32 and int32 as stored, float16 widened
        (exactly) to float32, other integers to int32.  Any other stored type is refused."""
        tag = self.dtype_tag(name)
        if tag not in ACCEPTED_TAGS["float"] and tag not in ACCEPTED_TAGS["int"]:
            raise WeightsError(f"tensor {name} is stored as {tag}: weights must be F32, BF16 or F16, integer tables an integer type",
                               wrong_dtype={name: (ACCEPTED_TAGS["float"] + ACCEPTED_TAGS["int"], tag)})
        t = self._where[name].tensor(name)
        if t.dtype == torch.float16:
            return t.to(torch.float32)      # exact widening
        if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8):
            return t.to(torch.int32)
        return t

    def sha256(self, name: str) -> str:
        """Hex digest of the tensor's bytes as stored."""
        t = self._where[name].tensor(name).contiguous()
        return hashlib.sha256(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"").hexdigest()

    def sha256_widened(self, name: str) -> Optional[str]:
        """Hex digest of a BF16 or F16 tensor's values widened (exactly) to little-endian float32, which is what
        the reference hashes (/root/reference/engine/src/loader.rs:147-182); None for other stored types, whose
        widened form is the stored one."""
        if self.dtype_tag(name) not in ("BF16", "F16"):
            return None
        t = self._where[name].tensor(name).to(torch.float32).contiguous()
        return hashlib.sha256(t.view(torch.uint8).numpy().tobytes() if t.numel() else b"").hexdigest()

    def close(self) -> None:
        for f in self.files:
            f.close()


def check_checkpoint(ckpt: Checkpoint, expected: Dict[str, WeightInfo]) -> None:
    """Raise one ``WeightsError`` that lists every missing, unexpected and mis-shaped tensor."""
    have = set(ckpt.names())
    missing = sorted(n for n, info in expected.items() if n not in have and not info.optional)
    unexpected = sorted(n for n in have if n not in expected)
    wrong, wrong_dt = {}, {}
    for n, info in expected.items():
        if n not in have:
            continue
        if tuple(ckpt.shape(n)) != tuple(info.shape):
            wrong[n] = (tuple(info.shape), tuple(ckpt.shape(n)))
        accepted = ACCEPTED_TAGS[getattr(info, "kind", "float")]
        if ckpt.dtype_tag(n) not in accepted:
            wrong_dt[n] = (accepted, ckpt.dtype_tag(n))
    if missing or unexpected or wrong or wrong_dt:
        lines = [f"checkpoint in {ckpt.model_dir} does not fit the model:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shapes ({len(wrong)}): " + ", ".join(
                f"{n} expected {list(e)} found {list(f)}" for n, (e, f) in sorted(wrong.items())))
        if wrong_dt:
            lines.append(f"  wrong element types ({len(wrong_dt)}): " + ", ".join(
                f"{n} stored as {f}, accepted {'/'.join(a)}" for n, (a, f) in sorted(wrong_dt.items())))
        raise WeightsError("\n".join(lines), missing, unexpected, wrong, wrong_dt)


def write_manifest(model_dir: str) -> str:
    """Write ``integrity.json`` for the folder's tensors as they are now; returns its path."""
    ckpt = Checkpoint(model_dir)
    hashes = {n: ckpt.sha256(n) for n in sorted(ckpt.names())}
    ckpt.close()
    path = os.path.join(model_dir, MANIFEST_NAME)
    with open(path, "w") as f:
        json.dump({"tensor_hashes": hashes}, f, indent=1, sort_keys=True)
    return path


def read_manifest(model_dir: str) -> Optional[Dict[str, str]]:
    path = os.path.join(model_dir, MANIFEST_NAME)
    if not os.path.exists(path):
        return None
    try:
        with open(path) as f:
            hashes = json.load(f)["tensor_hashes"]
        if not isinstance(hashes, dict) or not all(isinstance(v, str) for v in hashes.values()):
            raise ValueError("tensor_hashes must map names to hex digests")
    except (OSError, ValueError, KeyError, TypeError) as e:
        raise WeightsError(f"{path}: not an integrity manifest: {e}") from e
    return hashes


def load_into(model, model_dir: str, verify: Optional[bool] = None) -> None:
    """Check the folder's tensors against ``model`` and load them, tensor by tensor.
    ``verify``: None checks the tensors against ``integrity.json`` when the folder has one, True demands
    one, False skips it."""
    try:
        ckpt = Checkpoint(model_dir)
    except SafetensorsError as e:
        raise WeightsError(str(e)) from e
    expected = model.expected_weights()
    check_checkpoint(ckpt, expected)
    have = set(ckpt.names())
    manifest = read_manifest(model_dir) if verify is not False else None
    if verify is True and manifest is None:
        raise WeightsError(f"{model_dir} has no {MANIFEST_NAME} to verify against")
    if manifest:
        absent = sorted(n for n in manifest if n not in have)
        if absent:
            raise WeightsError(f"{MANIFEST_NAME} names tensors the checkpoint does not hold: " + ", ".join(absent), absent)

    def get(name: str, optional: bool = False) -> Optional[torch.Tensor]:
        if name not in have:
            if optional:
                return None
            raise WeightsError(f"missing tensor {name}", [name])
        if manifest and name in manifest:
            got = ckpt.sha256(name)
            if got != manifest[name].lower() and ckpt.sha256_widened(name) != manifest[name].lower():
                raise WeightsError(f"tensor {name} fails its integrity check: expected sha256 {manifest[name]}, got {got}")
        return ckpt.tensor(name)

    # a tied output head reads the embedding matrix; a matrix of its own that the checkpoint still holds is not
    # an error (/root/reference/engine/src/weights.rs:156-166 falls back to the embedding only when it is absent),
    # but the user should know that it is not what runs
    ignored = sorted(n for n, info in expected.items() if info.init == "skip" and n in have)
    if ignored:
        warnings.warn(f"checkpoint in {model_dir} holds {', '.join(ignored)}, but the configuration ties that tensor to "
                      f"another (tie_word_embeddings): the stored tensor is ignored", stacklevel=2)
    model.load_weights(get)
    ckpt.close()

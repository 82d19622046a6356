"""Random-weights mode: write a model folder from a configuration and a seed.

The reference has this as a test fixture only (seeded matrices, norm weights
1.0, /root/reference/engine/src/model.rs:11335-11409); here it is a mode of the
product.  Matrices are N(0, std), norm weights are 1.0 (or, with
``norm_jitter``, 1 + N(0, norm_jitter) so that a forgotten norm weight shows).
Each tensor has a generator of its own, keyed by seed and name, so its values do
not depend on the order tensors are made in.
"""
from __future__ import annotations

import hashlib
import os
from typing import Callable, Dict, Optional

import torch

from ..parts.inventory import expected_weights
from ..parts.base import WeightInfo
from .safetensors_io import write_safetensors

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "float16": torch.float16}


def _tensor_seed(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(name: str, info: WeightInfo, seed: int, std: float, norm_jitter: float,
                  dtype: torch.dtype) -> torch.Tensor:
    g = torch.Generator(device="cpu")
    g.manual_seed(_tensor_seed(seed, name))
    if info.init == "ones":
        t = torch.ones(info.shape, dtype=torch.float32)
        if norm_jitter:
            t += torch.randn(info.shape, generator=g, dtype=torch.float32) * norm_jitter
    else:
        t = torch.randn(info.shape, generator=g, dtype=torch.float32) * std
    return t.to(dtype)


def random_weights(config, seed: int = 0, std: float = 0.02, norm_jitter: float = 0.0,
                   dtype: str = "bfloat16") -> Dict[str, torch.Tensor]:
    spec = config.build_spec()
    td = _DTYPES[dtype]
    out = {}
    for name, info in expected_weights(spec).items():
        if info.init == "skip":
            continue
        out[name] = random_tensor(name, info, seed, std, norm_jitter, td)
    return out


def write_random_model(config, out_dir: str, seed: int = 0, std: float = 0.02, norm_jitter: float = 0.0,
                       dtype: str = "bfloat16") -> str:
    """Write ``config.json`` and ``model.safetensors`` into ``out_dir``; returns it."""
    os.makedirs(out_dir, exist_ok=True)
    cfg = config
    if hasattr(cfg, "torch_dtype"):
        cfg.torch_dtype = dtype
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        f.write(cfg.to_json())
    tensors = random_weights(cfg, seed, std, norm_jitter, dtype)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors.items(),
                      metadata={"format": "pt", "seed": seed})
    return out_dir

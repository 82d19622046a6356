"""Random-weights mode: write a model folder from a configuration and a seed.

The reference has this as a test fixture only (seeded matrices, norm weights
1.0, /root/reference/engine/src/model.rs:11335-11409); here it is a mode of the
product.  Matrices are N(0, std), norm weights are 1.0 (or, with
``norm_jitter``, 1 + N(0, norm_jitter) so that a forgotten norm weight shows).
Each tensor has a stream of its own, keyed by seed and name, and element i of a tensor
depends on (that key, i) alone: a counter-based Box-Muller deviate built from correctly
rounded float64 operations only (csrc/counter_normal.h), so the host library here and the
device kernel (``ops.fill_normal``) give every element the same bits, and a model made in
device memory can be regenerated tensor by tensor on the host.
"""
from __future__ import annotations

import ctypes
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


def fill_normal_host(out: torch.Tensor, seed: int, mean: float, std: float) -> torch.Tensor:
    """Fill a contiguous float32 or bfloat16 host tensor with mean + std * N(0, 1); element i depends only on
    (seed, i) and equals what the device kernel writes there."""
    from ..cache import native
    if out.device.type != "cpu" or not out.is_contiguous() or out.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("fill_normal_host: needs a contiguous float32 or bfloat16 host tensor")
    lib = native.lib()
    rc = lib.hr_fill_normal(ctypes.c_void_p(out.data_ptr()), 0 if out.dtype == torch.float32 else 1,
                            ctypes.c_size_t(out.numel()), ctypes.c_ulonglong(seed & (2 ** 64 - 1)),
                            ctypes.c_double(mean), ctypes.c_double(std), int(min(16, os.cpu_count() or 1)))
    if rc != 0:
        raise RuntimeError("fill_normal_host failed")
    return out


def random_tensor(name: str, info: WeightInfo, seed: int, std: float, norm_jitter: float,
                  dtype: torch.dtype) -> torch.Tensor:
    """The tensor ``name`` of the random model with this seed.  Matrices are drawn in the stored type when
    that is float32 or bfloat16 (float16: drawn as float32, then rounded); norm weights are float32 values
    1 + jitter, then converted."""
    key = _tensor_seed(seed, name)
    if info.init == "ones":
        t = torch.ones(info.shape, dtype=torch.float32)
        if norm_jitter:
            fill_normal_host(t, key, 1.0, norm_jitter)
        return t.to(dtype)
    if dtype in (torch.float32, torch.bfloat16):
        return fill_normal_host(torch.empty(info.shape, dtype=dtype), key, 0.0, std)
    return fill_normal_host(torch.empty(info.shape, dtype=torch.float32), key, 0.0, std).to(dtype)


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

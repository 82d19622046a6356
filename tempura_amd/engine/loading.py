"""From a model folder to a model on the device."""
from __future__ import annotations

import torch

from ..config import load_config
from ..weights.loader import load_into
from ..weights.random_init import random_tensor
from .model import CausalLM

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"dtype must be bfloat16 or float32, got {dtype}")
        return dtype
    try:
        return _DTYPES[str(dtype)]
    except KeyError:
        raise ValueError(f"dtype must be one of {sorted(_DTYPES)}, got {dtype!r}") from None


class NoDeviceError(RuntimeError):
    """The device that was asked for is not there."""


def require_device(device) -> torch.device:
    """``device`` as a torch.device; one clear error when it names a GPU and none is visible (the engine has no
    CPU path: on the CPU only the tests' stand-in operations run, with device "cpu")."""
    device = torch.device(device)
    if device.type == "cuda" and not torch.cuda.is_available():
        raise NoDeviceError(f"no GPU is visible to this process (device {str(device)!r} was asked for, "
                            "torch.cuda.is_available() is False); tempura_amd runs on an AMD MI355X and has no CPU path")
    return device


def load_model(model_dir: str, dtype="bfloat16", device="cuda:0") -> CausalLM:
    """Read ``config.json``, pick the architecture from the registry, build it, load its weights."""
    device = require_device(device)
    config = load_config(model_dir)
    model = CausalLM(config.build_spec(), parse_dtype(dtype), torch.device(device))
    model.config = config
    load_into(model, model_dir)
    return model


def random_model(config, seed: int = 0, dtype="bfloat16", device="cuda:0", std: float = 0.02,
                 norm_jitter: float = 0.0, on_device: bool = None, values_as=None) -> CausalLM:
    """A model with seeded random weights made tensor by tensor, never written to disk
    (for sizes whose folder would be tens of gigabytes).  With ``on_device`` (the default on a
    GPU) each tensor is filled by a kernel in device memory, with the same values as the host
    generator's that ``write_random_model`` uses.  ``values_as`` (a dtype name) rounds the matrix
    values to that type first, so that a float32 model can hold exactly a bfloat16 model's weights."""
    device = require_device(device)
    from ..kernels import ops
    from ..weights.random_init import _tensor_seed
    td = parse_dtype(dtype)
    dev = torch.device(device)
    if on_device is None:
        on_device = dev.type == "cuda"
    model = CausalLM(config.build_spec(), td, dev)
    model.config = config
    expected = model.expected_weights()
    store = torch.bfloat16 if td == torch.bfloat16 else torch.float32

    def get(name, optional=False):
        info = expected[name]
        if info.init == "skip":
            return None
        if not on_device:
            return random_tensor(name, info, seed, std, norm_jitter, store)
        if info.init == "ones":
            t = torch.ones(info.shape, dtype=torch.float32, device=dev)
            if norm_jitter:
                # (rounded to the stored type as a written folder's norm weights are)
                t = ops.fill_normal(t, _tensor_seed(seed, name), 1.0, norm_jitter).to(store).to(torch.float32)
            return t
        t = torch.empty(info.shape, dtype=parse_dtype(values_as) if values_as else store, device=dev)
        return ops.fill_normal(t, _tensor_seed(seed, name), 0.0, std).to(store)

    model.load_weights(get)
    return model

"""The counter-based generator of random weights: host library, numpy twin and (on the GPU) the device kernel
give every element the same bits."""
import math

import numpy as np
import pytest
import torch

import helpers
import plain_random
from tempura_amd.config import LlamaConfig
from tempura_amd.weights import random_weights
from tempura_amd.weights.random_init import _tensor_seed, fill_normal_host


@pytest.mark.parametrize("seed", [0, 1, 12345678901234567, 2 ** 63 - 5, 2 ** 64 - 1])
def test_host_library_equals_the_numpy_twin(seed):
    n = 1_000_003
    got = fill_normal_host(torch.empty(n, dtype=torch.float32), seed, 0.25, 0.02)
    ref = plain_random.fill_normal((n,), seed, 0.25, 0.02)
    assert np.array_equal(got.numpy().view(np.uint32), ref.view(np.uint32))
    # bfloat16 is the float32 value rounded to nearest even, nothing else
    got16 = fill_normal_host(torch.empty(n, dtype=torch.bfloat16), seed, 0.25, 0.02)
    assert torch.equal(got16, torch.from_numpy(ref).to(torch.bfloat16))


def test_elements_depend_on_seed_and_index_only():
    whole = plain_random.fill_normal((5000,), 99, 0.0, 1.0)
    assert np.array_equal(plain_random.fill_normal((100,), 99, 0.0, 1.0, start=1234), whole[1234:1334])
    host = fill_normal_host(torch.empty(5000, dtype=torch.float32), 99, 0.0, 1.0).numpy()
    assert np.array_equal(host, whole)
    assert not np.array_equal(plain_random.fill_normal((5000,), 98, 0.0, 1.0), whole)


def test_deviates_are_box_muller_of_the_hashed_uniforms():
    """The spelled-out logarithm, root and cosine agree with the library's to 1e-9 (the truncations are below
    2e-12), so the stream is N(0, 1) as far as 24-bit uniforms make one."""
    z = plain_random.normal_deviates(5, 0, 200_000)
    i = np.arange(200_000, dtype=np.uint64)
    h = plain_random._splitmix64(np.uint64(5) ^ plain_random._splitmix64(i))
    u = ((h >> np.uint64(40)).astype(np.float64) + 1.0) / 2.0 ** 24
    v = ((h >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.float64) / 2.0 ** 24
    ref = np.sqrt(-2.0 * np.log(u)) * np.cos(2.0 * math.pi * v)
    assert np.abs(z - ref).max() < 1e-9
    big = plain_random.normal_deviates(6, 0, 4_000_000)
    assert abs(big.mean()) < 3e-3 and abs(big.std() - 1.0) < 2e-3 and abs((big ** 4).mean() - 3.0) < 2e-2
    assert abs(np.mean(big[:-1] * big[1:])) < 3e-3, "neighbouring elements are uncorrelated"


def test_extreme_uniforms():
    """u = 1 gives exactly 0 (no negative zero under the root), the smallest u the largest radius."""
    # the formula's pieces at the ends of the range, through the same code path: find elements whose 24-bit
    # fields are extreme by scanning a stream
    i = np.arange(1 << 22, dtype=np.uint64)
    h = plain_random._splitmix64(np.uint64(3) ^ plain_random._splitmix64(i))
    a = (h >> np.uint64(40)).astype(np.int64)
    z = plain_random.normal_deviates(3, 0, 1 << 22)
    assert np.all(np.isfinite(z)) and np.abs(z).max() < math.sqrt(2 * 24 * math.log(2)) + 1e-9
    top = np.nonzero(a == a.max())[0]
    assert np.all(np.abs(z[top]) <= math.sqrt(-2 * math.log((a.max() + 1) / 2 ** 24)) + 1e-9)


def test_model_tensors_come_from_named_streams():
    cfg = LlamaConfig.from_dict(helpers.CONFIGS["A"].to_dict())
    w = random_weights(cfg, seed=7, std=0.05, norm_jitter=0.1, dtype="float32")
    name = "model.layers.1.mlp.down_proj.weight"
    key = plain_random.tensor_key(7, name)
    assert key == _tensor_seed(7, name)
    ref = plain_random.fill_normal(tuple(w[name].shape), key, 0.0, 0.05)
    assert np.array_equal(w[name].numpy(), ref)
    norm = "model.layers.0.input_layernorm.weight"
    assert np.array_equal(w[norm].numpy(), plain_random.fill_normal((cfg.hidden_size,), plain_random.tensor_key(7, norm), 1.0, 0.1))
    wb = random_weights(cfg, seed=7, std=0.05, norm_jitter=0.1, dtype="bfloat16")
    assert torch.equal(wb[name], torch.from_numpy(ref).to(torch.bfloat16))

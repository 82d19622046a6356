"""The plain implementation (tests/plain.py, whole sequences in PyTorch float64) against a second one of another
form and language (tests/native/plain_llama.cpp: token by token with a growing list of keys and values, scalar
C++ loops), and its attention scale against the library routine's default.

What these pin beside the reference's text: the order inside a layer, the two residual additions, the final norm
before the head, the attention scale 1/sqrt(head size), the llama3 frequency rule in place, grouped heads, tying and
the window, each written twice, independently, from /root/reference's formulas.  (Model code of installed packages
is no source for this build, so no library model stands in as the second implementation.)"""
import os
import struct
import subprocess

import numpy as np
import pytest
import torch

import helpers
import plain

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def second(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("native") / "plain_llama")
    subprocess.run(["g++", "-O2", "-std=c++17", "-o", exe, os.path.join(ROOT, "tests", "native", "plain_llama.cpp")], check=True)
    return exe


def _run_second(exe, cfg, W, tokens, tmp_path):
    H, L = cfg["hidden_size"], cfg["num_hidden_layers"]
    nH = cfg["num_attention_heads"]
    nKV = cfg.get("num_key_value_heads", nH)
    D = cfg.get("head_dim") or H // nH
    tied = bool(cfg.get("tie_word_embeddings", False)) or "lm_head.weight" not in W
    window = cfg.get("sliding_window") or 0
    lt = cfg.get("layer_types")
    windowed = [1 if (window and (lt is None or lt[l] == "sliding_attention")) else 0 for l in range(L)]
    rs = cfg.get("rope_scaling")
    if rs is not None and rs.get("rope_type", rs.get("type")) in (None, "default"):
        rs = None
    consts = [cfg.get("rms_norm_eps", 1e-5), cfg.get("rope_theta", 10000.0)] + \
        ([1.0, rs["factor"], rs["low_freq_factor"], rs["high_freq_factor"], float(rs["original_max_position_embeddings"])] if rs else [0.0] * 5)
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(src, "wb") as f:
        f.write(struct.pack("<11i", 0x4C4C414D, H, cfg["intermediate_size"], L, nH, nKV, D, cfg["vocab_size"], int(tied), len(tokens), int(window)))
        f.write(struct.pack(f"<{L}i", *windowed))
        f.write(struct.pack("<7d", *consts))
        f.write(struct.pack(f"<{len(tokens)}i", *tokens))
        names = ["model.embed_tokens.weight"]
        for l in range(L):
            p = f"model.layers.{l}."
            names += [p + n for n in ("input_layernorm.weight", "self_attn.q_proj.weight", "self_attn.k_proj.weight", "self_attn.v_proj.weight",
                                      "self_attn.o_proj.weight", "post_attention_layernorm.weight", "mlp.gate_proj.weight", "mlp.up_proj.weight",
                                      "mlp.down_proj.weight")]
        names.append("model.norm.weight")
        if not tied:
            names.append("lm_head.weight")
        for n in names:
            f.write(W[n].double().contiguous().numpy().astype("<f8").tobytes())
    subprocess.run([exe, src, dst], check=True, timeout=600)
    return torch.from_numpy(np.fromfile(dst, dtype="<f8").reshape(len(tokens), cfg["vocab_size"]))


@pytest.mark.parametrize("name,n", [("A", 70), ("B", 90), ("C", 60), ("D", 40), ("E", 33)])
def test_two_plain_implementations_agree(tiny_dirs, second, tmp_path, name, n):
    cfg, W = tiny_dirs.plain_model(name, "float32")
    toks = helpers.random_tokens(cfg["vocab_size"], n, seed=31)
    a = plain.forward(cfg, W, toks)
    b = _run_second(second, cfg, W, toks, tmp_path)
    assert helpers.rel_err(b, a) < 1e-11, f"{name}: the two plain implementations differ by {helpers.rel_err(b, a):.3e}"


def test_second_implementation_can_fail(tiny_dirs, second, tmp_path):
    """The comparison is not empty: with the two norm weights of a layer exchanged the second implementation is
    far from the first."""
    cfg, W = tiny_dirs.plain_model("A", "float32")
    toks = helpers.random_tokens(cfg["vocab_size"], 20, seed=32)
    a = plain.forward(cfg, W, toks)
    W2 = dict(W)
    W2["model.layers.0.input_layernorm.weight"], W2["model.layers.0.post_attention_layernorm.weight"] = \
        W["model.layers.0.post_attention_layernorm.weight"], W["model.layers.0.input_layernorm.weight"]
    assert helpers.rel_err(_run_second(second, cfg, W2, toks, tmp_path), a) > 1e-3


def test_attention_scale_is_the_library_default_in_place(tiny_dirs, monkeypatch):
    """Inside the whole model, with rotation, grouped heads and the causal mask in place: the attention of
    ``plain.forward`` replaced by torch's ``scaled_dot_product_attention`` with ITS default scale (1 / sqrt of the
    head size) and its own causal mask gives the same logits.  The replacement ignores the scale it is handed, so
    1/D, no scale or sqrt of the hidden size in ``plain.forward`` would all fail here."""
    cfg, W = tiny_dirs.plain_model("A", "float32")
    toks = helpers.random_tokens(cfg["vocab_size"], 48, seed=33)
    want = plain.forward(cfg, W, toks)

    def library_attention(q, k, v, scale, window=None, kv_offset=0, stored=None):
        assert window is None and stored is None
        T, nH, D = q.shape
        group = nH // k.shape[1]
        kk, vv = k.repeat_interleave(group, dim=1), v.repeat_interleave(group, dim=1)
        o = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1)[None], kk.transpose(0, 1)[None], vv.transpose(0, 1)[None],
                                                             is_causal=True)
        return o[0].transpose(0, 1).reshape(T, nH * D)
    monkeypatch.setattr(plain, "attention", library_attention)
    got = plain.forward(cfg, W, toks)
    assert helpers.rel_err(got, want) < 1e-12

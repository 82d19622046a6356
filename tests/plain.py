"""Plain, slow implementation of the Llama 3 forward pass, written from the
reference's formulas: whole sequences, no cache, one function per part, float64
by default.  It shares no code with the engine; the engine is graded against it.

Every function cites where in /root/reference its formula comes from.
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np
import torch


# ---- reading a model folder (own reader: no code shared with the engine) --------------
def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    with open(path, "rb") as f:
        raw = f.read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8: 8 + hlen])
    base = 8 + hlen
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        buf = raw[base + b: base + e]
        dt = info["dtype"]
        if dt == "F32":
            t = torch.from_numpy(np.frombuffer(buf, dtype="<f4").copy()).double()
        elif dt == "BF16":
            u = np.frombuffer(buf, dtype="<u2").astype(np.uint32) << 16
            t = torch.from_numpy(u.view(np.float32).copy()).double()
        elif dt == "F16":
            t = torch.from_numpy(np.frombuffer(buf, dtype="<f2").astype(np.float32)).double()
        else:
            raise ValueError(f"plain reader: dtype {dt}")
        out[name] = t.reshape(info["shape"])
    return out


def read_model_dir(model_dir: str):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


# ---- parts -----------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y_i = x_i * (1 / sqrt(mean(x^2) + eps)) * w_i; eps inside the root, added to the mean.
    /root/reference/kernels/src/ggml/ops_llama.rs:201-216"""
    mean = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    scale = 1.0 / torch.sqrt(mean + eps)
    return x * scale * w


def rope_inv_freq(head_dim: int, theta: float, scaling: Optional[dict]) -> torch.Tensor:
    """freq_d = 1 / theta^(2d/D) for d < D/2 (/root/reference/kernels/src/rope.rs:36), and the
    llama3 rule on wavelengths (/root/reference/kernels/src/rope.rs:848-881)."""
    half = head_dim // 2
    out = []
    for d in range(half):
        freq = 1.0 / (theta ** (2.0 * d / head_dim))
        if scaling is not None:
            factor = scaling["factor"]
            orig = float(scaling["original_max_position_embeddings"])
            low_ff = scaling["low_freq_factor"]
            high_ff = scaling["high_freq_factor"]
            wavelen = 2.0 * math.pi / freq
            low_freq_wavelen = orig / low_ff
            high_freq_wavelen = orig / high_ff
            if wavelen < high_freq_wavelen:
                pass
            elif wavelen > low_freq_wavelen:
                freq = freq / factor
            else:
                smooth = (orig / wavelen - low_ff) / (high_ff - low_ff)
                freq = freq / factor * (1.0 - smooth) + freq * smooth
        out.append(freq)
    return torch.tensor(out, dtype=torch.float64)


def rope(x: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, attn_factor: float = 1.0) -> torch.Tensor:
    """x [T, heads, D]; split-half pairs (d, d + D/2):
    x[d]' = x0 cos - x1 sin; x[d+D/2]' = x0 sin + x1 cos, angle = pos * inv_freq[d].
    /root/reference/kernels/src/rope.rs:18-53 and 900-921"""
    half = x.shape[-1] // 2
    ang = positions.to(torch.float64)[:, None] * inv_freq[None, :]          # [T, half]
    c = (torch.cos(ang) * attn_factor)[:, None, :]
    s = (torch.sin(ang) * attn_factor)[:, None, :]
    x0, x1 = x[..., :half], x[..., half:]
    return torch.cat([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1)


def as_bfloat16(x: torch.Tensor) -> torch.Tensor:
    """x rounded to bfloat16 (nearest, ties to even) and widened again: what storing it in 16 bits does."""
    return x.to(torch.float32).to(torch.bfloat16).to(x.dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int] = None,
              kv_offset: int = 0, stored=None) -> torch.Tensor:
    """q [T, nH, D], k, v [S, nKV, D] with S = kv_offset + T; kv head of head h is
    h // (nH / nKV); query row s sees keys j <= (S - T) + s and, with a window w, j >= limit - w + 1;
    score = dot * scale; softmax over the visible keys; out = sum p_j v_j.
    /root/reference/kernels/src/attention.rs:28-87
    ``stored``: see ``forward``; here it rounds the unnormalised probabilities that are multiplied with the
    values (their sum is taken before the rounding)."""
    T, nH, D = q.shape
    S, nKV, _ = k.shape
    group = nH // nKV
    out = torch.zeros(T, nH, D, dtype=q.dtype)
    for h in range(nH):
        kv_h = h // group
        for s in range(T):
            limit = (S - T) + s
            start = 0
            if window is not None and limit >= window:
                start = limit - window + 1
            scores = (k[start: limit + 1, kv_h] @ q[s, h]) * scale
            p = torch.exp(scores - scores.max())
            if stored is None:
                p = p / p.sum()
                out[s, h] = p @ v[start: limit + 1, kv_h]
            else:
                out[s, h] = (stored(p) @ v[start: limit + 1, kv_h]) / p.sum()
    return out.reshape(T, nH * D)


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)).  /root/reference/kernels/src/ggml/vec_llama.rs:808-810"""
    return x / (1.0 + torch.exp(-x))


def swiglu_ffn(x: torch.Tensor, wg: torch.Tensor, wu: torch.Tensor, wd: torch.Tensor, stored=None) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)), weights [out, in], y = x W^T.
    /root/reference/engine/src/model.rs:1203-1231,1301-1313"""
    a = silu(x @ wg.T) * (x @ wu.T)
    if stored is not None:
        a = stored(a)
    return a @ wd.T


# ---- whole model --------------------------------------------------------------------------
def layer_window(cfg: dict, layer: int) -> Optional[int]:
    w = cfg.get("sliding_window")
    if w is None:
        return None
    lt = cfg.get("layer_types")
    if lt is None or lt[layer] == "sliding_attention":
        return int(w)
    return None


def decoder_layer(cfg: dict, get, l: int, h: torch.Tensor, pos: torch.Tensor, inv_freq: torch.Tensor, stored=None) -> torch.Tensor:
    """One layer on the residual stream h [T, hidden] of one whole sequence: norm, q/k/v, rope on q and k,
    attention, o, add, norm, feed-forward, add (/root/reference/engine/src/model.rs:952-1314).
    ``get(name)`` returns the layer's tensors by checkpoint name."""
    keep = stored if stored is not None else (lambda t: t)
    H = cfg["hidden_size"]
    nH = cfg["num_attention_heads"]
    nKV = cfg.get("num_key_value_heads", nH)
    D = cfg.get("head_dim") or H // nH
    eps = cfg.get("rms_norm_eps", 1e-5)
    T = h.shape[0]
    scale = 1.0 / math.sqrt(D)                                          # model.rs:1078
    p = f"model.layers.{l}."
    x = keep(rmsnorm(h, get(p + "input_layernorm.weight"), eps))
    q = (x @ get(p + "self_attn.q_proj.weight").T).reshape(T, nH, D)
    k = (x @ get(p + "self_attn.k_proj.weight").T).reshape(T, nKV, D)
    v = keep((x @ get(p + "self_attn.v_proj.weight").T).reshape(T, nKV, D))
    q = keep(rope(q, pos, inv_freq))
    k = keep(rope(k, pos, inv_freq))
    a = keep(attention(q, k, v, scale, layer_window(cfg, l), stored=stored))
    h = h + a @ get(p + "self_attn.o_proj.weight").T
    x = keep(rmsnorm(h, get(p + "post_attention_layernorm.weight"), eps))
    return h + swiglu_ffn(x, get(p + "mlp.gate_proj.weight"), get(p + "mlp.up_proj.weight"), get(p + "mlp.down_proj.weight"), stored)


def forward(cfg: dict, weights, tokens: List[int], dtype=torch.float64,
            position_offset: int = 0, stored=None) -> torch.Tensor:
    """Logits [T, vocab] at every position of one whole sequence, no cache.
    ``weights``: tensors by checkpoint name, or a function name -> tensor (or None for a tensor the checkpoint
    does not hold) that is asked for each tensor when it is needed, so that a large model can be streamed layer
    by layer.
    ``position_offset`` shifts every position (positions are session.position + t,
    /root/reference/engine/src/model.rs:686-688); only distances count, so logits must not change.
    Layers in order (``decoder_layer``), then final norm and output projection
    (model.rs:1355-1398), the output matrix being the embedding when the file has none
    (/root/reference/engine/src/weights.rs:156-166).
    ``stored`` (for instance ``as_bfloat16``) is applied to every value that 16-bit serving keeps in 16 bits
    between two operations: the normed rows fed to a product, q, k and v, the unnormalised probabilities, the
    attention output and the gated activations; everything else (sums, norms, softmax statistics, the residual
    stream) stays exact.  The distance of such a run from the exact one is the rounding noise that the storage
    type alone explains, the yardstick the 16-bit engine is measured with."""
    return forward_many(cfg, weights, [tokens], [stored], dtype, position_offset)[0][0]


def forward_many(cfg: dict, weights, sequences, stored_variants=(None,), dtype=torch.float64, position_offset: int = 0):
    """``forward`` for several sequences and several ``stored`` variants at once: result[i][j] is the logits of
    sequence i under variant j.  Every tensor is fetched once per layer and used for all of them, so a model
    whose weights are streamed (``weights`` a function) is read once."""
    if callable(weights):
        fetch = weights
    else:
        fetch = weights.get

    def get(name):
        t = fetch(name)
        return None if t is None else t.to(dtype)
    H = cfg["hidden_size"]
    nH = cfg["num_attention_heads"]
    D = cfg.get("head_dim") or H // nH
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg.get("rope_theta", 10000.0)
    rs = cfg.get("rope_scaling")
    if rs is not None and rs.get("rope_type", rs.get("type")) in (None, "default"):
        rs = None
    inv_freq = rope_inv_freq(D, theta, rs)
    embed = get("model.embed_tokens.weight")
    hs = [[embed[torch.tensor(tokens)] for _ in stored_variants] for tokens in sequences]    # model.rs:672-684, no scaling
    pos = [torch.arange(len(tokens)) + position_offset for tokens in sequences]
    for l in range(cfg["num_hidden_layers"]):
        held = {}

        def layer_get(name):
            if name not in held:
                held[name] = get(name)
            return held[name]
        for i in range(len(sequences)):
            for j, stored in enumerate(stored_variants):
                hs[i][j] = decoder_layer(cfg, layer_get, l, hs[i][j], pos[i], inv_freq, stored)
    norm_w = get("model.norm.weight")
    lm = None if cfg.get("tie_word_embeddings", False) else get("lm_head.weight")
    if lm is None:
        lm = embed
    out = []
    for i in range(len(sequences)):
        row = []
        for j, stored in enumerate(stored_variants):
            x = rmsnorm(hs[i][j], norm_w, eps)
            row.append((stored(x) if stored is not None else x) @ lm.T)
        out.append(row)
    return out


def greedy_generate(cfg: dict, weights: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """Greedy continuation: argmax of the last position's logits, the last maximum winning on ties
    (/root/reference/engine/src/model.rs:459-473,9693-9815); the whole sequence is recomputed each step."""
    seq = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, weights, seq)[-1]
        mx = logits.max()
        tok = int(torch.nonzero(logits == mx).max())
        out.append(tok)
        seq.append(tok)
    return out

"""``tempura inspect``: what a model folder holds, without loading it onto a device.

Prints the fields the reference's inspect prints (format, architecture, hidden size, layers,
heads with KV heads, vocabulary, tensors, size; /root/reference/model/src/inspect.rs:84-135,160-198)
plus head size, feed-forward width, rotary settings, eps, tying, dtype, parameter count and cache
bytes per token.
"""
from __future__ import annotations

import glob
import os
from typing import Any, Dict

from .config import load_config
from .weights.safetensors_io import SafetensorsFile


def inspect(model_dir: str) -> Dict[str, Any]:
    cfg = load_config(model_dir)
    files = sorted(glob.glob(os.path.join(model_dir, "*.safetensors")))
    n_tensors, size, dtypes = 0, 0, set()
    for p in files:
        f = SafetensorsFile(p)
        n_tensors += len(f.names())
        dtypes.update(f.dtype_tag(n) for n in f.names())
        size += os.path.getsize(p)
        f.close()
    rs = cfg.rope_scaling
    return {
        "format": "safetensors" if files else "none",
        "architecture": cfg.architecture,
        "hidden_size": cfg.hidden_size,
        "layers": cfg.num_hidden_layers,
        "attention_heads": cfg.num_attention_heads,
        "kv_heads": cfg.num_key_value_heads,
        "head_dim": cfg.head_dim,
        "intermediate_size": cfg.intermediate_size,
        "vocab_size": cfg.vocab_size,
        "max_position_embeddings": cfg.max_position_embeddings,
        "rope_theta": cfg.rope_theta,
        "rope_scaling": None if rs is None else f"{rs.rope_type} factor {rs.factor} low {rs.low_freq_factor} "
                                                 f"high {rs.high_freq_factor} original {rs.original_max_position_embeddings}",
        "rms_norm_eps": cfg.rms_norm_eps,
        "sliding_window": cfg.sliding_window,
        "tied_embeddings": cfg.tie_word_embeddings,
        "dtypes": sorted(dtypes),
        "tensors": n_tensors,
        "size_bytes": size,
        "parameters": cfg.num_parameters(),
        "kv_bytes_per_token_bf16": cfg.kv_bytes_per_token(2),
    }


def format_report(info: Dict[str, Any]) -> str:
    gqa = "MHA" if info["kv_heads"] == info["attention_heads"] else ("MQA" if info["kv_heads"] == 1 else "GQA")
    lines = [
        f"Format:          {info['format']}",
        f"Architecture:    {info['architecture']}",
        f"Hidden size:     {info['hidden_size']}",
        f"Layers:          {info['layers']}",
        f"Attention heads: {info['attention_heads']} ({info['kv_heads']} KV heads, {gqa}), head size {info['head_dim']}",
        f"Feed-forward:    {info['intermediate_size']}",
        f"Vocab size:      {info['vocab_size']}",
        f"Max positions:   {info['max_position_embeddings']}",
        f"Rotary:          theta {info['rope_theta']:g}, scaling {info['rope_scaling'] or 'none'}",
        f"Norm eps:        {info['rms_norm_eps']:g}",
        f"Window:          {info['sliding_window'] or 'none'}",
        f"Tied embeddings: {'yes' if info['tied_embeddings'] else 'no'}",
        f"Stored dtypes:   {', '.join(info['dtypes']) or '-'}",
        f"Tensors:         {info['tensors']}",
        f"Size:            {info['size_bytes'] / 1e6:.1f} MB",
        f"Parameters:      {info['parameters'] / 1e6:.2f} M",
        f"Cache per token: {info['kv_bytes_per_token_bf16'] / 1024:.1f} KiB (bfloat16)",
    ]
    return "\n".join(lines)

"""Typed configuration of the Llama 3 architecture, read from config.json keys.

Key names, required keys and defaults follow the reference's parser
(/root/reference/engine/src/config.rs:390-497): ``hidden_size``,
``num_attention_heads``, ``num_hidden_layers``, ``intermediate_size`` and
``vocab_size`` are required; ``num_key_value_heads`` defaults to the head count,
``head_dim`` to hidden/heads, ``max_position_embeddings`` to 4096,
``rope_theta`` to 10000, ``rms_norm_eps`` (fallback key ``layer_norm_eps``) to
1e-5, and ``sliding_window`` is honoured when present (config.rs:514-517).
The reference reads ``rope_scaling["type"]`` only (config.rs:466); released
Llama 3.1 files say ``"rope_type"``, so both keys are accepted here.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field, asdict
from typing import Any, Dict, List, Optional

from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec


class ConfigError(ValueError):
    """A config.json that cannot be used: missing key, bad value, bad JSON."""


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of kind llama3 (/root/reference/kernels/src/rope.rs:848-881)."""

    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


_REQUIRED = ("hidden_size", "num_attention_heads", "num_hidden_layers", "intermediate_size", "vocab_size")


def _as_int(d: Dict[str, Any], key: str, default=None) -> int:
    v = d.get(key, default)
    if v is None:
        raise ConfigError(f"config.json: missing field '{key}'")
    if isinstance(v, bool) or not isinstance(v, (int, float)) or int(v) != v:
        raise ConfigError(f"config.json: field '{key}' must be an integer, got {v!r}")
    return int(v)


def _as_float(d: Dict[str, Any], key: str, default: float) -> float:
    v = d.get(key)
    if v is None:
        return float(default)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: field '{key}' must be a number, got {v!r}")
    return float(v)


@dataclass
class LlamaConfig:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int = 4096
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    sliding_window: Optional[int] = None
    layer_types: Optional[List[str]] = None
    torch_dtype: str = "bfloat16"
    bos_token_id: Optional[int] = None
    eos_token_id: List[int] = field(default_factory=list)
    architecture: str = "LlamaForCausalLM"

    # ---- reading -------------------------------------------------------
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        for k in _REQUIRED:
            if d.get(k) is None:
                raise ConfigError(f"config.json: missing field '{k}'")
        hidden = _as_int(d, "hidden_size")
        heads = _as_int(d, "num_attention_heads")
        if heads <= 0:
            raise ConfigError("config.json: num_attention_heads must be positive")
        kv = _as_int(d, "num_key_value_heads", heads)
        head_dim = _as_int(d, "head_dim", hidden // heads)
        eps_key = "rms_norm_eps" if d.get("rms_norm_eps") is not None else "layer_norm_eps"
        eps = _as_float(d, eps_key, 1e-5)

        act = d.get("hidden_act")
        if act not in (None, "silu", "swish"):
            raise ConfigError(f"config.json: hidden_act {act!r} is not Llama's gated SiLU")
        for bias_key in ("attention_bias", "mlp_bias"):
            if d.get(bias_key):
                raise ConfigError(f"config.json: {bias_key}=true is not supported (Llama 3 has no biases)")

        rs = d.get("rope_scaling")
        scaling = None
        if rs is not None:
            if not isinstance(rs, dict):
                raise ConfigError("config.json: rope_scaling must be an object")
            kind = rs.get("rope_type", rs.get("type"))
            if kind in (None, "default"):
                scaling = None
            elif kind == "llama3":
                max_pos_default = _as_int(d, "max_position_embeddings", 4096)
                scaling = RopeScaling(
                    rope_type="llama3",
                    factor=_as_float(rs, "factor", 1.0),
                    low_freq_factor=_as_float(rs, "low_freq_factor", 1.0),
                    high_freq_factor=_as_float(rs, "high_freq_factor", 4.0),
                    original_max_position_embeddings=_as_int(
                        rs, "original_max_position_embeddings", max_pos_default),
                )
            else:
                raise ConfigError(f"config.json: rope_scaling type {kind!r} is not supported (only 'llama3')")

        eos = d.get("eos_token_id")
        if eos is None:
            eos_list: List[int] = []
        elif isinstance(eos, list):
            eos_list = [int(e) for e in eos]
        else:
            eos_list = [int(eos)]

        window = d.get("sliding_window")
        if window is not None:
            window = _as_int(d, "sliding_window")
        layer_types = d.get("layer_types")
        if layer_types is not None:
            layer_types = [str(t) for t in layer_types]

        archs = d.get("architectures")
        arch = archs[0] if isinstance(archs, list) and archs else d.get("model_type", "llama")

        cfg = cls(
            hidden_size=hidden,
            intermediate_size=_as_int(d, "intermediate_size"),
            num_hidden_layers=_as_int(d, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=kv,
            head_dim=head_dim,
            vocab_size=_as_int(d, "vocab_size"),
            max_position_embeddings=_as_int(d, "max_position_embeddings", 4096),
            rms_norm_eps=eps,
            rope_theta=_as_float(d, "rope_theta", 10000.0),
            rope_scaling=scaling,
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            sliding_window=window,
            layer_types=layer_types,
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))),
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=eos_list,
            architecture=str(arch),
        )
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, text: str) -> "LlamaConfig":
        try:
            d = json.loads(text)
        except json.JSONDecodeError as e:
            raise ConfigError(f"config.json: malformed JSON: {e}") from e
        if not isinstance(d, dict):
            raise ConfigError("config.json: top level must be an object")
        return cls.from_dict(d)

    @classmethod
    def from_dir(cls, model_dir: str) -> "LlamaConfig":
        path = os.path.join(model_dir, "config.json")
        try:
            with open(path, "r") as f:
                text = f.read()
        except OSError as e:
            raise ConfigError(f"cannot read {path}: {e}") from e
        return cls.from_json(text)

    # ---- checks --------------------------------------------------------
    def validate(self) -> None:
        pos = ("hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
               "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings")
        for k in pos:
            if getattr(self, k) <= 0:
                raise ConfigError(f"config.json: {k} must be positive, got {getattr(self, k)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config.json: num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim ({self.head_dim}) must be even for rotary pairs")
        if not (self.rms_norm_eps > 0):
            raise ConfigError("config.json: rms_norm_eps must be positive")
        if not (self.rope_theta > 0):
            raise ConfigError("config.json: rope_theta must be positive")
        if self.sliding_window is not None and self.sliding_window <= 0:
            raise ConfigError("config.json: sliding_window must be positive when given")
        if self.layer_types is not None:
            if len(self.layer_types) != self.num_hidden_layers:
                raise ConfigError("config.json: layer_types must have one entry per layer")
            for t in self.layer_types:
                if t not in ("full_attention", "sliding_attention"):
                    raise ConfigError(f"config.json: layer type {t!r} unknown")
                if t == "sliding_attention" and self.sliding_window is None:
                    raise ConfigError("config.json: sliding_attention layer needs sliding_window")
        rs = self.rope_scaling
        if rs is not None:
            if rs.factor <= 0 or rs.original_max_position_embeddings <= 0:
                raise ConfigError("config.json: rope_scaling factor and original length must be positive")
            if rs.high_freq_factor == rs.low_freq_factor:
                raise ConfigError("config.json: rope_scaling high_freq_factor must differ from low_freq_factor")

    # ---- writing -------------------------------------------------------
    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None if self.rope_scaling is None else asdict(self.rope_scaling),
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
            "torch_dtype": self.torch_dtype,
        }
        if self.sliding_window is not None:
            d["sliding_window"] = self.sliding_window
        if self.layer_types is not None:
            d["layer_types"] = list(self.layer_types)
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_id:
            d["eos_token_id"] = self.eos_token_id if len(self.eos_token_id) > 1 else self.eos_token_id[0]
        return d

    def to_json(self) -> str:
        return json.dumps(self.to_dict(), indent=2)

    # ---- derived -------------------------------------------------------
    def layer_window(self, layer: int) -> Optional[int]:
        """The attention window of a layer, or None when it sees every key."""
        if self.sliding_window is None:
            return None
        if self.layer_types is None:
            return self.sliding_window
        return self.sliding_window if self.layer_types[layer] == "sliding_attention" else None

    def num_parameters(self) -> int:
        h, i, v = self.hidden_size, self.intermediate_size, self.vocab_size
        q = self.num_attention_heads * self.head_dim
        kv = self.num_key_value_heads * self.head_dim
        per_layer = h * q + 2 * h * kv + q * h + 3 * h * i + 2 * h
        return self.num_hidden_layers * per_layer + v * h * (1 if self.tie_word_embeddings else 2) + h

    def kv_bytes_per_token(self, elem_bytes: int = 2) -> int:
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * elem_bytes

    def build_spec(self) -> ModelSpec:
        """Describe this model to the engine.

        Tensor names are the ones the reference requires
        (/root/reference/engine/src/weights.rs:205-228): three global tensors and
        nine per layer.  A layer is [pre-norm attention, pre-norm feed-forward]
        (/root/reference/engine/src/architecture.rs:56-65).
        """
        rope_params: Dict[str, Any] = {
            "head_dim": self.head_dim,
            "theta": self.rope_theta,
            "scaling": None if self.rope_scaling is None else asdict(self.rope_scaling),
        }
        layers = []
        for l in range(self.num_hidden_layers):
            p = f"model.layers.{l}"
            mixer = PartSpec(
                "attention",
                params={
                    "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads,
                    "head_dim": self.head_dim,
                    "scale": float(self.head_dim) ** -0.5,
                    "window": self.layer_window(l),
                    "position": PartSpec("rope", params=rope_params),
                },
                weights={
                    "q": f"{p}.self_attn.q_proj.weight",
                    "k": f"{p}.self_attn.k_proj.weight",
                    "v": f"{p}.self_attn.v_proj.weight",
                    "o": f"{p}.self_attn.o_proj.weight",
                },
            )
            ffn = PartSpec(
                "swiglu",
                params={"intermediate_size": self.intermediate_size},
                weights={
                    "gate": f"{p}.mlp.gate_proj.weight",
                    "up": f"{p}.mlp.up_proj.weight",
                    "down": f"{p}.mlp.down_proj.weight",
                },
            )
            layers.append(LayerSpec("prenorm", {
                "mixer_norm": PartSpec("rmsnorm", {"eps": self.rms_norm_eps}, {"weight": f"{p}.input_layernorm.weight"}),
                "mixer": mixer,
                "ffn_norm": PartSpec("rmsnorm", {"eps": self.rms_norm_eps}, {"weight": f"{p}.post_attention_layernorm.weight"}),
                "ffn": ffn,
            }))
        embed_name = "model.embed_tokens.weight"
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            layers=layers,
            order=[LayerCall(l) for l in range(self.num_hidden_layers)],
            final_norm=PartSpec("rmsnorm", {"eps": self.rms_norm_eps}, {"weight": "model.norm.weight"}),
            embedding=PartSpec("embedding", {}, {"weight": embed_name}),
            lm_head=PartSpec("lm_head", {"tied": self.tie_word_embeddings, "tied_to": embed_name},
                             {"weight": "lm_head.weight"}),
            eos_token_ids=list(self.eos_token_id),
            bos_token_id=self.bos_token_id,
        )


def _llama3_scaling(factor: float, orig: int) -> RopeScaling:
    return RopeScaling("llama3", factor, 1.0, 4.0, orig)


#: Named sizes for random-weight runs (the reference selects presets with
#: ``--model-config``, /root/reference/server/src/lib.rs:59-64).
PRESETS: Dict[str, LlamaConfig] = {
    "tiny-a": LlamaConfig(64, 192, 2, 4, 2, 16, 256, 128, 1e-5, 10000.0, None, False),
    "tiny-b": LlamaConfig(96, 320, 3, 8, 1, 12, 384, 256, 1e-6, 500000.0, _llama3_scaling(8.0, 64), True),
    "llama-3.1-8b": LlamaConfig(4096, 14336, 32, 32, 8, 128, 128256, 131072, 1e-5, 500000.0,
                                _llama3_scaling(8.0, 8192), False),
    "llama-3.2-3b": LlamaConfig(3072, 8192, 28, 24, 8, 128, 128256, 131072, 1e-5, 500000.0,
                                _llama3_scaling(32.0, 8192), True),
    "llama-3.1-70b": LlamaConfig(8192, 28672, 80, 64, 8, 128, 128256, 131072, 1e-5, 500000.0,
                                 _llama3_scaling(8.0, 8192), False),
}
